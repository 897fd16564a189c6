// tg_api.hip -- version, error reporting and helpers shared by every entry point.
#include <cstdarg>
#include <cstdio>

#include "tg_common.hpp"

namespace tg {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

}  // namespace tg

extern "C" int tg_version(void) { return TG_ABI_VERSION; }

extern "C" const char *tg_last_error(void) { return tg::g_error; }

extern "C" int tg_num_tiles(int width, int height, int tile_w, int tile_h) {
    if (width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0) return 0;
    return tg::ceil_div(width, tile_w) * tg::ceil_div(height, tile_h);
}
