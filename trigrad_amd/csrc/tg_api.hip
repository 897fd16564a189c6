// tg_api.hip -- version, error reporting, per-kernel timing; helpers shared by every entry point.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

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

// ---- per-kernel timing ---------------------------------------------------------
struct ProfileRecord {
    const char *name;
    int launches;
    hipEvent_t start, stop;
};
static bool g_profile_on = false;
static std::mutex g_profile_mutex;
static std::vector<ProfileRecord> g_profile_records;

ProfileScope::ProfileScope(const char *name, hipStream_t s, int launches) : slot(-1), stream(s) {
    if (!g_profile_on) return;
    ProfileRecord r;
    r.name = name;
    r.launches = launches;
    if (hipEventCreate(&r.start) != hipSuccess) return;
    if (hipEventCreate(&r.stop) != hipSuccess) { (void)hipEventDestroy(r.start); return; }
    (void)hipEventRecord(r.start, s);
    std::lock_guard<std::mutex> lock(g_profile_mutex);
    slot = (int)g_profile_records.size();
    g_profile_records.push_back(r);
}

ProfileScope::~ProfileScope() {
    if (slot < 0) return;
    std::lock_guard<std::mutex> lock(g_profile_mutex);
    if (slot < (int)g_profile_records.size()) (void)hipEventRecord(g_profile_records[slot].stop, stream);
}

static bool g_force_tickets = false;

int resident_workgroups(const void *kernel, int threads, int *cache, size_t dynamic_lds) {
    if (g_force_tickets) return 0;  // "unknown": the callers then number their tiles by ticket
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    if (cache[dev] == 0) {
        int per_cu = 0;
        hipDeviceProp_t prop;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, dynamic_lds) != hipSuccess ||
            hipGetDeviceProperties(&prop, dev) != hipSuccess) {
            (void)hipGetLastError();
            cache[dev] = -1;
        } else {
            cache[dev] = per_cu * prop.multiProcessorCount > 0 ? per_cu * prop.multiProcessorCount : -1;
        }
    }
    return cache[dev] > 0 ? cache[dev] : 0;
}

int reserve_lds(const char *fn, const void *kernel, size_t bytes, size_t *reserved) {
    if (bytes <= 64 * 1024) return 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        set_error("%s: no current device", fn);
        return (int)hipErrorInvalidDevice;
    }
    if (bytes <= reserved[dev]) return 0;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("%s: cannot reserve %zu bytes of LDS per workgroup: %s", fn, bytes, hipGetErrorString(e));
        return (int)e;
    }
    reserved[dev] = bytes;
    return 0;
}

}  // namespace tg

extern "C" int tg_version(void) { return TG_ABI_VERSION; }

extern "C" int tg_precision_bits(void) { return (int)(8 * sizeof(tg_real)); }

extern "C" const char *tg_last_error(void) { return tg::g_error; }

extern "C" int tg_num_tiles(int width, int height, int tile_w, int tile_h) {
    if (width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0) return 0;
    return tg::ceil_div(width, tile_w) * tg::ceil_div(height, tile_h);
}

extern "C" void tg_profile_enable(int on) { tg::g_profile_on = on != 0; }

extern "C" void tg_force_tickets(int on) { tg::g_force_tickets = on != 0; }

extern "C" int tg_profile_report(char *buffer, size_t capacity) {
    using namespace tg;
    std::vector<ProfileRecord> records;
    {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        records.swap(g_profile_records);
    }
    struct Sum { long count = 0; double ms = 0.0; };
    std::map<std::string, Sum> sums;
    for (const ProfileRecord &r : records) {
        float ms = 0.0f;
        if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            Sum &s = sums[r.name];
            s.count += r.launches;
            s.ms += ms;
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    std::string text;
    char line[256];
    for (const auto &kv : sums) {
        snprintf(line, sizeof(line), "%s %ld %.6f\n", kv.first.c_str(), kv.second.count, kv.second.ms);
        text += line;
    }
    if (!buffer || capacity == 0) return (int)text.size();
    const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
    memcpy(buffer, text.data(), n);
    buffer[n] = '\0';
    return (int)text.size();
}
