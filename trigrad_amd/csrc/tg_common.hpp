// tg_common.hpp -- shared host helpers and device arithmetic for the gfx950 kernels.
//
// Arithmetic contract: every expression below that feeds a classification
// (tile bounds, depth key, inside test, per-pixel depth, transmittance) is
// evaluated exactly as the reference source writes it, one IEEE-754 operation
// per source operator, no fused multiply-add.  The library must therefore be
// compiled with -ffp-contract=off; floating-point division is hipcc's correctly rounded
// default.  Reference lines are relative to src/trigrad/ of the reference tree.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <cfloat>
#include <limits>

#include "../../include/trigrad_hip.h"

namespace tg {

// The scalar type of the build (util.h:5-20): float, or double when the library
// is compiled with -DTG_DOUBLE_PRECISION (the reference's DOUBLE_PRECISION).
#ifdef TG_DOUBLE_PRECISION
using real = double;
using real4 = double4;
#else
using real = float;
using real4 = float4;
#endif
static_assert(sizeof(real) == sizeof(tg_real), "the header's tg_real is the kernels' scalar type");
__host__ __device__ __forceinline__ real4 make_real4(real x, real y, real z, real w) {
    real4 v;
    v.x = x; v.y = y; v.z = z; v.w = w;
    return v;
}

constexpr real kEffZero = std::numeric_limits<real>::min();  // util.h:24
constexpr real kMaxOpacity = (real)0.9999;                    // util.h:22
constexpr real kFarKey = (real)1e30;                          // render.cu:259
constexpr int kWave = 64;

// ---- host side ---------------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);

// Per-kernel timing (the counterpart of the reference's CudaTimer,
// render.cu:11-49): when enabled through tg_profile_enable, every launch is
// bracketed by a pair of events on its stream; tg_profile_report waits for
// them and sums the elapsed time per kernel name.
struct ProfileScope {
    ProfileScope(const char *name, hipStream_t stream, int launches = 1);  // launches: kernels of that name inside the pair
    ~ProfileScope();
    int slot;
    hipStream_t stream;
};
#define TG_LAUNCH_AS(name, kernel, grid, block, lds, stream, ...)       \
    do {                                                               \
        tg::ProfileScope tg_profile_scope(name, stream);               \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__); \
    } while (0)
#define TG_LAUNCH(kernel, grid, block, lds, stream, ...) TG_LAUNCH_AS(#kernel, kernel, grid, block, lds, stream, __VA_ARGS__)

// Workgroups of `kernel` that can be resident on the current device at once
// (0 if unknown).  A grid that is no larger needs no ticket to number its
// workgroups for a look-back chain: every workgroup is started without waiting
// for another to finish, so waiting on lower-numbered ones cannot deadlock.
int resident_workgroups(const void *kernel, int threads, int *cache /* [kMaxDevices] */, size_t dynamic_lds = 0);
constexpr int kMaxDevices = 64;
// Dynamic LDS beyond 64 KB has to be enabled per kernel and device once; `reserved` ([kMaxDevices], zero at
// first) remembers per device what the kernel has been given.
int reserve_lds(const char *fn, const void *kernel, size_t bytes, size_t *reserved);

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device arithmetic ---------------------------------------------------------
struct Rect { int x0, y0, x1, y1; };  // y0 == -1: the triangle touches no tile

__device__ __forceinline__ real min3(real a, real b, real c) {
    real m = a;
    m = (b < m) ? b : m;
    m = (c < m) ? c : m;
    return m;
}
__device__ __forceinline__ real max3(real a, real b, real c) {
    real m = a;
    m = (m < b) ? b : m;
    m = (m < c) ? c : m;
    return m;
}
__host__ __device__ __forceinline__ real abs_real(real v) { return v < (real)0 ? -v : v; }
__device__ __forceinline__ real clampf(real v, real lo, real hi) { return (v < lo) ? lo : ((hi < v) ? hi : v); }

// Tile coordinate of an NDC coordinate (render.cu:72-75).  The 0.5 literal of
// the source makes the product and quotient double precision.
__device__ __forceinline__ int tile_coord(real m, int extent, int tile, int ntiles) {
    real m1 = m + 1.0f;
    const double scaled = ((double)m1 * 0.5) * (double)extent;
    // dividing by a power of two is an exact scaling, so the reciprocal gives the same double
    const double t = ((tile & (tile - 1)) == 0) ? scaled * (1.0 / (double)tile) : scaled / (double)tile;
    return (int)clampf((real)t, 0.0f, (real)(ntiles - 1));
}

// render.cu:51-76 touched_tiles.
__device__ __forceinline__ Rect tile_rect(real ax, real ay, real bx, real by, real cx, real cy, int W, int H, int tw,
                                          int th, int tiles_x, int tiles_y) {
    real ux = bx - ax, uy = by - ay, vx = cx - ax, vy = cy - ay;
    real area2 = ux * vy - uy * vx;
    Rect r;
    if (abs_real(area2) < kEffZero || isnan(area2) || isinf(area2)) {
        r.x0 = 0; r.y0 = -1; r.x1 = 0; r.y1 = -1;
        return r;
    }
    r.x0 = tile_coord(min3(ax, bx, cx), W, tw, tiles_x);
    r.y0 = tile_coord(min3(ay, by, cy), H, th, tiles_y);
    r.x1 = tile_coord(max3(ax, bx, cx), W, tw, tiles_x);
    r.y1 = tile_coord(max3(ay, by, cy), H, th, tiles_y);
    return r;
}
__device__ __forceinline__ uint32_t rect_count(const Rect &r) {
    return (r.y0 == -1) ? 0u : (uint32_t)(r.x1 - r.x0 + 1) * (uint32_t)(r.y1 - r.y0 + 1);
}

// Order-preserving map of a floating-point value to an unsigned integer of the
// same width (ascending values give ascending integers).
__device__ __forceinline__ uint32_t orderable_bits(float f) {
    uint32_t b = __float_as_uint(f);
    return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ uint64_t orderable_bits(double f) {
    uint64_t b = (uint64_t)__double_as_longlong(f);
    return b ^ ((b >> 63) ? ~0ull : (1ull << 63));
}

// An int carried in a slot of the scalar type, bit for bit.
__device__ __forceinline__ float int_in_real(int v, float) { return __int_as_float(v); }
__device__ __forceinline__ double int_in_real(int v, double) { return __longlong_as_double((long long)v); }
__device__ __forceinline__ real int_in_real(int v) { return int_in_real(v, real()); }
__device__ __forceinline__ int int_of_real(float v) { return __float_as_int(v); }
__device__ __forceinline__ int int_of_real(double v) { return (int)__double_as_longlong(v); }

// render.cu:78-88: bary = M * (x, y, 1).
__device__ __forceinline__ void bary_apply(const real m[9], real px, real py, real &b0, real &b1, real &b2) {
    b0 = m[0] * px + m[1] * py + m[2];
    b1 = m[3] * px + m[4] * py + m[5];
    b2 = m[6] * px + m[7] * py + m[8];
}
// Strictly inside: all three at least FLT_MIN (render.cu:401, 438, 482).
__device__ __forceinline__ bool bary_inside(real b0, real b1, real b2) {
    return !(b0 < kEffZero || b1 < kEffZero || b2 < kEffZero);
}
// util.h:245-250 interpolate3 with per-vertex weights.
__device__ __forceinline__ real interp_w(real b0, real b1, real b2, real a, real b, real c, real w0, real w1, real w2) {
    real denom = b0 * w0 + b1 * w1 + b2 * w2;
    return (b0 * a * w0 + b1 * b * w1 + b2 * c * w2) / denom;
}
// Same with unit weights (multiplication by 1.0f is exact, so it is omitted).
__device__ __forceinline__ real interp_1(real b0, real b1, real b2, real a, real b, real c) {
    real denom = b0 + b1 + b2;
    return (b0 * a + b1 * b + b2 * c) / denom;
}
// Pixel centre in NDC: double expression rounded once (render.cu:561-562).
__device__ __forceinline__ real pixel_ndc(int i, int extent) {
    return (real)(((double)(real)i + 0.5) / (double)(real)extent * 2.0 - 1.0);
}

// ---- wave64 DPP scan -----------------------------------------------------------
template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_add_u32(uint32_t v) {
    // lanes whose source is out of range (or whose row is masked off) receive 0
    return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, 0xf, false);
}
// Inclusive prefix sum over the 64 lanes of a wave (all lanes must be active).
__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v) {
    v = dpp_add_u32<0x111, 0xf>(v);  // row_shr:1
    v = dpp_add_u32<0x112, 0xf>(v);  // row_shr:2
    v = dpp_add_u32<0x114, 0xf>(v);  // row_shr:4
    v = dpp_add_u32<0x118, 0xf>(v);  // row_shr:8
    v = dpp_add_u32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add_u32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

}  // namespace tg
