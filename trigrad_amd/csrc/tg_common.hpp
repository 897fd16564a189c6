// tg_common.hpp -- shared host helpers and device arithmetic for the gfx950 kernels.
//
// Arithmetic contract: every expression below that feeds a classification
// (tile bounds, depth key, inside test, per-pixel depth, transmittance) is
// evaluated exactly as the reference source writes it, one IEEE-754 operation
// per source operator, no fused multiply-add.  The library must therefore be
// compiled with -ffp-contract=off; float division is hipcc's correctly rounded
// default.  Reference lines are relative to src/trigrad/ of the reference tree.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <cfloat>

#include "../../include/trigrad_hip.h"

namespace tg {

constexpr float kEffZero = FLT_MIN;       // util.h:24
constexpr float kMaxOpacity = 0.9999f;    // util.h:22
constexpr float kFarKey = 1e30f;          // render.cu:259
constexpr int kWave = 64;

// ---- host side ---------------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);

// Per-kernel timing (the counterpart of the reference's CudaTimer,
// render.cu:11-49): when enabled through tg_profile_enable, every launch is
// bracketed by a pair of events on its stream; tg_profile_report waits for
// them and sums the elapsed time per kernel name.
struct ProfileScope {
    ProfileScope(const char *name, hipStream_t stream);
    ~ProfileScope();
    int slot;
    hipStream_t stream;
};
#define TG_LAUNCH(kernel, grid, block, lds, stream, ...)               \
    do {                                                               \
        tg::ProfileScope tg_profile_scope(#kernel, stream);            \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__); \
    } while (0)

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device arithmetic ---------------------------------------------------------
struct Rect { int x0, y0, x1, y1; };  // y0 == -1: the triangle touches no tile

__device__ __forceinline__ float min3(float a, float b, float c) {
    float m = a;
    m = (b < m) ? b : m;
    m = (c < m) ? c : m;
    return m;
}
__device__ __forceinline__ float max3(float a, float b, float c) {
    float m = a;
    m = (m < b) ? b : m;
    m = (m < c) ? c : m;
    return m;
}
__device__ __forceinline__ float clampf(float v, float lo, float hi) { return (v < lo) ? lo : ((hi < v) ? hi : v); }

// Tile coordinate of an NDC coordinate (render.cu:72-75).  The 0.5 literal of
// the source makes the product and quotient double precision.
__device__ __forceinline__ int tile_coord(float m, int extent, int tile, int ntiles) {
    float m1 = m + 1.0f;
    const double scaled = ((double)m1 * 0.5) * (double)extent;
    // dividing by a power of two is an exact scaling, so the reciprocal gives the same double
    const double t = ((tile & (tile - 1)) == 0) ? scaled * (1.0 / (double)tile) : scaled / (double)tile;
    return (int)clampf((float)t, 0.0f, (float)(ntiles - 1));
}

// render.cu:51-76 touched_tiles.
__device__ __forceinline__ Rect tile_rect(float ax, float ay, float bx, float by, float cx, float cy, int W, int H, int tw,
                                          int th, int tiles_x, int tiles_y) {
    float ux = bx - ax, uy = by - ay, vx = cx - ax, vy = cy - ay;
    float area2 = ux * vy - uy * vx;
    Rect r;
    if (fabsf(area2) < kEffZero || isnan(area2) || isinf(area2)) {
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

// Order-preserving map float -> uint32 (ascending floats give ascending integers).
__device__ __forceinline__ uint32_t orderable_bits(float f) {
    uint32_t b = __float_as_uint(f);
    return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}

// render.cu:78-88: bary = M * (x, y, 1).
__device__ __forceinline__ void bary_apply(const float m[9], float px, float py, float &b0, float &b1, float &b2) {
    b0 = m[0] * px + m[1] * py + m[2];
    b1 = m[3] * px + m[4] * py + m[5];
    b2 = m[6] * px + m[7] * py + m[8];
}
// Strictly inside: all three at least FLT_MIN (render.cu:401, 438, 482).
__device__ __forceinline__ bool bary_inside(float b0, float b1, float b2) {
    return !(b0 < kEffZero || b1 < kEffZero || b2 < kEffZero);
}
// util.h:245-250 interpolate3 with per-vertex weights.
__device__ __forceinline__ float interp_w(float b0, float b1, float b2, float a, float b, float c, float w0, float w1, float w2) {
    float denom = b0 * w0 + b1 * w1 + b2 * w2;
    return (b0 * a * w0 + b1 * b * w1 + b2 * c * w2) / denom;
}
// Same with unit weights (multiplication by 1.0f is exact, so it is omitted).
__device__ __forceinline__ float interp_1(float b0, float b1, float b2, float a, float b, float c) {
    float denom = b0 + b1 + b2;
    return (b0 * a + b1 * b + b2 * c) / denom;
}
// Pixel centre in NDC: double expression rounded once (render.cu:561-562).
__device__ __forceinline__ float pixel_ndc(int i, int extent) {
    return (float)(((double)(float)i + 0.5) / (double)(float)extent * 2.0 - 1.0);
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
