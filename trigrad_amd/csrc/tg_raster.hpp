// tg_raster.hpp -- pieces shared by the forward and backward tile kernels.
//
// Launch shape: grid (tiles_x, tiles_y, parts); a workgroup of at most 256 threads
// owns pixels [z*blockDim, (z+1)*blockDim) of its tile in row-major order, so a
// 16x16 tile is exactly one workgroup of four waves and larger tiles are split
// into several workgroups that walk the same list.  A tile's sorted list is consumed in
// batches: up to kBatch threads each gather one list entry (triangle id ->
// vertex ids -> vertex data, bary matrix, attributes) into an LDS record, then
// every pixel thread walks the records; all lanes read the same record at the
// same time, which LDS serves as a broadcast.
#pragma once
#include "tg_common.hpp"

namespace tg {

constexpr int kBatch = 128;         // list entries staged per batch
constexpr int kBoundSpan = 256;     // list entries per depth bound (tg_list_bounds)
constexpr int kLayers = 32;         // per-pixel selection batch (render.cu:570, :655)
constexpr int kMaxTilePixels = 1024;  // tile_w * tile_h limit of the API (wrapper.py:143)
constexpr int kTileThreads = 256;     // workgroup size limit
constexpr int kGatherAhead = 4;       // records a lane of a per-pixel-order kernel fetches together

struct RasterArgs {
    const real4 *vertices;
    const int32_t *indices;
    const real *colors;
    const real *opacities;
    const int32_t *sorted_ids;
    const int32_t *offsets;
    const real *bary;
    const real *batch_bounds;  // per tile and kBoundSpan entries: lower bound of the pixel depths from there on; may be null
    const int32_t *far_start;  // per tile: first list position whose entries the bounds do not cover (with batch_bounds)
    int W, H, tw, th;
    real thr;
    int max_layers;
};

struct PixelCoord {
    int ix, iy, index;
    bool valid;
    real px, py;
};

__device__ __forceinline__ PixelCoord pixel_of_thread(const RasterArgs &a, int tile_x, int tile_y) {
    PixelCoord p;
    const int t = blockIdx.z * blockDim.x + threadIdx.x;
    int lx, ly;
    if (((a.tw | a.th) & 7) == 0) {
        // a wave takes a square of 8 x 8 pixels: fewer list entries touch a square than a strip of the
        // same area, so the waves cull more and share an entry among more lanes
        const int squares_x = a.tw >> 3, square = t >> 6, l = t & 63;
        lx = (square % squares_x) * 8 + (l & 7);
        ly = (square / squares_x) * 8 + (l >> 3);
    } else {
        lx = t % a.tw;
        ly = t / a.tw;
    }
    p.ix = tile_x * a.tw + lx;
    p.iy = tile_y * a.th + ly;
    p.valid = (t < a.tw * a.th) && p.ix < a.W && p.iy < a.H;  // render.cu:554
    p.index = p.iy * a.W + p.ix;
    p.px = pixel_ndc(p.ix, a.W);
    p.py = pixel_ndc(p.iy, a.H);
    return p;
}

// The tile a workgroup of a (tiles_x, tiles_y, parts) launch takes.  Workgroups go to the eight XCDs of the device in
// turn in the order of their linear index, and every XCD has an L2 of its own; neighbouring tiles share list
// entries (a triangle that covers two tiles is in both lists), vertices and matrices.  So the workgroups
// that reach one XCD take consecutive tiles of an order that keeps neighbours together: bands of kTileBand
// tile rows, column by column inside a band.  XCD k gets the k-th eighth of that order, and the workgroups that
// run there at one time cover a compact block of the image.
#ifndef TG_XCD_TILES
#define TG_XCD_TILES 1
#endif
#ifndef TG_TILE_BAND_FORWARD
#define TG_TILE_BAND_FORWARD 8
#endif
#ifndef TG_TILE_BAND_BACKWARD
#define TG_TILE_BAND_BACKWARD 1
#endif
constexpr int kXcds = 8;
constexpr int kTileBandForward = TG_TILE_BAND_FORWARD, kTileBandBackward = TG_TILE_BAND_BACKWARD;
struct TileId { int x, y, index; };
template <int kTileBand>
__device__ __forceinline__ TileId tile_of_workgroup() {
    const int tiles_x = (int)gridDim.x, tiles_y = (int)gridDim.y, n = tiles_x * tiles_y;
    const int linear = (int)(blockIdx.y * gridDim.x + blockIdx.x);
    TileId t;
#if TG_XCD_TILES
    const int per = n / kXcds, rest = n % kXcds;
    const int xcd = linear % kXcds, turn = linear / kXcds;
    const int place = xcd < rest ? xcd * (per + 1) + turn : rest * (per + 1) + (xcd - rest) * per + turn;
    const int band = place / (kTileBand * tiles_x), within = place - band * (kTileBand * tiles_x);
    const int rows = min(kTileBand, tiles_y - band * kTileBand);
    t.x = within / rows;
    t.y = band * kTileBand + within % rows;
#else
    t.x = linear % tiles_x;
    t.y = linear / tiles_x;
#endif
    t.index = t.y * tiles_x + t.x;
    return t;
}
__device__ __forceinline__ PixelCoord pixel_of_thread(const RasterArgs &a, const TileId &t) { return pixel_of_thread(a, t.x, t.y); }

// Everything process_forward (render.cu:417-453) reads for one list entry.
struct alignas(16) BlendRecord {
    real m[9];
    real w[3];
    real iw[3];   // 1/w per vertex (render.cu:444)
    real op[3];
    real col[9];  // vertex a rgb, vertex b rgb, vertex c rgb
    real pad;
};
static_assert(sizeof(BlendRecord) == 28 * sizeof(real), "BlendRecord layout");
constexpr int kBlendWords = 27;  // scalars of a BlendRecord without its padding; odd

// What select_next_k_in_tile (render.cu:375-415) reads for one list entry.
struct alignas(16) DepthRecord {
    real m[9];
    real z[3];
    real w[3];
    real pad;
};
static_assert(sizeof(DepthRecord) == 16 * sizeof(real), "DepthRecord layout");

struct TriIds { int tri, ia, ib, ic; };

__device__ __forceinline__ TriIds load_ids(const RasterArgs &a, int j) {
    TriIds t;
    t.tri = a.sorted_ids[j];
    t.ia = a.indices[3 * (int64_t)t.tri];
    t.ib = a.indices[3 * (int64_t)t.tri + 1];
    t.ic = a.indices[3 * (int64_t)t.tri + 2];
    return t;
}

__device__ __forceinline__ void gather_blend(const RasterArgs &a, int j, BlendRecord &r) {
    const TriIds t = load_ids(a, j);
    const real *m = a.bary + 9 * (int64_t)t.tri;
#pragma unroll
    for (int k = 0; k < 9; k++) r.m[k] = m[k];
    const real wa = a.vertices[t.ia].w, wb = a.vertices[t.ib].w, wc = a.vertices[t.ic].w;
    r.w[0] = wa; r.w[1] = wb; r.w[2] = wc;
    r.iw[0] = 1.0f / wa; r.iw[1] = 1.0f / wb; r.iw[2] = 1.0f / wc;
    r.op[0] = a.opacities[t.ia]; r.op[1] = a.opacities[t.ib]; r.op[2] = a.opacities[t.ic];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        r.col[k] = a.colors[3 * (int64_t)t.ia + k];
        r.col[3 + k] = a.colors[3 * (int64_t)t.ib + k];
        r.col[6 + k] = a.colors[3 * (int64_t)t.ic + k];
    }
}

__device__ __forceinline__ void gather_depth(const RasterArgs &a, int j, DepthRecord &r) {
    const TriIds t = load_ids(a, j);
    const real *m = a.bary + 9 * (int64_t)t.tri;
#pragma unroll
    for (int k = 0; k < 9; k++) r.m[k] = m[k];
    const real4 va = a.vertices[t.ia], vb = a.vertices[t.ib], vc = a.vertices[t.ic];
    r.z[0] = va.z; r.z[1] = vb.z; r.z[2] = vc.z;
    r.w[0] = va.w; r.w[1] = vb.w; r.w[2] = vc.w;
}

// Saved hit masks (tile order).  The buffer starts with one word per workgroup of the tile launch
// (index hit_mask_head_index()): the largest `last` among the workgroup's pixels, i.e. how much of the
// list the backward pass has to walk, known to it without waiting for its pixels' loads.  Then, from
// word hit_mask_head_words() on, word (chunk * slots + slot) holds, for the pixel in thread slot `slot`
// of its tile, which of 64 consecutive list entries cover it.  The chunks of a tile whose list starts
// at `start` are numbered from start / 64 + tile: consecutive tiles never share a chunk, and
// n_keys / 64 + n_tiles + 1 chunks hold every list.
__device__ __forceinline__ int64_t hit_mask_chunk(int start, int tile, int relative_position) {
    return (int64_t)(start >> 6) + tile + (relative_position >> 6);
}
__device__ __forceinline__ int64_t hit_mask_head_index(int tile) { return (int64_t)tile * gridDim.z + blockIdx.z; }
__device__ __forceinline__ int64_t hit_mask_head_words() { return (int64_t)gridDim.x * gridDim.y * gridDim.z; }

// Batch bounds: word batch_bound_index(start, tile, p) holds, for the tile whose
// list starts at `start`, a lower bound of the per-pixel depth of every entry at
// relative position >= p (p a multiple of kBoundSpan) and < far_start[tile].  From
// far_start on the list holds the entries whose clipped polygon was empty (sort
// key 1e30): they lie at the end of the list whatever their depth, almost never
// cover a pixel, and are always looked at.  Tiles never share a word;
// n_keys / kBoundSpan + n_tiles + 1 words hold every list.
__device__ __forceinline__ int64_t batch_bound_index(int start, int tile, int relative_position) {
    return (int64_t)(start / kBoundSpan) + tile + relative_position / kBoundSpan;
}

// Front-to-back compositing state of one pixel (render.cu:564-574).
struct PixelState {
    real alpha = 1.0f, c0 = 0.0f, c1 = 0.0f, c2 = 0.0f, depth = 0.0f, weight = 0.0f;
    int blended = 0;
};

// The arithmetic of process_forward for a fragment known to be inside.
__device__ __forceinline__ void blend_fragment(PixelState &s, const BlendRecord &r, real b0, real b1, real b2) {
    real o = interp_w(b0, b1, b2, r.op[0], r.op[1], r.op[2], r.w[0], r.w[1], r.w[2]);
    o = clampf(o, 0.0f, kMaxOpacity);
    const real k0 = interp_w(b0, b1, b2, r.col[0], r.col[3], r.col[6], r.w[0], r.w[1], r.w[2]);
    const real k1 = interp_w(b0, b1, b2, r.col[1], r.col[4], r.col[7], r.w[0], r.w[1], r.w[2]);
    const real k2 = interp_w(b0, b1, b2, r.col[2], r.col[5], r.col[8], r.w[0], r.w[1], r.w[2]);
    const real z = interp_1(b0, b1, b2, r.iw[0], r.iw[1], r.iw[2]);
    const real ao = s.alpha * o;
    s.depth = s.depth + ao * z;
    s.weight = s.weight + ao;
    s.c0 = s.c0 + ao * k0;
    s.c1 = s.c1 + ao * k1;
    s.c2 = s.c2 + ao * k2;
    s.alpha *= (1.0f - o);
    s.blended++;
}

// ---- host-side launch helpers (defined in tg_forward.hip) ---------------------------
struct TileLaunch { dim3 grid; int threads; };
TileLaunch tile_launch(int width, int height, int tile_w, int tile_h, int max_threads);
int pixel_order_threads(int preferred);
size_t pixel_order_lds_bytes(int n_threads, int staged_entries, size_t position_bytes = sizeof(int));
int check_raster_args(const char *fn, int width, int height, int tile_w, int tile_h, int max_layers);

// ---- per-wave culling ------------------------------------------------------------------
// A wave owns 64 pixels of the tile.  Before its lanes test a list entry, the
// entry is tested once against the rectangle spanned by the wave's pixel
// centres.  The test is exact, not approximate: every IEEE operation is monotone
// in each operand, so the inside test's own expression m0*x + m1*y + m2,
// evaluated with the same operations at the corner that maximises it, bounds
// the value every pixel of the rectangle would compute.  If that bound is below
// the inside threshold for one of the three coordinates, no lane can hit.
struct WaveRect { real x_lo, x_hi, y_lo, y_hi; };

__device__ __forceinline__ bool may_touch(const real m[9], const WaveRect &r) {
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const real mx = m[3 * k], my = m[3 * k + 1];
        const real x = (mx >= 0.0f) ? r.x_hi : r.x_lo;
        const real y = (my >= 0.0f) ? r.y_hi : r.y_lo;
        const real bound = mx * x + my * y + m[3 * k + 2];
        if (bound < kEffZero) return false;  // a NaN bound never culls
    }
    return true;
}

__device__ __forceinline__ real min_real(real a, real b) { return (b < a) ? b : a; }
__device__ __forceinline__ real max_real(real a, real b) { return (a < b) ? b : a; }
__device__ __forceinline__ real wave_min(real v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = min_real(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ real wave_max(real v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max_real(v, __shfl_xor(v, off, kWave));
    return v;
}

constexpr int kMaxTileWaves = kTileThreads / kWave;

// Every wave publishes the rectangle of its valid pixels (an empty rectangle,
// lo > hi, if it has none); call with all threads, followed by __syncthreads().
__device__ __forceinline__ void publish_wave_rect(const PixelCoord &p, WaveRect *s_rects) {
    const real big = 3.0e38f;
    WaveRect r;
    r.x_lo = wave_min(p.valid ? p.px : big);
    r.x_hi = wave_max(p.valid ? p.px : -big);
    r.y_lo = wave_min(p.valid ? p.py : big);
    r.y_hi = wave_max(p.valid ? p.py : -big);
    if ((threadIdx.x & (kWave - 1)) == 0) s_rects[threadIdx.x / kWave] = r;
}

// Bit w of the result: wave w has to look at the entry.
__device__ __forceinline__ uint32_t waves_touched(const real m[9], const WaveRect *s_rects, int n_waves) {
    uint32_t bits = 0;
#pragma unroll 1
    for (int w = 0; w < n_waves; w++) {
        const WaveRect r = s_rects[w];
        if (r.x_lo <= r.x_hi && may_touch(m, r)) bits |= 1u << w;
    }
    return bits;
}

// 64 staged entries starting at `first`: mask of those the calling wave has to look at.
__device__ __forceinline__ uint64_t wave_candidates(const uint8_t *s_touch, int first, int n_entries, int wave) {
    const int e = first + (threadIdx.x & (kWave - 1));
    const bool mine = e < n_entries && ((s_touch[e] >> wave) & 1u);
    return __builtin_amdgcn_ballot_w64(mine);
}

// Inside tests of one staged batch for the calling lane's pixel: bit e of the
// result (word e / 64) is set when record e covers the pixel.  All lanes of the
// wave read the same record at the same time (LDS broadcast); only records that
// can touch the wave's pixels are looked at.  Rec must have a member m[9].
template <int kWords, typename Rec>
__device__ __forceinline__ void batch_hit_mask(const Rec *s_rec, const uint8_t *s_touch, int nb, int wave, real px, real py,
                                               uint64_t m[kWords]) {
#pragma unroll
    for (int wd = 0; wd < kWords; wd++) {
        const uint64_t todo = wave_candidates(s_touch, wd * kWave, nb, wave);
        // the lane's mask is built in 32-bit halves: a set bit then costs three vector operations, not six
        uint32_t half[2] = {0u, 0u};
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t left = (uint32_t)(todo >> (32 * h));
            while (left) {
                const int bit = __builtin_ctz(left);
                left &= left - 1;
                real b0, b1, b2;
                bary_apply(s_rec[wd * kWave + 32 * h + bit].m, px, py, b0, b1, b2);
                if (bary_inside(b0, b1, b2)) half[h] |= 1u << bit;
            }
        }
        m[wd] = ((uint64_t)half[1] << 32) | half[0];
    }
}

// Lowest set bit of a mask of kWords 64-bit words, removed from the mask; -1 if the mask is empty.
template <int kWords>
__device__ __forceinline__ int pop_lowest(uint64_t m[kWords]) {
    int e = -1;
#pragma unroll
    for (int wd = 0; wd < kWords; wd++)
        if (e < 0 && m[wd]) {
            e = 64 * wd + __builtin_ctzll(m[wd]);
            m[wd] &= m[wd] - 1;
        }
    return e;
}

// Per-pixel candidate lists of the per-pixel-sort mode live in LDS, slot-major:
// entry `slot` of thread `t` is at [slot * n_threads + t] (conflict-free).
template <typename Pos>
struct TopKOf {
    real *depth;
    Pos *pos;
    int n_threads;
    __device__ __forceinline__ real &d(int slot) const { return depth[slot * n_threads + threadIdx.x]; }
    __device__ __forceinline__ Pos &j(int slot) const { return pos[slot * n_threads + threadIdx.x]; }
};
using TopK = TopKOf<int>;

}  // namespace tg
