// tg_binning.hip -- tile binning (count, scan, key emission) and bary matrices.
//
// Three routes to the same keys, all with one thread per KEY in the emission (a triangle that covers thousands of
// tiles is spread over thousands of lanes) and the clip polygon of a key in LDS:
//   stage by stage   bin_count_kernel (12 B indices + 3 x 16 B vertex gathers read, 4 B written per triangle), the
//                    scan of tg_scan.hip, bin_emit_kernel (reads the triangle again, 12 B written per key)
//   two calls        bin_setup_kernel (count + scan + a 48-byte record per triangle in one pass), then
//                    bin_emit_records_kernel from the records; the host reads K in between
//   one call         frame_scan_kernel + frame_emit_kernel: as the two calls, with nothing to clear beforehand,
//                    the digit totals of the sort from two additions per triangle, K read on the device, and only
//                    the clip passes run that a key needs
// The count + scan kernels and bary_kernel (60 B read, 36 B written per triangle) are bound by memory traffic, the
// emission kernels by the vector instructions of the clipping.
#include "tg_raster.hpp"
#include "tg_scan.hpp"
#include "tg_sort_plan.hpp"

namespace tg {

constexpr int kBinThreads = 256;

struct TriXYZ { real ax, ay, az, bx, by, bz, cx, cy, cz; bool ok; };

// A triangle that names a vertex outside [0, n_vertices) is treated as
// degenerate (all coordinates zero) instead of being dereferenced.
__device__ __forceinline__ TriXYZ load_triangle(const real4 *__restrict__ vertices, int n_vertices,
                                                const int32_t *__restrict__ indices, int t) {
    const int ia = indices[3 * (int64_t)t], ib = indices[3 * (int64_t)t + 1], ic = indices[3 * (int64_t)t + 2];
    TriXYZ r;
    r.ok = (unsigned)ia < (unsigned)n_vertices && (unsigned)ib < (unsigned)n_vertices && (unsigned)ic < (unsigned)n_vertices;
    const real4 zero = make_real4(0.f, 0.f, 0.f, 0.f);
    const real4 a = r.ok ? vertices[ia] : zero, b = r.ok ? vertices[ib] : zero, c = r.ok ? vertices[ic] : zero;
    r.ax = a.x; r.ay = a.y; r.az = a.z;
    r.bx = b.x; r.by = b.y; r.bz = b.z;
    r.cx = c.x; r.cy = c.y; r.cz = c.z;
    return r;
}

// The three corners of the triangle with the vertex numbers (ia, ib, ic), zeros for a triangle that names a
// vertex outside [0, n_vertices).
__device__ __forceinline__ void fetch_corners(const real4 *__restrict__ vertices, int n_vertices, int ia, int ib, int ic, real4 &a,
                                              real4 &b, real4 &c) {
    const bool ok = (unsigned)ia < (unsigned)n_vertices && (unsigned)ib < (unsigned)n_vertices && (unsigned)ic < (unsigned)n_vertices;
    a = b = c = make_real4(0.f, 0.f, 0.f, 0.f);
    if (ok) {
        a = vertices[ia];
        b = vertices[ib];
        c = vertices[ic];
    }
}

__global__ __launch_bounds__(kBinThreads) void bin_count_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                                const int32_t *__restrict__ indices, int n_triangles, int W,
                                                                int H, int tw, int th, int tiles_x, int tiles_y,
                                                                uint32_t *__restrict__ tri_counts) {
    const int t = blockIdx.x * kBinThreads + threadIdx.x;
    if (t >= n_triangles) return;
    const TriXYZ p = load_triangle(vertices, n_vertices, indices, t);
    const Rect r = tile_rect(p.ax, p.ay, p.bx, p.by, p.cx, p.cy, W, H, tw, th, tiles_x, tiles_y);
    tri_counts[t] = rect_count(r);
}

// Per-thread polygon storage in LDS, slot-major so that lanes never conflict.
constexpr int kPolyCap = 8;
constexpr int kOwnerWindow = 1024;  // triangle offsets staged per workgroup for the owner search
template <int THREADS>
struct PolyLdsOf {
    real x[kPolyCap][THREADS];
    real y[kPolyCap][THREADS];
};
using PolyLds = PolyLdsOf<kBinThreads>;

// One Sutherland-Hodgman pass (render.cu:159-189) against nx*x + ny*y - d >= 0, in place.  Returns the new
// vertex count.  The polygon is read into registers first (the loop over the eight slots is unrolled, so
// they are plain registers and every distance is computed once); the output goes back to the same LDS slots
// at its own running index.  When every vertex is inside, the pass reproduces its input and nothing is written.
template <typename Poly>
__device__ __forceinline__ int clip_pass(Poly &lds, int n_in, real nx, real ny, real d) {
    const int tid = threadIdx.x;
    real px[kPolyCap], py[kPolyCap], dist[kPolyCap];
    bool all_in = true;
#pragma unroll
    for (int i = 0; i < kPolyCap; i++) {
        if (i < n_in) {
            px[i] = lds.x[i][tid];
            py[i] = lds.y[i][tid];
            dist[i] = nx * px[i] + ny * py[i] - d;
            all_in = all_in && (dist[i] >= 0.0f);
        }
    }
    if (all_in) return n_in;
    int n_out = 0;
    real p0x = lds.x[n_in - 1][tid], p0y = lds.y[n_in - 1][tid];
    real d0 = nx * p0x + ny * p0y - d;
    bool in0 = d0 >= 0.0f;
#pragma unroll
    for (int i = 0; i < kPolyCap; i++) {
        if (i < n_in) {
            const real p1x = px[i], p1y = py[i];
            const real d1 = dist[i];
            const bool in1 = d1 >= 0.0f;
            // A convex polygon gains at most one vertex per pass (7 after four); the
            // capacity test only matters for slivers whose in/out pattern alternates
            // by rounding, where vertices beyond the eighth are dropped.
            if (in1 != in0 && n_out < kPolyCap) {
                const real t = d0 / (d0 - d1);
                lds.x[n_out][tid] = p0x + t * (p1x - p0x);
                lds.y[n_out][tid] = p0y + t * (p1y - p0y);
                n_out++;
            }
            if (in1 && n_out < kPolyCap) {
                lds.x[n_out][tid] = p1x;
                lds.y[n_out][tid] = p1y;
                n_out++;
            }
            p0x = p1x; p0y = p1y; d0 = d1; in0 = in1;
        }
    }
    return n_out;
}

// Index of the triangle that owns key k: the last i with tri_offsets[i] <= k.
__device__ __forceinline__ int owner_of_key(const uint32_t *__restrict__ tri_offsets, int n_triangles, uint32_t k) {
    int lo = 0, hi = n_triangles;  // invariant: tri_offsets[lo] <= k, answer in [lo, hi)
    while (hi - lo > 1) {
        const int mid = lo + ((hi - lo) >> 1);
        if (tri_offsets[mid] <= k) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(kBinThreads) void bin_emit_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                               const int32_t *__restrict__ indices, int n_triangles, int W,
                                                               int H, int tw, int th, int tiles_x, int tiles_y,
                                                               const uint32_t *__restrict__ tri_offsets, int64_t n_keys,
                                                               const uint32_t *__restrict__ owner_heads, uint32_t owner_capacity,
                                                               uint64_t *__restrict__ keys, uint32_t *__restrict__ payload) {
    __shared__ PolyLds lds;
    __shared__ uint32_t s_offsets[kOwnerWindow];
    const int tid = threadIdx.x;
    const int64_t k0 = (int64_t)blockIdx.x * kBinThreads;
    const int64_t k = k0 + tid;
    // The owners of this workgroup's 256 keys lie between the owner of its first
    // key and the owner of the next workgroup's first key; the scan noted both
    // (otherwise two workgroup-uniform binary searches find them).  The offsets
    // in between are staged in LDS and searched there.
    int t_first, t_last;
    if (owner_heads && blockIdx.x < owner_capacity) {
        t_first = (int)owner_heads[blockIdx.x];
        t_last = (k0 + kBinThreads < n_keys && blockIdx.x + 1 < owner_capacity) ? (int)owner_heads[blockIdx.x + 1] : n_triangles - 1;
    } else {
        const int64_t k_last = (k0 + kBinThreads <= n_keys ? k0 + kBinThreads : n_keys) - 1;
        t_first = owner_of_key(tri_offsets, n_triangles, (uint32_t)k0);
        t_last = owner_of_key(tri_offsets, n_triangles, (uint32_t)k_last);
    }
    const int span = t_last - t_first + 1;
    const bool windowed = span <= kOwnerWindow;
    if (windowed)
        for (int i = tid; i < span; i += kBinThreads) s_offsets[i] = tri_offsets[t_first + i];
    __syncthreads();
    if (k >= n_keys) return;  // no barrier below: the polygon arrays are private per thread

    int t;
    uint32_t owner_offset;
    if (windowed) {
        int lo = 0, hi = span;  // s_offsets[lo] <= k, answer in [lo, hi)
        while (hi - lo > 1) {
            const int mid = lo + ((hi - lo) >> 1);
            if (s_offsets[mid] <= (uint32_t)k) lo = mid; else hi = mid;
        }
        t = t_first + lo;
        owner_offset = s_offsets[lo];
    } else {
        t = owner_of_key(tri_offsets, n_triangles, (uint32_t)k);
        owner_offset = tri_offsets[t];
    }
    const uint32_t local = (uint32_t)k - owner_offset;
    const TriXYZ p = load_triangle(vertices, n_vertices, indices, t);
    const Rect r = tile_rect(p.ax, p.ay, p.bx, p.by, p.cx, p.cy, W, H, tw, th, tiles_x, tiles_y);
    const uint32_t ny = (uint32_t)(r.y1 - r.y0 + 1);
    const int tx = r.x0 + (int)(local / ny);  // tile x outer, tile y inner (render.cu:235-236)
    const int ty = r.y0 + (int)(local % ny);

    // render.cu:140-152 compute_plane
    const real det = p.ax * (p.by - p.cy) + p.bx * (p.cy - p.ay) + p.cx * (p.ay - p.by);
    const real id = (real)(1.0 / (double)det);
    const real A = (p.az * (p.by - p.cy) + p.bz * (p.cy - p.ay) + p.cz * (p.ay - p.by)) * id;
    const real B = (p.ax * (p.bz - p.cz) + p.bx * (p.cz - p.az) + p.cx * (p.az - p.bz)) * id;
    const real C = (p.ax * (p.by * p.cz - p.cy * p.bz) + p.bx * (p.cy * p.az - p.ay * p.cz) + p.cx * (p.ay * p.bz - p.by * p.az)) * id;

    // render.cu:243-246 tile rectangle in NDC
    const real xmin = (real)(tx * tw) / (real)W * 2.0f - 1.0f;
    const real xmax = (real)((tx + 1) * tw) / (real)W * 2.0f - 1.0f;
    const real ymin = (real)(ty * th) / (real)H * 2.0f - 1.0f;
    const real ymax = (real)((ty + 1) * th) / (real)H * 2.0f - 1.0f;

    lds.x[0][tid] = p.ax; lds.y[0][tid] = p.ay;
    lds.x[1][tid] = p.bx; lds.y[1][tid] = p.by;
    lds.x[2][tid] = p.cx; lds.y[2][tid] = p.cy;
    int n = 3;
    n = clip_pass(lds, n, 1.0f, 0.0f, xmin);                 // render.cu:254-257
    if (n > 0) n = clip_pass(lds, n, -1.0f, 0.0f, -xmax);
    if (n > 0) n = clip_pass(lds, n, 0.0f, 1.0f, ymin);
    if (n > 0) n = clip_pass(lds, n, 0.0f, -1.0f, -ymax);

    real key = kFarKey;  // render.cu:259
    if (n > 0) {
        real md = std::numeric_limits<real>::max();
        for (int i = 0; i < n; i++) {
            const real pd = A * lds.x[i][tid] + B * lds.y[i][tid] + C;  // render.cu:154-157
            md = (pd < md) ? pd : md;
        }
        key = md;
    }
    const uint32_t tile = (uint32_t)(ty * tiles_x + tx);
#ifdef TG_DOUBLE_PRECISION
    keys[k] = orderable_bits(key);  // all 64 bits are depth; the tile ids follow the depth keys
    keys[n_keys + k] = tile;
#else
    keys[k] = ((uint64_t)tile << 32) | orderable_bits(key);
#endif
    payload[k] = (uint32_t)t;
}

// ---- the frame's binning in two launches ---------------------------------------------------------------
//
// bin_setup_kernel counts and scans in one pass over the triangles (the tile's count total goes through the
// same decoupled look-back as the plain scan) and leaves, per triangle, a record of what the emission needs
// for each of its keys: the depth plane, the first tile and the rows of the tile rectangle, the three
// corners.  bin_emit_records_kernel then reads one record per key instead of the triangle's indices and
// vertices, and does per key only what depends on the tile: the clip and the minimum.
//
// Frame state (caller's memory, tg_bin_setup_workspace_bytes): scan ticket, the sort's tickets, the digit
// totals of the tile passes, the NDC edges of the tile columns and rows, the scan's state words.  bin_init_kernel clears it and fills in the edges.
constexpr int kRecordReals = TG_RECORD_SCALARS;  // three planes of M x 4: A B C x0 | ax ay bx by | cx cy y0 ny
static_assert(kRecordReals == 12, "three real4 per triangle");
constexpr int kStateTicketWords = 64;   // word 0: scan ticket; kSweepTicketWord..+7: sweep tickets
constexpr int kStateTotalsWords = kEmitDigitPasses * kRadix * kTotalsStride;

struct FrameState {
    uint32_t *tickets;
    uint32_t *totals;
    real *edges;       // tiles_x + 1 column edges, then tiles_y + 1 row edges
    uint64_t *states;  // one per kScanTile triangles
    size_t bytes;
};

static FrameState frame_state(void *base, int64_t n_triangles, int tiles_x, int tiles_y) {
    FrameState f;
    char *p = (char *)base;
    size_t o = 0;
    f.tickets = (uint32_t *)(p + o); o += kStateTicketWords * 4;
    f.totals = (uint32_t *)(p + o);  o += kStateTotalsWords * 4;
    f.states = (uint64_t *)(p + o);  o += (size_t)(ceil_div64(n_triangles, kScanTile) + 1) * 8;
    f.edges = (real *)(p + o);       o += (size_t)(tiles_x + tiles_y + 2) * sizeof(real);
    f.bytes = (o + 255) & ~(size_t)255;
    return f;
}

__global__ __launch_bounds__(1024) void bin_init_kernel(uint32_t *zero, size_t zero_words, real *edges, int W, int H, int tw, int th,
                                                        int tiles_x, int tiles_y, uint32_t *total_and_status) {
    for (size_t i = threadIdx.x; i < zero_words; i += blockDim.x) zero[i] = 0;
    // render.cu:243-246: the edges of tile column tx are entries tx and tx + 1
    for (int i = threadIdx.x; i <= tiles_x; i += blockDim.x) edges[i] = (real)(i * tw) / (real)W * 2.0f - 1.0f;
    for (int i = threadIdx.x; i <= tiles_y; i += blockDim.x) edges[tiles_x + 1 + i] = (real)(i * th) / (real)H * 2.0f - 1.0f;
    if (threadIdx.x < 2) total_and_status[threadIdx.x] = 0;
}

// Adds the digits of the tile passes (plan: shifts count from key bit 0, the tile number starts at bit 32) of
// every tile of the calling lane's rectangle to the workgroup's LDS counters.  A rectangle of up to 64 tiles
// is walked by its lane; larger ones are taken one after the other by the whole wave, 64 tiles at a time, so
// that a triangle that covers thousands of tiles does not hold its wave up.  All 64 lanes call this.
constexpr uint32_t kLaneRectTiles = 64;
__device__ __forceinline__ void count_tile_digits(const Rect &r, uint32_t count, int tiles_x, const PassPlan &plan,
                                                  uint32_t (*hist)[kRadix]) {
    const int lane = threadIdx.x & (kWave - 1);
    const int shift0 = plan.shift[0] - 32, shift1 = plan.shift[1] - 32;
    const uint32_t mask0 = (1u << plan.bits[0]) - 1, mask1 = (1u << plan.bits[1]) - 1;
    const bool two = plan.passes > 1;
    if (count > 0 && count <= kLaneRectTiles) {
        for (int tx = r.x0; tx <= r.x1; tx++)
            for (int ty = r.y0; ty <= r.y1; ty++) {
                const uint32_t tile = (uint32_t)(ty * tiles_x + tx);
                atomicAdd(&hist[0][(tile >> shift0) & mask0], 1u);
                if (two) atomicAdd(&hist[1][(tile >> shift1) & mask1], 1u);
            }
    }
    uint64_t large = __builtin_amdgcn_ballot_w64(count > kLaneRectTiles);
    while (large) {
        const int src = __builtin_ctzll(large);
        large &= large - 1;
        const int x0 = __shfl(r.x0, src, kWave), y0 = __shfl(r.y0, src, kWave);
        const int ny = __shfl(r.y1, src, kWave) - y0 + 1, nx = __shfl(r.x1, src, kWave) - x0 + 1;
        // lane l takes the tiles l, l + 64, ... of the rectangle in column-major order (column = tile x)
        int col = lane / ny, row = lane % ny;
        const int col_step = kWave / ny, row_step = kWave % ny;
        while (col < nx) {
            const uint32_t tile = (uint32_t)((y0 + row) * tiles_x + x0 + col);
            atomicAdd(&hist[0][(tile >> shift0) & mask0], 1u);
            if (two) atomicAdd(&hist[1][(tile >> shift1) & mask1], 1u);
            col += col_step;
            row += row_step;
            if (row >= ny) { row -= ny; col++; }
        }
    }
}

__global__ __launch_bounds__(kScanThreads) void bin_setup_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                                 const int32_t *__restrict__ indices, int n_triangles, int W, int H,
                                                                 int tw, int th, int tiles_x, int tiles_y,
                                                                 uint32_t *__restrict__ tri_offsets, real4 *__restrict__ records,
                                                                 uint32_t *total, uint32_t *status, uint32_t *ticket, uint64_t *states,
                                                                 int n_scan_tiles, uint32_t head_capacity, uint32_t *__restrict__ heads,
                                                                 PassPlan plan, uint32_t *totals) {
    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_wave_total[kScanThreads / kWave];
    __shared__ uint32_t s_tile_prefix;
    __shared__ uint32_t s_count[kScanTile];
    __shared__ uint32_t s_hist[kEmitDigitPasses][kRadix];
    if (totals && threadIdx.x < kRadix)
        for (int p = 0; p < kEmitDigitPasses; p++) s_hist[p][threadIdx.x] = 0;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    if (tid == 0) s_tile = ticket ? atomicAdd(ticket, 1u) : blockIdx.x;  // no ticket: the whole grid is resident
    __syncthreads();
    const int tile = (int)s_tile;
    const int64_t base = (int64_t)tile * kScanTile + (int64_t)tid * 4;

    // Triangle by triangle across the lanes (neighbouring lanes take neighbouring triangles, so the index
    // loads and the record stores of a wave are contiguous); the counts then change hands through LDS so that
    // every thread scans four consecutive ones.
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t t = (int64_t)tile * kScanTile + k * kScanThreads + tid;
        uint32_t count = 0;
        Rect rect = {0, -1, 0, -1};
        if (t < n_triangles) {
            const TriXYZ p = load_triangle(vertices, n_vertices, indices, (int)t);
            const Rect r = tile_rect(p.ax, p.ay, p.bx, p.by, p.cx, p.cy, W, H, tw, th, tiles_x, tiles_y);
            count = rect_count(r);
            // render.cu:140-152 compute_plane
            const real det = p.ax * (p.by - p.cy) + p.bx * (p.cy - p.ay) + p.cx * (p.ay - p.by);
            const real id = (real)(1.0 / (double)det);
            const real A = (p.az * (p.by - p.cy) + p.bz * (p.cy - p.ay) + p.cz * (p.ay - p.by)) * id;
            const real B = (p.ax * (p.bz - p.cz) + p.bx * (p.cz - p.az) + p.cx * (p.az - p.bz)) * id;
            const real C = (p.ax * (p.by * p.cz - p.cy * p.bz) + p.bx * (p.cy * p.az - p.ay * p.cz) + p.cx * (p.ay * p.bz - p.by * p.az)) * id;
            records[t] = make_real4(A, B, C, int_in_real(r.x0));
            records[(int64_t)n_triangles + t] = make_real4(p.ax, p.ay, p.bx, p.by);
            records[2 * (int64_t)n_triangles + t] = make_real4(p.cx, p.cy, int_in_real(r.y0), int_in_real(r.y1 - r.y0 + 1));
            rect = r;
        }
        s_count[k * kScanThreads + tid] = count;
        if (totals) count_tile_digits(rect, count, tiles_x, plan, s_hist);
    }
    __syncthreads();
    if (totals && tid < kRadix)
        for (int p = 0; p < plan.passes; p++) {
            const uint32_t c = s_hist[p][tid];
            if (c) atomicAdd(&totals[p * kRadix + tid], c);
        }
    uint32_t x[4];
#pragma unroll
    for (int k = 0; k < 4; k++) x[k] = s_count[tid * 4 + k];
    const uint32_t thread_sum = x[0] + x[1] + x[2] + x[3];
    const uint32_t incl = wave_inclusive_scan_u32(thread_sum);
    if (lane == kWave - 1) s_wave_total[wave] = incl;
    __syncthreads();
    if (wave == 0) {
        uint32_t wt = (lane < kScanThreads / kWave) ? s_wave_total[lane] : 0u;
        uint32_t wincl = wave_inclusive_scan_u32(wt);
        uint32_t tile_total = (uint32_t)__builtin_amdgcn_readlane((int)wincl, kScanThreads / kWave - 1);
        if (lane < kScanThreads / kWave) s_wave_total[lane] = wincl - wt;  // exclusive wave offsets
        const uint32_t prefix = scan_tile_prefix(states, tile, tile_total, n_scan_tiles, total, status);
        if (lane == 0) s_tile_prefix = prefix;
    }
    __syncthreads();
    uint32_t run = s_tile_prefix + s_wave_total[wave] + (incl - thread_sum);
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t t = base + k;
        if (t >= n_triangles) break;
        tri_offsets[t] = run;
        if (heads && x[k] != 0) {
            // triangle t owns the key positions [run, run + x): note for every multiple of 256 who owns it
            const uint32_t first = (run + kBinThreads - 1) / kBinThreads, last = (run + x[k] - 1) / kBinThreads;
            for (uint32_t h = first; h <= last && h < head_capacity; h++) heads[h] = (uint32_t)t;
        }
        run += x[k];
    }
}


// One thread per key, like bin_emit_kernel, from the triangles' records.  A workgroup takes `chunks_per_group`
// consecutive chunks of 256 keys.  It also counts the digits of the tile passes of the sort that follows (plan,
// totals: LDS counters, one global atomic per digit and workgroup at the end) and clears zero_words words
// from `zero` on (the sort's look-back words).
__global__ __launch_bounds__(kBinThreads) void bin_emit_records_kernel(const real4 *__restrict__ records,
                                                                       const uint32_t *__restrict__ tri_offsets, int n_triangles,
                                                                       int64_t n_keys, const uint32_t *__restrict__ owner_heads,
                                                                       uint32_t owner_capacity, const real *__restrict__ edges,
                                                                       int tiles_x, int tiles_y, uint64_t *__restrict__ keys,
                                                                       uint32_t *__restrict__ payload, uint32_t *zero,
                                                                       size_t zero_words, uint32_t *clear_word,
                                                                       uint32_t *sweep_tickets, int chunks_per_group) {
    __shared__ PolyLds lds;
    __shared__ uint32_t s_offsets[kOwnerWindow];
    const int tid = threadIdx.x;
    for (size_t i = (size_t)blockIdx.x * kBinThreads + tid; i < zero_words; i += (size_t)gridDim.x * kBinThreads) zero[i] = 0;
    if (clear_word && blockIdx.x == 0 && tid == 0) *clear_word = 0;
    // the sweeps that follow count their tickets up from zero: a frame state may serve more than one sorting call
    if (sweep_tickets && blockIdx.x == 0 && tid < kMaxPasses) sweep_tickets[tid] = 0;
    const int64_t n_chunks = (n_keys + kBinThreads - 1) / kBinThreads;
    const int64_t chunk_end = ((int64_t)blockIdx.x + 1) * chunks_per_group < n_chunks ? ((int64_t)blockIdx.x + 1) * chunks_per_group : n_chunks;
    for (int64_t chunk = (int64_t)blockIdx.x * chunks_per_group; chunk < chunk_end; chunk++) {
        const int64_t k0 = chunk * kBinThreads;
        const int64_t k = k0 + tid;
        // The owners of the chunk's 256 keys lie between the owner of its first key and the owner of the next
        // chunk's first key; the scan noted both (otherwise two uniform binary searches find them).
        int t_first, t_last;
        if (owner_heads && chunk < owner_capacity) {
            t_first = (int)owner_heads[chunk];
            t_last = (k0 + kBinThreads < n_keys && chunk + 1 < owner_capacity) ? (int)owner_heads[chunk + 1] : n_triangles - 1;
        } else {
            const int64_t k_last = (k0 + kBinThreads <= n_keys ? k0 + kBinThreads : n_keys) - 1;
            t_first = owner_of_key(tri_offsets, n_triangles, (uint32_t)k0);
            t_last = owner_of_key(tri_offsets, n_triangles, (uint32_t)k_last);
        }
        const int span = t_last - t_first + 1;
        const bool windowed = span <= kOwnerWindow;
        __syncthreads();  // the previous chunk's searches are done with s_offsets
        if (windowed)
            for (int i = tid; i < span; i += kBinThreads) s_offsets[i] = tri_offsets[t_first + i];
        __syncthreads();
        if (k >= n_keys) continue;  // the polygon arrays are private per thread; the barriers above are uniform

        int t;
        uint32_t owner_offset;
        if (windowed) {
            int lo = 0, hi = span;  // s_offsets[lo] <= k, answer in [lo, hi)
            while (hi - lo > 1) {
                const int mid = lo + ((hi - lo) >> 1);
                if (s_offsets[mid] <= (uint32_t)k) lo = mid; else hi = mid;
            }
            t = t_first + lo;
            owner_offset = s_offsets[lo];
        } else {
            t = owner_of_key(tri_offsets, n_triangles, (uint32_t)k);
            owner_offset = tri_offsets[t];
        }
        const uint32_t local = (uint32_t)k - owner_offset;
        const real4 r0 = records[t], r1 = records[(int64_t)n_triangles + t], r2 = records[2 * (int64_t)n_triangles + t];
        const real A = r0.x, B = r0.y, C = r0.z;
        const uint32_t ny = (uint32_t)int_of_real(r2.w);
        const int tx = int_of_real(r0.w) + (int)(local / ny);  // tile x outer, tile y inner (render.cu:235-236)
        const int ty = int_of_real(r2.z) + (int)(local % ny);

        // render.cu:243-246 tile rectangle in NDC
        const real xmin = edges[tx], xmax = edges[tx + 1];  // a few hundred scalars that every key reads: they stay in cache
        const real ymin = edges[tiles_x + 1 + ty], ymax = edges[tiles_x + 2 + ty];

        lds.x[0][tid] = r1.x; lds.y[0][tid] = r1.y;
        lds.x[1][tid] = r1.z; lds.y[1][tid] = r1.w;
        lds.x[2][tid] = r2.x; lds.y[2][tid] = r2.y;
        int n = 3;
        n = clip_pass(lds, n, 1.0f, 0.0f, xmin);                 // render.cu:254-257
        if (n > 0) n = clip_pass(lds, n, -1.0f, 0.0f, -xmax);
        if (n > 0) n = clip_pass(lds, n, 0.0f, 1.0f, ymin);
        if (n > 0) n = clip_pass(lds, n, 0.0f, -1.0f, -ymax);

        real key = kFarKey;  // render.cu:259
        if (n > 0) {
            real md = std::numeric_limits<real>::max();
            for (int i = 0; i < n; i++) {
                const real pd = A * lds.x[i][tid] + B * lds.y[i][tid] + C;  // render.cu:154-157
                md = (pd < md) ? pd : md;
            }
            key = md;
        }
        const uint32_t tile = (uint32_t)(ty * tiles_x + tx);
#ifdef TG_DOUBLE_PRECISION
        keys[k] = orderable_bits(key);  // all 64 bits are depth; the tile ids follow the depth keys
        keys[n_keys + k] = tile;
#else
        keys[k] = ((uint64_t)tile << 32) | orderable_bits(key);
#endif
        payload[k] = (uint32_t)t;
    }
}

// ---- the frame's binning: two launches that leave nothing for the host to do in between ------------------
//
// frame_scan_kernel   counts and scans in one pass over the triangles, like bin_setup_kernel, and leaves the same
//                     records; but every word it shares between workgroups or calls carries the call's epoch, so
//                     nothing has to be cleared before the launch: a state word of another epoch is "not yet
//                     written".  The digit totals go to one of two sets in turn (a call counts into one and
//                     clears the other).  The look-back reads 512 predecessors per round trip.
// frame_emit_kernel   one workgroup per kEmitChunk key positions.  It reads K from the device, so it is launched
//                     for the capacity of the key buffers before the host knows K.  Per key it runs only those
//                     of the four clip passes that can change the polygon, and keys that run the same number of
//                     passes are put on the same wave.
// Which passes can be skipped: a pass whose half plane holds every vertex reproduces its input (render.cu:159-189).
// While the polygon is the triangle itself that is a comparison of the triangle's bounds with the tile edge.  A
// vertex made by an earlier pass is p0 + t (p1 - p0) with 0 <= t <= 1, which rounding can push past the
// bounds of p0 and p1 by at most 5 ulps of the largest coordinate; over four passes that stays below 2^-19 of
// it.  So a pass is left out only when the bounds clear the tile edge by that margin, and is run, with its own
// test of every vertex, whenever they do not: the polygon is the reference's in every case.
constexpr int kEmitThreads = 256;
[[maybe_unused]] constexpr int kEmitWaves = kEmitThreads / kWave;
constexpr int kEmitKeys = 2;  // keys per thread
constexpr int kEmitChunk = kEmitThreads * kEmitKeys;
constexpr int kFrameMaxTiles = 1 << 21;  // the reciprocal multiply finds a key's column exactly up to here
constexpr int kFrameTotalsWords = 2 * kEmitDigitPasses * kRadix;  // two sets: a call counts into one and clears the other
constexpr int kLookSlots = 8;  // state words a lane of the look-back reads per round trip
constexpr uint32_t kEpochMask = 0x3fffffffu;

// A workgroup barrier that orders the LDS traffic only.  __syncthreads also waits for every global load and
// store the wave has in flight, which these kernels' barriers, all between LDS phases, have no use for.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// State word of the scan: bits 63..62 = 1 tile total, 2 inclusive prefix; bits 61..32 = the call's epoch;
// bits 31..0 = the value.  A word whose epoch is another call's counts as not written.
__device__ __forceinline__ uint64_t stamped(uint32_t flag, uint32_t epoch, uint32_t value) {
    return ((uint64_t)flag << 62) | ((uint64_t)(epoch & kEpochMask) << 32) | value;
}
__device__ __forceinline__ uint32_t stamp_flag(uint64_t word, uint32_t epoch) {
    return ((uint32_t)(word >> 32) & kEpochMask) == (epoch & kEpochMask) ? (uint32_t)(word >> 62) : 0u;
}

// Called by the first wave of the workgroup that owns `tile`: publishes the tile's total, adds up the totals of
// all earlier tiles (64 * kLookSlots state words per round trip, the nearest inclusive prefix ends the walk),
// publishes the inclusive prefix and returns the exclusive one.  The last tile writes the grand total.
__device__ __forceinline__ uint32_t frame_tile_prefix(uint64_t *states, int tile, uint32_t tile_total, int n_tiles, uint32_t epoch,
                                                      uint32_t *total_and_status) {
    const int lane = threadIdx.x & (kWave - 1);
    if (lane == 0) __hip_atomic_store(&states[tile], stamped(tile == 0 ? 2u : 1u, epoch, tile_total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t sum = 0;
    bool timed_out = false;
    for (int look = tile - 1; look >= 0; look -= kWave * kLookSlots) {
        uint64_t word[kLookSlots];
#pragma unroll
        for (int k = 0; k < kLookSlots; k++) {
            const int idx = look - (k * kWave + lane);
            word[k] = idx >= 0 ? __hip_atomic_load(&states[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : stamped(2u, epoch, 0u);
        }
        bool done = false;
#pragma unroll
        for (int k = 0; k < kLookSlots; k++) {
            if (done) continue;  // uniform
            const int idx = look - (k * kWave + lane);
            uint32_t spins = 0;
            while (stamp_flag(word[k], epoch) == 0 && spins < kSpinLimit) {
                __builtin_amdgcn_s_sleep(1);
                word[k] = __hip_atomic_load(&states[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                spins++;
            }
            const uint32_t flag = stamp_flag(word[k], epoch);
            if (flag == 0) timed_out = true;
            const uint64_t inclusive_lanes = __builtin_amdgcn_ballot_w64(flag == 2);
            const int first = inclusive_lanes ? __builtin_ctzll(inclusive_lanes) : kWave;
            if (flag != 0 && lane <= first) sum += (uint32_t)word[k];
            done = inclusive_lanes != 0;
        }
        if (done) break;
    }
    const uint32_t prefix = wave_sum(sum);
    if (__builtin_amdgcn_ballot_w64(timed_out) && lane == 0) total_and_status[1] = epoch;
    if (lane == 0) {
        if (tile != 0) __hip_atomic_store(&states[tile], stamped(2u, epoch, prefix + tile_total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tile == n_tiles - 1) total_and_status[0] = prefix + tile_total;
    }
    return prefix;
}

__global__ __launch_bounds__(kScanThreads) void frame_scan_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                                  const int32_t *__restrict__ indices, int n_triangles, int W, int H,
                                                                  int tw, int th, int tiles_x, int tiles_y, uint32_t epoch,
                                                                  uint32_t *__restrict__ tri_offsets, real4 *__restrict__ records,
                                                                  uint32_t *total_and_status, uint32_t *ticket, uint64_t *states,
                                                                  int n_scan_tiles, uint32_t head_capacity, uint32_t *__restrict__ heads,
                                                                  uint32_t *totals, uint32_t *totals_next,
                                                                  real *__restrict__ edges, uint32_t *zero, size_t zero_words,
                                                                  uint32_t *clear_word) {
    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_wave_total[kScanThreads / kWave];
    __shared__ uint32_t s_tile_prefix;
    __shared__ uint32_t s_count[kScanTile];
    // difference arrays of the keys per tile column and per tile row: a triangle adds its rows at its first column
    // and takes them off behind its last one, likewise for the rows; the running sums are the digit counts
    __shared__ uint32_t s_diff[kEmitDigitPasses][kRadix + 1];
    __shared__ uint32_t s_digit_wave[kScanThreads / kWave];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    if (totals && tid <= kRadix)
        for (int p = 0; p < kEmitDigitPasses; p++) s_diff[p][tid] = 0;
    if (tid == 0) {
        uint32_t mine = blockIdx.x;  // no ticket: the whole grid is resident
        if (ticket) {
            mine = atomicAdd(ticket, 1u);
            if (mine == (uint32_t)n_scan_tiles - 1) atomicExch(ticket, 0u);  // all tickets are out: ready for the next call
        }
        s_tile = mine;
    }
    // side jobs: what the sort wants cleared, the other set of digit totals, the NDC edges of the tile columns and rows
    for (size_t i = (size_t)blockIdx.x * kScanThreads + tid; i < zero_words; i += (size_t)gridDim.x * kScanThreads) zero[i] = 0;
    if (blockIdx.x == 0) {
        if (totals_next && tid < kEmitDigitPasses * kRadix) totals_next[tid] = 0;
        if (clear_word && tid == 0) *clear_word = 0;
        // render.cu:243-246: the edges of tile column tx are entries tx and tx + 1
        for (int i = tid; i <= tiles_x; i += kScanThreads) edges[i] = (real)(i * tw) / (real)W * 2.0f - 1.0f;
        for (int i = tid; i <= tiles_y; i += kScanThreads) edges[tiles_x + 1 + i] = (real)(i * th) / (real)H * 2.0f - 1.0f;
    }
    lds_barrier();
    const int tile = (int)s_tile;
    const int64_t base = (int64_t)tile * kScanTile + (int64_t)tid * 4;

    // Triangle by triangle across the lanes (neighbouring lanes take neighbouring triangles, so the index
    // loads and the record stores of a wave are contiguous); the counts then change hands through LDS so that
    // every thread scans four consecutive ones.
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t t = (int64_t)tile * kScanTile + k * kScanThreads + tid;
        uint32_t count = 0;
        Rect rect = {0, -1, 0, -1};
        if (t < n_triangles) {
            const TriXYZ p = load_triangle(vertices, n_vertices, indices, (int)t);
            const Rect r = tile_rect(p.ax, p.ay, p.bx, p.by, p.cx, p.cy, W, H, tw, th, tiles_x, tiles_y);
            count = rect_count(r);
            // render.cu:140-152 compute_plane
            const real det = p.ax * (p.by - p.cy) + p.bx * (p.cy - p.ay) + p.cx * (p.ay - p.by);
            const real id = (real)(1.0 / (double)det);
            const real A = (p.az * (p.by - p.cy) + p.bz * (p.cy - p.ay) + p.cz * (p.ay - p.by)) * id;
            const real B = (p.ax * (p.bz - p.cz) + p.bx * (p.cz - p.az) + p.cx * (p.az - p.bz)) * id;
            const real C = (p.ax * (p.by * p.cz - p.cy * p.bz) + p.bx * (p.cy * p.az - p.ay * p.cz) + p.cx * (p.ay * p.bz - p.by * p.az)) * id;
            records[t] = make_real4(A, B, C, int_in_real(r.x0));
            records[(int64_t)n_triangles + t] = make_real4(p.ax, p.ay, p.bx, p.by);
            records[2 * (int64_t)n_triangles + t] = make_real4(p.cx, p.cy, int_in_real(r.y0), int_in_real(r.y1 - r.y0 + 1));
            rect = r;
        }
        s_count[k * kScanThreads + tid] = count;
        if (totals && count) {
            const uint32_t nx = (uint32_t)(rect.x1 - rect.x0 + 1), ny = (uint32_t)(rect.y1 - rect.y0 + 1);
            atomicAdd(&s_diff[0][rect.x0], ny);
            atomicAdd(&s_diff[0][rect.x1 + 1], 0u - ny);
            atomicAdd(&s_diff[1][rect.y0], nx);
            atomicAdd(&s_diff[1][rect.y1 + 1], 0u - nx);
        }
    }
    lds_barrier();
    if (totals) {  // running sums of the difference arrays: waves 0..3 take the columns, 4..7 the rows
        static_assert(kScanThreads == kEmitDigitPasses * kRadix, "one thread per digit of the two passes");
        const int p = tid / kRadix, d = tid & (kRadix - 1);
        const uint32_t digit_incl = wave_inclusive_scan_u32(s_diff[p][d]);
        if (lane == kWave - 1) s_digit_wave[wave] = digit_incl;
        lds_barrier();
        uint32_t keys_of_digit = digit_incl;
        for (int w = p * (kRadix / kWave); w < wave; w++) keys_of_digit += s_digit_wave[w];
        if (keys_of_digit) atomicAdd(&totals[p * kRadix + d], keys_of_digit);
    }
    uint32_t x[4];
#pragma unroll
    for (int k = 0; k < 4; k++) x[k] = s_count[tid * 4 + k];
    const uint32_t thread_sum = x[0] + x[1] + x[2] + x[3];
    const uint32_t incl = wave_inclusive_scan_u32(thread_sum);
    if (lane == kWave - 1) s_wave_total[wave] = incl;
    lds_barrier();
    if (wave == 0) {
        uint32_t wt = (lane < kScanThreads / kWave) ? s_wave_total[lane] : 0u;
        uint32_t wincl = wave_inclusive_scan_u32(wt);
        uint32_t tile_total = (uint32_t)__builtin_amdgcn_readlane((int)wincl, kScanThreads / kWave - 1);
        if (lane < kScanThreads / kWave) s_wave_total[lane] = wincl - wt;  // exclusive wave offsets
        const uint32_t prefix = frame_tile_prefix(states, tile, tile_total, n_scan_tiles, epoch, total_and_status);
        if (lane == 0) s_tile_prefix = prefix;
    }
    lds_barrier();
    uint32_t run = s_tile_prefix + s_wave_total[wave] + (incl - thread_sum);
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t t = base + k;
        if (t >= n_triangles) break;
        tri_offsets[t] = run;
        if (x[k] != 0) {
            // triangle t owns the key positions [run, run + x): note for every multiple of kEmitChunk who owns it
            const uint32_t first = (run + kEmitChunk - 1) / kEmitChunk, last = (run + x[k] - 1) / kEmitChunk;
            for (uint32_t h = first; h <= last && h < head_capacity; h++) heads[h] = (uint32_t)t;
        }
        run += x[k];
    }
}

#ifndef TG_DOUBLE_PRECISION
__device__ __forceinline__ uint32_t dpp_max_u32_step(uint32_t v, uint32_t o) { return o > v ? o : v; }
template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    return dpp_max_u32_step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, 0xf, false));
}
__device__ __forceinline__ uint32_t wave_inclusive_max_u32(uint32_t v) {
    v = dpp_max_u32<0x111, 0xf>(v);
    v = dpp_max_u32<0x112, 0xf>(v);
    v = dpp_max_u32<0x114, 0xf>(v);
    v = dpp_max_u32<0x118, 0xf>(v);
    v = dpp_max_u32<0x142, 0xa>(v);
    v = dpp_max_u32<0x143, 0xc>(v);
    return v;
}

struct EmitLds {
    PolyLdsOf<kEmitThreads> poly;  // the polygon of the key a thread clips
    uint32_t owner[kEmitChunk];    // per key position of the chunk: first the marks of the triangles' first keys, then the owners
    uint16_t queue[kEmitChunk];    // the chunk's keys that need clipping, those with the most passes first
    uint32_t wave_owner[kEmitWaves];
    uint32_t bucket[4];            // keys of the chunk with 4, 3, 2, 1 passes to run
};

// What a key needs from its triangle's record and its position in the tile rectangle.
struct FrameKey {
    real A, B, C, ax, ay, bx, by, cx, cy;
    real xmin, xmax, ymin, ymax;  // render.cu:243-246 tile rectangle in NDC
    uint32_t tile_id;
};
__device__ __forceinline__ FrameKey frame_key(const real4 *__restrict__ records, int n_triangles, int t, uint32_t local,
                                              const real *__restrict__ edges, int tiles_x, int column_bits) {
    const real4 r0 = records[t], r1 = records[(int64_t)n_triangles + t], r2 = records[2 * (int64_t)n_triangles + t];
    FrameKey k;
    k.A = r0.x; k.B = r0.y; k.C = r0.z;
    k.ax = r1.x; k.ay = r1.y; k.bx = r1.z; k.by = r1.w; k.cx = r2.x; k.cy = r2.y;
    const uint32_t ny = (uint32_t)int_of_real(r2.w);
    // column = local / ny, row = local % ny (tile x outer, tile y inner, render.cu:235-236): the reciprocal
    // multiply is off by at most one for local < 2^21
    uint32_t col = (uint32_t)((float)local * __builtin_amdgcn_rcpf((float)ny));
    int row = (int)local - (int)(col * ny);
    if (row < 0) { col--; row += (int)ny; } else if (row >= (int)ny) { col++; row -= (int)ny; }
    const int tx = int_of_real(r0.w) + (int)col, ty = int_of_real(r2.z) + row;
    k.xmin = edges[tx]; k.xmax = edges[tx + 1];  // a few hundred scalars that every key reads: they stay in cache
    k.ymin = edges[tiles_x + 1 + ty]; k.ymax = edges[tiles_x + 2 + ty];
    // the key's high word: the tile number, or for the sort by column and row the pair ty << column_bits | tx
    k.tile_id = column_bits ? ((uint32_t)ty << column_bits) | (uint32_t)tx : (uint32_t)(ty * tiles_x + tx);
    return k;
}
// The clip passes that may change the key's polygon (bit b: pass b of render.cu:254-257), see above.
__device__ __forceinline__ uint32_t frame_key_passes(const FrameKey &k) {
    const real lo_x = min3(k.ax, k.bx, k.cx), hi_x = max3(k.ax, k.bx, k.cx);
    const real lo_y = min3(k.ay, k.by, k.cy), hi_y = max3(k.ay, k.by, k.cy);
    const real x_abs = abs_real(lo_x) > abs_real(hi_x) ? abs_real(lo_x) : abs_real(hi_x);
    const real y_abs = abs_real(lo_y) > abs_real(hi_y) ? abs_real(lo_y) : abs_real(hi_y);
    const real slack_x = x_abs * 1.9073486328125e-06f + 1e-37f, slack_y = y_abs * 1.9073486328125e-06f + 1e-37f;  // 2^-19
    uint32_t todo = 0;
    if (!(lo_x - slack_x >= k.xmin)) todo |= 1u;
    if (!(hi_x + slack_x <= k.xmax)) todo |= 2u;
    if (!(lo_y - slack_y >= k.ymin)) todo |= 4u;
    if (!(hi_y + slack_y <= k.ymax)) todo |= 8u;
    return todo;
}

__global__ __launch_bounds__(kEmitThreads) void frame_emit_kernel(const real4 *__restrict__ records, const uint32_t *__restrict__ tri_offsets,
                                                                  int n_triangles, const uint32_t *__restrict__ total_and_status,
                                                                  uint32_t key_capacity, const uint32_t *__restrict__ heads,
                                                                  uint32_t head_capacity, const real *__restrict__ edges, int tiles_x,
                                                                  int column_bits, uint64_t *__restrict__ keys,
                                                                  uint32_t *__restrict__ payload) {
    __shared__ EmitLds L;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const uint32_t total = total_and_status[0];
    const uint32_t n_keys = total < key_capacity ? total : key_capacity;  // keys beyond the buffers are left out
    const uint32_t k0 = blockIdx.x * (uint32_t)kEmitChunk;
    if (k0 >= n_keys) return;
    // The owners of the chunk's keys lie between the owner of its first key and the owner of the next chunk's
    // first key; the scan noted both (otherwise two uniform binary searches find them).
    int t_first, t_last;
    if (blockIdx.x < head_capacity) {
        t_first = (int)heads[blockIdx.x];
        t_last = (k0 + kEmitChunk < total && blockIdx.x + 1 < head_capacity) ? (int)heads[blockIdx.x + 1] : n_triangles - 1;
    } else {
        const uint32_t k_last = (k0 + kEmitChunk <= n_keys ? k0 + kEmitChunk : n_keys) - 1;
        t_first = owner_of_key(tri_offsets, n_triangles, k0);
        t_last = owner_of_key(tri_offsets, n_triangles, k_last);
    }
    const int span = t_last - t_first + 1;
    L.owner[tid] = 0;
    L.owner[kEmitThreads + tid] = 0;
    if (tid < 4) L.bucket[tid] = 0;
    lds_barrier();
    // every triangle of the span marks the position of its first key in the chunk with its number (+ 1); of
    // several triangles at one position (all but the last own no key) the last counts
    for (int i = tid; i < span; i += kEmitThreads) {
        const uint32_t off = tri_offsets[t_first + i];
        if (off < k0 + kEmitChunk) atomicMax(&L.owner[off > k0 ? off - k0 : 0u], (uint32_t)i + 1u);
    }
    lds_barrier();
    // a running maximum over the marks gives every key position its triangle
    {
        uint32_t m0 = L.owner[2 * tid], m1 = L.owner[2 * tid + 1];
        m1 = m1 > m0 ? m1 : m0;
        const uint32_t wmax = wave_inclusive_max_u32(m1);
        if (lane == kWave - 1) L.wave_owner[wave] = wmax;
        uint32_t before = (uint32_t)__shfl_up((int)wmax, 1, kWave);
        if (lane == 0) before = 0;
        lds_barrier();
        for (int w = 0; w < wave; w++) before = L.wave_owner[w] > before ? L.wave_owner[w] : before;
        L.owner[2 * tid] = m0 > before ? m0 : before;
        L.owner[2 * tid + 1] = m1 > before ? m1 : before;
    }
    lds_barrier();

    // every key of the chunk, neighbouring keys on neighbouring lanes: its tile and the passes it needs.  A key
    // that needs none is done here (its polygon is the triangle, render.cu:262-267); the others queue up by
    // their number of passes.
    uint32_t entry[kEmitKeys], slot[kEmitKeys];
#pragma unroll
    for (int k = 0; k < kEmitKeys; k++) {
        const uint32_t in_chunk = (uint32_t)k * kEmitThreads + tid, at = k0 + in_chunk;
        uint32_t e = 0, at_slot = 0;
        if (at < n_keys) {
            const uint32_t m = L.owner[in_chunk];
            const int t = t_first + (m ? (int)m - 1 : 0);  // every key position has a mark at or before it
            const FrameKey key = frame_key(records, n_triangles, t, at - tri_offsets[t], edges, tiles_x, column_bits);
            const uint32_t todo = frame_key_passes(key);
            if (todo == 0) {
                real md = std::numeric_limits<real>::max();
                real pd = key.A * key.ax + key.B * key.ay + key.C;  // render.cu:154-157
                md = (pd < md) ? pd : md;
                pd = key.A * key.bx + key.B * key.by + key.C;
                md = (pd < md) ? pd : md;
                pd = key.A * key.cx + key.B * key.cy + key.C;
                md = (pd < md) ? pd : md;
                keys[at] = ((uint64_t)key.tile_id << 32) | orderable_bits(md);
                payload[at] = (uint32_t)t;
            } else {
                e = 0x8000u | todo | (in_chunk << 4);
                at_slot = atomicAdd(&L.bucket[4 - __builtin_popcount(todo)], 1u);
            }
        }
        entry[k] = e;
        slot[k] = at_slot;
    }
    lds_barrier();
    const uint32_t b4 = L.bucket[0], b3 = L.bucket[1], b2 = L.bucket[2], b1 = L.bucket[3];
    const uint32_t queued = b4 + b3 + b2 + b1;
#pragma unroll
    for (int k = 0; k < kEmitKeys; k++)
        if (entry[k]) {
            const int passes = __builtin_popcount(entry[k] & 15u);
            const uint32_t first = passes == 4 ? 0u : passes == 3 ? b4 : passes == 2 ? b4 + b3 : b4 + b3 + b2;
            L.queue[first + slot[k]] = (uint16_t)entry[k];
        }
    lds_barrier();
    // the queue, 64 keys at a time per wave: neighbours run the same number of passes
#pragma unroll 1
    for (uint32_t q = (uint32_t)wave * kWave; q < queued; q += kEmitThreads) {
        if (q + lane >= queued) continue;
        const uint32_t e = L.queue[q + lane];
        const uint32_t in_chunk = (e >> 4) & (kEmitChunk - 1), at = k0 + in_chunk;
        uint32_t todo = e & 15u;
        const uint32_t m = L.owner[in_chunk];
        const int t = t_first + (m ? (int)m - 1 : 0);
        const FrameKey key = frame_key(records, n_triangles, t, at - tri_offsets[t], edges, tiles_x, column_bits);
        L.poly.x[0][tid] = key.ax; L.poly.y[0][tid] = key.ay;
        L.poly.x[1][tid] = key.bx; L.poly.y[1][tid] = key.by;
        L.poly.x[2][tid] = key.cx; L.poly.y[2][tid] = key.cy;
        int n = 3;
        while (todo) {
            const uint32_t b = (uint32_t)__builtin_ctz(todo);
            todo &= todo - 1;
            const real nx = b == 0 ? 1.0f : (b == 1 ? -1.0f : 0.0f), nyv = b == 2 ? 1.0f : (b == 3 ? -1.0f : 0.0f);
            const real d = b == 0 ? key.xmin : (b == 1 ? -key.xmax : (b == 2 ? key.ymin : -key.ymax));
            n = clip_pass(L.poly, n, nx, nyv, d);
            if (n <= 0) todo = 0;
        }
        real depth = kFarKey;  // render.cu:259
        if (n > 0) {
            real md = std::numeric_limits<real>::max();
            for (int i = 0; i < n; i++) {
                const real pd = key.A * L.poly.x[i][tid] + key.B * L.poly.y[i][tid] + key.C;  // render.cu:154-157
                md = (pd < md) ? pd : md;
            }
            depth = md;
        }
        keys[at] = ((uint64_t)key.tile_id << 32) | orderable_bits(depth);
        payload[at] = (uint32_t)t;
    }
}
#endif  // !TG_DOUBLE_PRECISION


// Lower bounds of the per-pixel depths (render.cu:404: interpolate3 of the vertex z with the vertex w
// as weights) of the rest of every tile list, per batch of kBoundSpan entries.  With positive finite
// weights the interpolated depth is a convex combination of the three vertex depths, so it cannot lie
// below their minimum by more than the rounding of the few operations involved; 32 ulps of the largest
// |z| are subtracted for that.  An entry with a weight that is not positive and finite bounds nothing
// (-inf).  Entries whose sort key is 1e30 (empty clipped polygon, render.cu:259) sit at the end of the
// list whatever their depth: the bounds leave them out, far_start[tile] is the position of the first
// one (the list length if there is none), and the reader looks at everything from there on.  The
// double build's sorted keys no longer hold the depth, so nothing is left out there.
// A first kernel writes every triangle's own bound; then one workgroup per tile: its waves take the
// batches in turn and write each batch's own minimum, and the first wave turns those into minima over
// the rest of the list, walking from the far end.
constexpr int kBoundThreads = 256;

__global__ __launch_bounds__(kBinThreads) void triangle_low_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                                   const int32_t *__restrict__ indices, int n_triangles,
                                                                   real *__restrict__ triangle_low) {
    const int t = blockIdx.x * kBinThreads + threadIdx.x;
    if (t >= n_triangles) return;
    const real inf = std::numeric_limits<real>::infinity();
    const int id[3] = {indices[3 * (int64_t)t], indices[3 * (int64_t)t + 1], indices[3 * (int64_t)t + 2]};
    real zmin = inf, zabs = 0.0f;
    bool ok = true;
#pragma unroll
    for (int k = 0; k < 3; k++) {
        ok = ok && (unsigned)id[k] < (unsigned)n_vertices;
        const real4 v = ok ? vertices[id[k]] : make_real4(0.f, 0.f, 0.f, 0.f);
        ok = ok && v.w > 0.0f && v.w < inf && abs_real(v.z) < inf;  // false for NaN as well
        zmin = (v.z < zmin) ? v.z : zmin;
        zabs = (abs_real(v.z) > zabs) ? abs_real(v.z) : zabs;
    }
    triangle_low[t] = ok ? zmin - 32.0f * std::numeric_limits<real>::epsilon() * zabs : -inf;
}

__global__ __launch_bounds__(kBoundThreads) void list_bounds_kernel(const real *__restrict__ triangle_low, int n_triangles,
                                                                    const uint64_t *__restrict__ sorted_keys,
                                                                    const int32_t *__restrict__ sorted_ids,
                                                                    const int32_t *__restrict__ offsets,
                                                                    real *__restrict__ bounds, int32_t *__restrict__ far_start) {
    __shared__ int s_far;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int tile = blockIdx.x;
    const int start = offsets[tile], n = offsets[tile + 1] - start;
    const int n_batches = (n + kBoundSpan - 1) / kBoundSpan;
    const real inf = std::numeric_limits<real>::infinity();
    if (threadIdx.x == 0) s_far = n;
    __syncthreads();
    for (int b = wave; b < n_batches; b += kBoundThreads / kWave) {
        real low = inf;
        bool any_far = false;
        int first_far = n;
#pragma unroll
        for (int c = kBoundSpan / kWave - 1; c >= 0; c--) {
            const int p = b * kBoundSpan + c * kWave + lane;
            real lb = inf;
            bool far = false;
            if (p < n) {
#ifndef TG_DOUBLE_PRECISION
                far = (uint32_t)sorted_keys[start + p] == orderable_bits(kFarKey);
#endif
                const int t = sorted_ids[start + p];
                lb = far ? inf : ((unsigned)t < (unsigned)n_triangles ? triangle_low[t] : -inf);
            }
            const uint64_t far_lanes = __builtin_amdgcn_ballot_w64(far);
            if (far_lanes) {
                any_far = true;
                first_far = b * kBoundSpan + c * kWave + __builtin_ctzll(far_lanes);
            }
            low = (lb < low) ? lb : low;
        }
        low = wave_min(low);
        if (lane == 0) {
            bounds[batch_bound_index(start, tile, b * kBoundSpan)] = low;
            if (any_far) atomicMin(&s_far, first_far);
        }
    }
    __threadfence_block();
    __syncthreads();
    if (wave != 0) return;
    real rest = inf;  // bound of everything behind the batches in hand
    for (int hi = n_batches; hi > 0; hi -= kWave) {
        const int b = hi - 1 - lane;  // lane 0 holds the farthest batch
        real v = (b >= 0) ? bounds[batch_bound_index(start, tile, b * kBoundSpan)] : inf;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const real o = __shfl_up(v, d);
            if (lane >= d) v = (o < v) ? o : v;
        }
        v = (rest < v) ? rest : v;
        if (b >= 0) bounds[batch_bound_index(start, tile, b * kBoundSpan)] = v;
        rest = __shfl(v, kWave - 1);
    }
    if (lane == 0) far_start[tile] = s_far;
}

// render.cu:310-337 cartesian_to_bary_kernel.
__global__ __launch_bounds__(kBinThreads) void bary_kernel(const real4 *__restrict__ vertices, int n_vertices,
                                                           const int32_t *__restrict__ indices, int n_triangles,
                                                           real *__restrict__ out) {
    const int t = blockIdx.x * kBinThreads + threadIdx.x;
    if (t >= n_triangles) return;
    const TriXYZ p = load_triangle(vertices, n_vertices, indices, t);
    real denom = p.ax * (p.by - p.cy) + p.bx * (p.cy - p.ay) + p.cx * (p.ay - p.by);
    if (abs_real(denom) < kEffZero) denom = 1.0f;
    real *m = out + 9 * (int64_t)t;
    m[0] = (p.by - p.cy) / denom;
    m[1] = (p.cx - p.bx) / denom;
    m[2] = (p.bx * p.cy - p.cx * p.by) / denom;
    m[3] = (p.cy - p.ay) / denom;
    m[4] = (p.ax - p.cx) / denom;
    m[5] = (p.cx * p.ay - p.ax * p.cy) / denom;
    m[6] = (p.ay - p.by) / denom;
    m[7] = (p.bx - p.ax) / denom;
    m[8] = (p.ax * p.by - p.bx * p.ay) / denom;
}

static int check_geometry(const char *fn, const void *vertices, int n_vertices, const void *indices, int n_triangles, int W, int H,
                          int tw, int th) {
    if (n_triangles < 0 || n_vertices < 0 || W <= 0 || H <= 0 || tw <= 0 || th <= 0 || (n_triangles > 0 && (!vertices || !indices))) {
        set_error("%s: null pointer, negative count or non-positive image/tile size", fn);
        return TG_E_ARG;
    }
    if ((uintptr_t)vertices & 15) {
        set_error("%s: vertices must be 16-byte aligned", fn);
        return TG_E_ARG;
    }
    return 0;
}

}  // namespace tg

using namespace tg;

extern "C" int tg_bin_count(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width, int height, int tile_w,
                            int tile_h, uint32_t *tri_counts, void *stream) {
    if (int e = check_geometry("tg_bin_count", vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h)) return e;
    if (n_triangles == 0) return 0;
    if (!tri_counts) { set_error("tg_bin_count: tri_counts is null"); return TG_E_ARG; }
    TG_LAUNCH(bin_count_kernel, dim3(ceil_div(n_triangles, kBinThreads)), dim3(kBinThreads), 0, (hipStream_t)stream,
                       (const real4 *)vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h,
                       ceil_div(width, tile_w), ceil_div(height, tile_h), tri_counts);
    return check_launch("bin_count_kernel");
}

extern "C" int tg_bin_emit(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width, int height, int tile_w,
                           int tile_h, const uint32_t *tri_offsets, int64_t n_keys, const uint32_t *owner_heads,
                           uint32_t owner_capacity, uint64_t *keys, uint32_t *payload, void *stream) {
    if (int e = check_geometry("tg_bin_emit", vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h)) return e;
    if (n_keys < 0 || n_keys > 0xffffffffll) { set_error("tg_bin_emit: n_keys out of range"); return TG_E_ARG; }
    if (n_keys == 0) return 0;
    if (n_triangles == 0 || !tri_offsets || !keys || !payload) { set_error("tg_bin_emit: null pointer"); return TG_E_ARG; }
    TG_LAUNCH(bin_emit_kernel, dim3((unsigned)ceil_div64(n_keys, kBinThreads)), dim3(kBinThreads), 0, (hipStream_t)stream,
                       (const real4 *)vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h,
                       ceil_div(width, tile_w), ceil_div(height, tile_h), tri_offsets, n_keys, owner_heads, owner_capacity, keys,
                       payload);
    return check_launch("bin_emit_kernel");
}

extern "C" int tg_bary(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, real *out,
                       void *stream) {
    if (int e = check_geometry("tg_bary", vertices, n_vertices, indices, n_triangles, 1, 1, 1, 1)) return e;
    if (n_triangles == 0) return 0;
    if (!out) { set_error("tg_bary: out is null"); return TG_E_ARG; }
    TG_LAUNCH(bary_kernel, dim3(ceil_div(n_triangles, kBinThreads)), dim3(kBinThreads), 0, (hipStream_t)stream,
                       (const real4 *)vertices, n_vertices, indices, n_triangles, out);
    return check_launch("bary_kernel");
}

extern "C" size_t tg_list_bound_words(int64_t n_keys, int n_tiles) {
    if (n_keys < 0 || n_tiles <= 0) return 0;
    return (size_t)(n_keys / kBoundSpan + n_tiles + 1);
}

extern "C" int tg_list_bounds(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles,
                              const uint64_t *sorted_keys, const int32_t *sorted_ids, const int32_t *offsets, int n_tiles,
                              real *triangle_low, real *bounds, int32_t *far_start, void *stream) {
    if (n_tiles <= 0 || n_vertices < 0 || n_triangles < 0 || !offsets || !bounds || !far_start || ((uintptr_t)vertices & 15) ||
        (n_triangles > 0 && (!vertices || !indices || !triangle_low))) {
        set_error("tg_list_bounds: null pointer, non-positive tile count or misaligned vertices");
        return TG_E_ARG;
    }
    if (n_triangles > 0) {
        TG_LAUNCH(triangle_low_kernel, dim3(ceil_div(n_triangles, kBinThreads)), dim3(kBinThreads), 0, (hipStream_t)stream,
                  (const real4 *)vertices, n_vertices, indices, n_triangles, triangle_low);
        if (int e = check_launch("triangle_low_kernel")) return e;
    }
    TG_LAUNCH(list_bounds_kernel, dim3(n_tiles), dim3(kBoundThreads), 0, (hipStream_t)stream, triangle_low, n_triangles,
              sorted_keys, sorted_ids, offsets, bounds, far_start);
    return check_launch("list_bounds_kernel");
}

extern "C" size_t tg_bin_setup_workspace_bytes(int32_t n_triangles, int width, int height, int tile_w, int tile_h) {
    if (n_triangles < 0 || width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0) return 0;
    return frame_state(nullptr, n_triangles, ceil_div(width, tile_w), ceil_div(height, tile_h)).bytes;
}

extern "C" int tg_bin_setup(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width,
                            int height, int tile_w, int tile_h, uint32_t *tri_offsets, real *records, uint32_t *total_and_status,
                            uint32_t head_capacity, uint32_t *heads, void *frame, size_t frame_bytes, void *stream) {
    if (int e = check_geometry("tg_bin_setup", vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h)) return e;
    if (!total_and_status || !frame || ((uintptr_t)frame & 255) || (n_triangles > 0 && (!tri_offsets || !records)) ||
        ((uintptr_t)records & (4 * sizeof(real) - 1))) {
        set_error("tg_bin_setup: null pointer, frame state not 256-byte aligned or records not aligned to four scalars");
        return TG_E_ARG;
    }
    const int tiles_x = ceil_div(width, tile_w), tiles_y = ceil_div(height, tile_h);
    const FrameState f = frame_state(frame, n_triangles, tiles_x, tiles_y);
    if (frame_bytes < f.bytes) {
        set_error("tg_bin_setup: frame state of %zu bytes, need %zu", frame_bytes, f.bytes);
        return TG_E_WORKSPACE;
    }
    hipStream_t s = (hipStream_t)stream;
    const int n_scan_tiles = (int)ceil_div64(n_triangles, kScanTile);
    const size_t zero_words = ((char *)f.edges - (char *)f.tickets) / 4;  // tickets, totals, scan states
    TG_LAUNCH(bin_init_kernel, dim3(1), dim3(1024), 0, s, f.tickets, zero_words, f.edges, width, height, tile_w, tile_h, tiles_x,
              tiles_y, total_and_status);
    if (int e = check_launch("bin_init_kernel")) return e;
    if (n_triangles == 0) return 0;
    static int resident_cache[kMaxDevices] = {0};
    uint32_t *ticket = f.tickets;
    if (n_scan_tiles <= resident_workgroups((const void *)bin_setup_kernel, kScanThreads, resident_cache)) ticket = nullptr;
    // the digits of the sort's tile passes are counted here, where every triangle's tile rectangle is at hand
    // (the double build sorts differently, and more than 65536 tiles take a third pass: no counts then)
    const PassPlan plan = tile_pass_plan(tiles_x * tiles_y);
    const bool count_digits = binning_counts_digits(tiles_x * tiles_y);
    TG_LAUNCH(bin_setup_kernel, dim3(n_scan_tiles), dim3(kScanThreads), 0, s, (const real4 *)vertices, n_vertices, indices, n_triangles,
              width, height, tile_w, tile_h, tiles_x, tiles_y, tri_offsets, (real4 *)records, total_and_status, total_and_status + 1,
              ticket, f.states, n_scan_tiles, head_capacity, heads, plan, count_digits ? f.totals : (uint32_t *)nullptr);
    return check_launch("bin_setup_kernel");
}

// ---- the frame's binning in one call ----
namespace tg {
struct FusedFrame {
    uint32_t *totals;  // two sets of kEmitDigitPasses * kRadix digit totals
    uint32_t *ticket;
    uint64_t *states;  // one word per kScanTile triangles
    real *edges;       // tiles_x + 1 column edges, then tiles_y + 1 row edges
    uint32_t *heads;   // the owner of every kEmitChunk-th key position
    uint32_t *tri_offsets;
    real4 *records;
    uint32_t head_capacity;
    size_t bytes;
};
static FusedFrame fused_frame(void *base, int64_t n_triangles, int64_t key_capacity, int tiles_x, int tiles_y) {
    FusedFrame f;
    char *p = (char *)base;
    size_t o = 0;
    const auto take = [&](size_t bytes) { char *at = p + o; o = (o + bytes + 255) & ~(size_t)255; return at; };
    f.totals = (uint32_t *)take((size_t)kFrameTotalsWords * 4);
    f.ticket = (uint32_t *)take(4);
    f.states = (uint64_t *)take((size_t)(ceil_div64(n_triangles, kScanTile) + 1) * 8);
    f.edges = (real *)take((size_t)(tiles_x + tiles_y + 2) * sizeof(real));
    f.head_capacity = (uint32_t)(key_capacity / kEmitChunk + 2);
    f.heads = (uint32_t *)take((size_t)f.head_capacity * 4);
    f.tri_offsets = (uint32_t *)take((size_t)n_triangles * 4);
    f.records = (real4 *)take((size_t)n_triangles * kRecordReals * sizeof(real));
    f.bytes = o;
    return f;
}
uint32_t *fused_frame_totals(void *frame, uint32_t epoch) { return (uint32_t *)frame + (epoch & 1u) * (kEmitDigitPasses * kRadix); }

__global__ void bin_frame_empty_kernel(uint32_t *total_and_status, uint32_t *clear_word) {
    if (threadIdx.x == 0) {
        total_and_status[0] = 0;
        if (clear_word) *clear_word = 0;
    }
}
}  // namespace tg

extern "C" int tg_bin_frame_supported(int width, int height, int tile_w, int tile_h) {
    if (sizeof(real) != 4 || width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0) return 0;
    const int64_t tiles_x = ceil_div(width, tile_w), tiles_y = ceil_div(height, tile_h);
    return tiles_x * tiles_y <= kFrameMaxTiles;
}

extern "C" size_t tg_bin_frame_workspace_bytes(int32_t n_triangles, int64_t key_capacity, int width, int height, int tile_w, int tile_h) {
    if (n_triangles < 0 || key_capacity < 0 || width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0) return 0;
    return fused_frame(nullptr, n_triangles, key_capacity, ceil_div(width, tile_w), ceil_div(height, tile_h)).bytes;
}

extern "C" int tg_bin_frame(const real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width,
                            int height, int tile_w, int tile_h, uint64_t *keys, uint32_t *values, int64_t key_capacity,
                            uint32_t *total_and_status, void *frame, size_t frame_bytes, uint32_t epoch, void *zero,
                            size_t zero_bytes, uint32_t *clear_word, void *stream) {
#ifdef TG_DOUBLE_PRECISION
    set_error("tg_bin_frame: the double build's depth keys take all 64 key bits; use tg_bin_setup and tg_build_tile_lists");
    return TG_E_ARG;
#else
    if (int e = check_geometry("tg_bin_frame", vertices, n_vertices, indices, n_triangles, width, height, tile_w, tile_h)) return e;
    if (!tg_bin_frame_supported(width, height, tile_w, tile_h)) {
        set_error("tg_bin_frame: more than %d tiles; use tg_bin_setup and tg_build_tile_lists", kFrameMaxTiles);
        return TG_E_ARG;
    }
    if (!total_and_status || !frame || ((uintptr_t)frame & 255) || key_capacity < 0 || key_capacity > kSortMaxN ||
        (key_capacity > 0 && (!keys || !values)) || ((uintptr_t)keys & 7) || ((uintptr_t)zero & 3) || (zero_bytes & 3) ||
        (zero_bytes > 0 && !zero) || (epoch & kEpochMask) == 0) {
        set_error("tg_bin_frame: null or misaligned pointer, key_capacity outside [0, 2^30), or an epoch whose low 30 bits are 0");
        return TG_E_ARG;
    }
    const int tiles_x = ceil_div(width, tile_w), tiles_y = ceil_div(height, tile_h);
    const FusedFrame f = fused_frame(frame, n_triangles, key_capacity, tiles_x, tiles_y);
    if (frame_bytes < f.bytes) {
        set_error("tg_bin_frame: frame state of %zu bytes, need %zu", frame_bytes, f.bytes);
        return TG_E_WORKSPACE;
    }
    hipStream_t s = (hipStream_t)stream;
    if (n_triangles == 0) {
        TG_LAUNCH(bin_frame_empty_kernel, dim3(1), dim3(64), 0, s, total_and_status, clear_word);
        return check_launch("bin_frame_empty_kernel");
    }
    const int n_scan_tiles = (int)ceil_div64(n_triangles, kScanTile);
    static int resident_cache[kMaxDevices] = {0};
    uint32_t *ticket = f.ticket;
    if (n_scan_tiles <= resident_workgroups((const void *)frame_scan_kernel, kScanThreads, resident_cache)) ticket = nullptr;
    const GridPlan grid = grid_plan(tiles_x, tiles_y);
    TG_LAUNCH(frame_scan_kernel, dim3(n_scan_tiles), dim3(kScanThreads), 0, s, (const real4 *)vertices, n_vertices, indices, n_triangles,
              width, height, tile_w, tile_h, tiles_x, tiles_y, epoch, f.tri_offsets, f.records, total_and_status, ticket, f.states,
              n_scan_tiles, f.head_capacity, f.heads, grid.on ? fused_frame_totals(frame, epoch) : (uint32_t *)nullptr,
              fused_frame_totals(frame, epoch + 1), f.edges, (uint32_t *)zero, zero_bytes / 4, clear_word);
    if (int e = check_launch("frame_scan_kernel")) return e;
    if (key_capacity == 0) return 0;
    // for every key position the buffers hold: the kernel reads K and the workgroups behind it leave at once
    TG_LAUNCH(frame_emit_kernel, dim3((unsigned)ceil_div64(key_capacity, kEmitChunk)), dim3(kEmitThreads), 0, s, f.records, f.tri_offsets,
              n_triangles, total_and_status, (uint32_t)key_capacity, f.heads, f.head_capacity, f.edges, tiles_x,
              grid.on ? grid.column_bits : 0, keys, values);
    return check_launch("frame_emit_kernel");
#endif
}

namespace tg {
// Launches the emission from records; it also clears zero_words words at `zero` (the look-back words of the
// sort that follows) and *clear_word.
int launch_emit_records(const char *fn, const real *records, const uint32_t *tri_offsets, int32_t n_triangles, int64_t n_keys,
                        uint32_t owner_capacity, const uint32_t *owner_heads, void *frame, int width, int height, int tile_w,
                        int tile_h, uint64_t *keys, uint32_t *payload, uint32_t *zero, size_t zero_words, uint32_t *clear_word,
                        hipStream_t s) {
    const int tiles_x = ceil_div(width, tile_w), tiles_y = ceil_div(height, tile_h);
    const FrameState f = frame_state(frame, n_triangles, tiles_x, tiles_y);
    const int64_t n_chunks = ceil_div64(n_keys, kBinThreads);
    const int chunks_per_group = 1;  // more (fewer, longer-lived workgroups) measured slower: 52 against 47 us on 2.2 M keys
    const unsigned grid = (unsigned)ceil_div64(n_chunks, chunks_per_group);
    TG_LAUNCH(bin_emit_records_kernel, dim3(grid), dim3(kBinThreads), 0, s, (const real4 *)records, tri_offsets, n_triangles, n_keys,
              owner_heads, owner_capacity, f.edges, tiles_x, tiles_y, keys, payload, zero, zero_words, clear_word,
              zero ? f.tickets + kSweepTicketWord : (uint32_t *)nullptr, chunks_per_group);
    return check_launch(fn);
}
uint32_t *frame_totals(void *frame, int32_t n_triangles, int tiles_x, int tiles_y) { return frame_state(frame, n_triangles, tiles_x, tiles_y).tickets + kStateTicketWords; }
uint32_t *frame_tickets(void *frame) { return (uint32_t *)frame; }
}  // namespace tg
