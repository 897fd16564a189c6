// tg_forward.hip -- forward rasterize-and-blend, one workgroup per tile.
//
// per_pixel_sort = 0 (tile order): the sorted tile list is staged into LDS in
//   batches of 128 records; each pixel composites front to back and stops as
//   soon as its transmittance falls to the threshold or max_layers fragments
//   are blended; the workgroup leaves the list when every pixel has stopped.
// per_pixel_sort = 1: each pixel repeatedly selects its next (up to 32) nearest
//   fragments in (pixel depth, list position) order by scanning the whole list
//   (records staged through LDS as above, candidate lists in LDS, slot-major),
//   then blends them; threshold and max_layers are tested between selections
//   only, as in the reference (render.cu:588).
//
// Not HBM-bound: per (pixel, entry) pair ~12 VALU operations and three
// broadcast LDS reads against 148 B of gathered data per ENTRY.
#include "tg_raster.hpp"

namespace tg {

struct ForwardOut {
    real4 *image;
    real *depthmap;
    real *weights;
    int32_t *ends;
    int32_t *last;
    real *last_depth;
    // Blend order, may be null: 2 * max_layers planes of H * W 16-bit words.  Plane l holds the low half of the
    // list position (relative to the tile's start) of every pixel's layer l; plane max_layers + l the high half,
    // written and read only in tiles whose list is longer than kShortList.
    uint16_t *fragments;
    uint64_t *hit_masks; // tile order: which list entries cover which pixel, 64 entries per word (see hit_mask_chunk); may be null
    const uint32_t *list_status;  // status word of the kernels that made the lists (TG_STATUS_*); may be null
};

// Lists whose sort gave up a wait are not to be read (unwritten entries may name anything): the frame's pixels
// are marked instead, so that the caller sees it in the image itself.
__device__ __forceinline__ bool lists_invalid(const ForwardOut &o) { return o.list_status && *o.list_status != TG_STATUS_OK; }
__device__ __forceinline__ void mark_pixel_invalid(const ForwardOut &o, const PixelCoord &p) {
    if (!p.valid) return;
    const real nan = std::numeric_limits<real>::quiet_NaN();
    o.image[p.index] = make_real4(nan, nan, nan, nan);
    o.depthmap[p.index] = nan;
    o.weights[p.index] = 0.0f;
    o.ends[p.index] = 0;
    if (o.last) o.last[p.index] = 0;
    if (o.last_depth) o.last_depth[p.index] = nan;
}

__device__ __forceinline__ void write_pixel(const ForwardOut &o, const PixelCoord &p, PixelState s, int last, real last_depth) {
    // render.cu:609-618
    real depth;
    if (s.weight > kEffZero) {
        depth = s.depth / s.weight;
    } else {
        depth = __builtin_inff();
        s.weight = 0.0f;
    }
    o.depthmap[p.index] = depth;
    o.weights[p.index] = s.weight;
    o.ends[p.index] = s.blended;
    if (o.last) o.last[p.index] = last;
    if (o.last_depth) o.last_depth[p.index] = last_depth;
    o.image[p.index] = make_real4(s.c0, s.c1, s.c2, s.alpha);
}

__global__ __launch_bounds__(kTileThreads) void forward_tile_order_kernel(RasterArgs a, ForwardOut out) {
    __shared__ BlendRecord s_rec[kBatch];
    __shared__ uint8_t s_touch[kBatch];
    __shared__ WaveRect s_rects[kMaxTileWaves];
    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int n_waves = blockDim.x / kWave;
    const TileId tile_id = tile_of_workgroup<kTileBandForward>();
    const int tile = tile_id.index;
    const PixelCoord p = pixel_of_thread(a, tile_id);
    if (lists_invalid(out)) {  // the same for the whole launch
        mark_pixel_invalid(out, p);
        return;
    }
    const int start = a.offsets[tile], end = a.offsets[tile + 1];
    publish_wave_rect(p, s_rects);
    uint64_t *const masks = out.hit_masks ? out.hit_masks + hit_mask_head_words() : nullptr;

    PixelState s;
    int last = 0;
    for (int batch = start; batch < end; batch += kBatch) {
        const bool running = p.valid && s.alpha > a.thr && s.blended < a.max_layers;
        if (!__syncthreads_or(running)) break;
        const int nb = min(kBatch, end - batch);
        for (int e = tid; e < nb; e += blockDim.x) {
            gather_blend(a, batch + e, s_rec[e]);
            s_touch[e] = (uint8_t)waves_touched(s_rec[e].m, s_rects, n_waves);
        }
        __syncthreads();
        // 1. inside tests; a lane keeps its hits as a 256-bit mask
        uint64_t m[kBatch / kWave];
        batch_hit_mask<kBatch / kWave>(s_rec, s_touch, nb, wave, p.px, p.py, m);
        if (!running) {
#pragma unroll
            for (int wd = 0; wd < kBatch / kWave; wd++) m[wd] = 0;
        }
        if (masks) {
            // kept for the backward pass, which then has no inside test to repeat
            const int64_t chunk = hit_mask_chunk(start, tile, batch - start);
            const int64_t slots = (int64_t)gridDim.z * blockDim.x, slot = (int64_t)blockIdx.z * blockDim.x + tid;
#pragma unroll
            for (int wd = 0; wd < kBatch / kWave; wd++)
                if (wd * kWave < nb) masks[(chunk + wd) * slots + slot] = m[wd];
        }
        // 2. every lane composites its own hits in list order, so the blend arithmetic
        //    runs with as many lanes busy as there are pixels with a fragment left
        while (true) {
            int e = -1;
            if (s.alpha > a.thr && s.blended < a.max_layers) e = pop_lowest<kBatch / kWave>(m);  // render.cu:578, tested before every fragment
            if (__builtin_amdgcn_ballot_w64(e >= 0) == 0) break;  // wave-uniform
            if (e >= 0) {
                const BlendRecord &r = s_rec[e];
                real b0, b1, b2;
                bary_apply(r.m, p.px, p.py, b0, b1, b2);
                blend_fragment(s, r, b0, b1, b2);
                last = batch + e - start + 1;
            }
        }
    }
    if (p.valid) write_pixel(out, p, s, last, 0.0f);
    if (out.hit_masks) {
        // how far into the list this workgroup's pixels got
        __shared__ int s_last;
        __syncthreads();
        if (tid == 0) s_last = 0;
        __syncthreads();
        int wave_last = p.valid ? last : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) wave_last = max(wave_last, __shfl_xor(wave_last, off, kWave));
        if ((tid & (kWave - 1)) == 0 && wave_last > 0) atomicMax(&s_last, wave_last);
        __syncthreads();
        if (tid == 0) out.hit_masks[hit_mask_head_index(tile)] = (uint64_t)s_last;
    }
}

// render.cu:338-373 insert_sorted_topk on an LDS candidate list of capacity `cap`.
template <typename Pos>
__device__ __forceinline__ void topk_insert(const TopKOf<Pos> &tk, int cap, int &n, real d, int j) {
    if (n == cap && d >= tk.d(cap - 1)) return;
    int i = (n < cap) ? n : cap - 1;
    while (i > 0 && d < tk.d(i - 1)) {
        tk.d(i) = tk.d(i - 1);
        tk.j(i) = tk.j(i - 1);
        i--;
    }
    tk.d(i) = d;
    tk.j(i) = (Pos)j;
    if (n < cap) n++;
}

constexpr int kSelectBatch = 128;       // list entries staged per batch where positions take an int
constexpr int kSelectBatchShort = 64;   // ... and where they take 16 bits
constexpr int kShortList = 0xffff;      // longest tile list whose positions fit 16 bits
constexpr int kLongListGroups = 256;    // workgroups that look for the tiles with longer lists

// The per-pixel-order forward pass of one tile.  Pos: how a candidate's list position (from the tile's
// start) is kept.  With uint16_t the candidate lists of a 16x16 tile take 48 KB instead of 64 KB, which
// together with 64 staged entries lets a CU hold three workgroups instead of two.
template <int kStage, typename Pos>  // kStage: list entries staged per batch
__device__ __forceinline__ void pixel_order_tile(const RasterArgs &a, const ForwardOut &out, int tile_x, int tile_y, int tiles_x,
                                                 unsigned char *s_dyn, uint8_t *s_touch, WaveRect *s_rects) {
    const int n_threads = blockDim.x;
    DepthRecord *s_rec = reinterpret_cast<DepthRecord *>(s_dyn);
    TopKOf<Pos> tk;
    tk.depth = reinterpret_cast<real *>(s_dyn + sizeof(DepthRecord) * kStage);
    tk.pos = reinterpret_cast<Pos *>(tk.depth + kLayers * n_threads);
    tk.n_threads = n_threads;

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int n_waves = blockDim.x / kWave;
    const int tile = tile_y * tiles_x + tile_x;
    const int start = a.offsets[tile], end = a.offsets[tile + 1];
    const PixelCoord p = pixel_of_thread(a, tile_x, tile_y);
    publish_wave_rect(p, s_rects);

    PixelState s;
    real last_depth = -__builtin_inff();  // render.cu:585-586
    int last_j = -1;  // list positions count from the tile's start
    bool active = p.valid;
    while (true) {
        const bool want = active && s.alpha > a.thr && s.blended < a.max_layers;  // render.cu:588
        if (!__syncthreads_or(want)) break;
        const int cap = want ? min(kLayers, a.max_layers - s.blended) : 0;
        int found = 0;
        // The records of the next batch are fetched into registers while this batch is worked on: the
        // chain of dependent loads (list -> indices -> vertices, matrix) of a batch takes as long as its
        // inside tests, and with two workgroups per CU nothing else would cover it.  (Not with depth
        // bounds, which make the batches jump.)
        const bool ahead = !a.batch_bounds && (int)blockDim.x >= kStage;
        DepthRecord fetched;
        if (ahead && tid < min(kStage, end - start)) gather_depth(a, start + tid, fetched);
        for (int batch = start; batch < end; batch += kStage) {
            const int nb = min(kStage, end - batch);
            if (a.batch_bounds) {
                // a lane needs nothing from here on when its list is full and its worst candidate is nearer than
                // every fragment the rest of the tile's list can produce (a full list rejects depths >= its worst)
                const real rest = a.batch_bounds[batch_bound_index(start, tile, batch - start)];
                const bool settled = !want || (found == cap && tk.d(cap - 1) <= rest);
                if (__syncthreads_and(settled)) {
                    // on to the batch that holds the first entry the bounds do not cover
                    const int resume = start + a.far_start[tile] / kStage * kStage;
                    if (resume > batch) {
                        batch = resume - kStage;
                        continue;
                    }
                }
            }
            __syncthreads();
            if (ahead) {
                if (tid < nb) {
                    s_rec[tid] = fetched;
                    s_touch[tid] = (uint8_t)waves_touched(fetched.m, s_rects, n_waves);
                }
            } else {
                for (int e = tid; e < nb; e += blockDim.x) {
                    gather_depth(a, batch + e, s_rec[e]);
                    s_touch[e] = (uint8_t)waves_touched(s_rec[e].m, s_rects, n_waves);
                }
            }
            __syncthreads();
            if (ahead && batch + kStage < end && tid < min(kStage, end - batch - kStage)) gather_depth(a, batch + kStage + tid, fetched);
            // inside tests into a per-lane mask, then every lane visits its own hits in
            // list order (the order insert_sorted_topk sees them in the reference)
            uint64_t m[kStage / kWave];
            batch_hit_mask<kStage / kWave>(s_rec, s_touch, nb, wave, p.px, p.py, m);
            if (!want) {
#pragma unroll
                for (int wd = 0; wd < kStage / kWave; wd++) m[wd] = 0;
            }
            while (true) {
                const int e = pop_lowest<kStage / kWave>(m);
                if (__builtin_amdgcn_ballot_w64(e >= 0) == 0) break;  // wave-uniform
                if (e < 0) continue;
                const DepthRecord &r = s_rec[e];
                real b0, b1, b2;
                bary_apply(r.m, p.px, p.py, b0, b1, b2);
                const real pd = interp_w(b0, b1, b2, r.z[0], r.z[1], r.z[2], r.w[0], r.w[1], r.w[2]);  // render.cu:404
                const int j = batch + e - start;
                if (pd < last_depth) continue;
                if (pd == last_depth && j <= last_j) continue;
                topk_insert(tk, cap, found, pd, j);
            }
        }
        // Selection is over: the staging area and the depth lists are dead apart from
        // the depth of the last fragment each lane is going to blend.  The space takes
        // the blend records of the first list entries (rows an odd number of words
        // apart: lanes reading different entries use different banks); entries
        // beyond it are gathered from memory.
        const int todo = (want && found > 0) ? min(found, a.max_layers - s.blended) : 0;
        const real todo_depth = todo > 0 ? tk.d(todo - 1) : 0.0f;
        __syncthreads();
        real *rows = reinterpret_cast<real *>(s_dyn);
        const int n_rows = min(end - start, (int)((sizeof(DepthRecord) * kStage + sizeof(real) * kLayers * n_threads) /
                                                   (sizeof(real) * kBlendWords)));
        for (int e = tid; e < n_rows; e += blockDim.x) {
            BlendRecord r;
            gather_blend(a, start + e, r);
            const real *w = reinterpret_cast<const real *>(&r);
#pragma unroll
            for (int k = 0; k < kBlendWords; k++) rows[e * kBlendWords + k] = w[k];
        }
        __syncthreads();
        if (want) {
            if (found == 0) {
                active = false;  // render.cu:594
            } else {
                // kGatherAhead records are fetched together: the chains of dependent loads
                // (list -> indices -> vertices) of those that come from memory overlap
                for (int i0 = 0; i0 < todo; i0 += kGatherAhead) {
                    BlendRecord r[kGatherAhead];
#pragma unroll
                    for (int u = 0; u < kGatherAhead; u++) {
                        const int rel = tk.j(min(i0 + u, todo - 1));
                        if (rel < n_rows) {
                            real *w = reinterpret_cast<real *>(&r[u]);
#pragma unroll
                            for (int k = 0; k < kBlendWords; k++) w[k] = rows[rel * kBlendWords + k];
                        } else {
                            gather_blend(a, start + rel, r[u]);
                        }
                    }
#pragma unroll
                    for (int u = 0; u < kGatherAhead; u++) {
                        if (i0 + u >= todo) break;
                        real b0, b1, b2;
                        bary_apply(r[u].m, p.px, p.py, b0, b1, b2);
                        if (!bary_inside(b0, b1, b2)) continue;  // cannot happen: the selection tested it
                        if (out.fragments) {
                            const int64_t plane = (int64_t)a.W * a.H, at = (int64_t)s.blended * plane + p.index;
                            const int rel = tk.j(i0 + u);
                            out.fragments[at] = (uint16_t)rel;
                            if (sizeof(Pos) > sizeof(uint16_t) && end - start > kShortList)
                                out.fragments[(int64_t)a.max_layers * plane + at] = (uint16_t)(rel >> 16);
                        }
                        blend_fragment(s, r[u], b0, b1, b2);
                    }
                }
                last_depth = todo_depth;
                last_j = tk.j(todo - 1);
                // fewer candidates than asked for: the list is exhausted, the next
                // selection would return nothing (render.cu:594)
                if (found < cap) active = false;
            }
        }
    }
    if (p.valid) write_pixel(out, p, s, last_j + 1, last_depth);
}

// One workgroup per tile.  With 16-bit positions the tiles whose lists are too long for them are left to
// forward_pixel_order_long_lists_kernel.
template <int kStage, typename Pos>
__global__ __launch_bounds__(kTileThreads) void forward_pixel_order_kernel(RasterArgs a, ForwardOut out) {
    extern __shared__ __align__(16) unsigned char s_dyn[];
    __shared__ uint8_t s_touch[kStage];
    __shared__ WaveRect s_rects[kMaxTileWaves];
    const TileId tile = tile_of_workgroup<kTileBandForward>();
    if (lists_invalid(out)) {  // the same for the whole launch
        mark_pixel_invalid(out, pixel_of_thread(a, tile));
        return;
    }
    if (sizeof(Pos) < sizeof(int) && a.offsets[tile.index + 1] - a.offsets[tile.index] > kShortList) return;
    pixel_order_tile<kStage, Pos>(a, out, tile.x, tile.y, gridDim.x, s_dyn, s_touch, s_rects);
}

// The tiles whose lists are longer than kShortList, with int positions: few or none, so a small grid
// looks through the tiles' list lengths (a workgroup through its share of the tiles, one tile per thread at a
// time) and takes those.
__global__ __launch_bounds__(kTileThreads) void forward_pixel_order_long_lists_kernel(RasterArgs a, ForwardOut out, int tiles_x,
                                                                                      int tiles_y) {
    extern __shared__ __align__(16) unsigned char s_dyn[];
    __shared__ uint8_t s_touch[kSelectBatch];
    __shared__ WaveRect s_rects[kMaxTileWaves];
    __shared__ uint64_t s_votes[kMaxTileWaves];
    if (lists_invalid(out)) return;  // the launch before this one has marked every pixel
    const int tiles = tiles_x * tiles_y;
    const int share = (tiles + (int)gridDim.x - 1) / (int)gridDim.x;
    const int first = blockIdx.x * share, past = min(first + share, tiles);
    const int n_waves = blockDim.x / kWave;
    for (int base = first; base < past; base += blockDim.x) {
        const int mine = base + (int)threadIdx.x;
        const bool is_long = mine < past && a.offsets[mine + 1] - a.offsets[mine] > kShortList;
        const uint64_t vote = __builtin_amdgcn_ballot_w64(is_long);
        __syncthreads();  // the round before is done with the votes
        if ((threadIdx.x & (kWave - 1)) == 0) s_votes[threadIdx.x / kWave] = vote;
        __syncthreads();
        for (int w = 0; w < n_waves; w++) {
            uint64_t todo = s_votes[w];
            while (todo) {  // the same for the whole workgroup
                const int tile = base + w * kWave + __builtin_ctzll(todo);
                todo &= todo - 1;
                __syncthreads();  // the tile before is done with the LDS
                pixel_order_tile<kSelectBatch, int>(a, out, tile % tiles_x, tile / tiles_x, tiles_x, s_dyn, s_touch, s_rects);
            }
        }
    }
}

TileLaunch tile_launch(int width, int height, int tile_w, int tile_h, int max_threads) {
    TileLaunch t;
    const int pixels = tile_w * tile_h;
    t.threads = min(ceil_div(pixels, kWave) * kWave, max_threads);
    t.grid = dim3(ceil_div(width, tile_w), ceil_div(height, tile_h), ceil_div(pixels, t.threads));
    return t;
}

// Workgroup size of the per-pixel-sort kernels.  Their candidate lists take
// 32 * (scalar + int) bytes of LDS per thread: 64 KB for the 256 threads of a
// 16x16 tile.  The selection kernels are bound by latency, so what counts is
// how many waves a CU holds: the forward kernel stages 128 list entries at a
// time (7.5 KB), two workgroups of 256 threads fit a CU.  Measured on the five
// configurations against 64, 192 and 256 staged entries and against tiles split
// over two workgroups of 128 threads or four of 64 (which stage every entry two
// or four times): 15 to 35 % faster than 256 entries and 128 threads.  The
// re-selecting backward kernel also keeps 43 KB of gradient sums.
// TRIGRAD_PIXEL_ORDER_THREADS (64, 128 or 256) overrides the workgroup size.
int pixel_order_threads(int preferred) {
    static int override = -1;
    if (override < 0) {
        override = 0;
        if (const char *e = getenv("TRIGRAD_PIXEL_ORDER_THREADS")) {
            const int x = atoi(e);
            if (x == 64 || x == 128 || x == 256) override = x;
        }
    }
    return override ? override : preferred;
}

size_t pixel_order_lds_bytes(int n_threads, int staged_entries, size_t position_bytes) {
    return sizeof(DepthRecord) * staged_entries + (size_t)kLayers * n_threads * (sizeof(real) + position_bytes);
}

int check_raster_args(const char *fn, int width, int height, int tile_w, int tile_h, int max_layers) {
    if (width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0 || tile_w * tile_h > kMaxTilePixels) {
        set_error("%s: image size must be positive and tile_w*tile_h in [1, %d]", fn, kMaxTilePixels);
        return TG_E_ARG;
    }
    if ((int64_t)width * height > 0x7fffffffll) {
        set_error("%s: image too large", fn);
        return TG_E_ARG;
    }
    if (max_layers <= 0) {
        set_error("%s: max_layers must be positive", fn);
        return TG_E_ARG;
    }
    return 0;
}

}  // namespace tg

using namespace tg;

extern "C" size_t tg_hit_mask_words(int64_t n_keys, int width, int height, int tile_w, int tile_h) {
    if (n_keys < 0 || width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0 || tile_w * tile_h > kMaxTilePixels) return 0;
    const TileLaunch tl = tile_launch(width, height, tile_w, tile_h, kTileThreads);
    const int64_t tiles = (int64_t)tl.grid.x * tl.grid.y;
    return (size_t)(tiles * tl.grid.z + (n_keys / kWave + tiles + 1) * (int64_t)tl.grid.z * tl.threads);
}

extern "C" int tg_render_forward(const real *vertices, const int32_t *indices, const real *colors, const real *opacities,
                                 const int32_t *sorted_ids, const int32_t *offsets, const real *bary, int width, int height,
                                 int tile_w, int tile_h, real early_stopping_threshold, int per_pixel_sort, int max_layers,
                                 real *image, real *depthmap, real *final_weights, int32_t *ends, int32_t *last,
                                 real *last_depth, uint16_t *fragments, uint64_t *hit_masks, const real *batch_bounds,
                                 const int32_t *far_start, const uint32_t *list_status, void *stream) {
    if (int e = check_raster_args("tg_render_forward", width, height, tile_w, tile_h, max_layers)) return e;
    if (!vertices || !indices || !colors || !opacities || !offsets || !bary || !image || !depthmap || !final_weights || !ends) {
        set_error("tg_render_forward: null pointer");
        return TG_E_ARG;
    }
    if (((uintptr_t)vertices & 15) || ((uintptr_t)image & 15)) {
        set_error("tg_render_forward: vertices and image must be 16-byte aligned");
        return TG_E_ARG;
    }
    RasterArgs a{(const real4 *)vertices, indices, colors, opacities, sorted_ids, offsets, bary,
                 per_pixel_sort ? batch_bounds : nullptr, (per_pixel_sort && batch_bounds) ? far_start : nullptr,
                 width, height, tile_w, tile_h, early_stopping_threshold, max_layers};
    if (batch_bounds && !far_start) {
        set_error("tg_render_forward: batch_bounds come with far_start");
        return TG_E_ARG;
    }
    if (fragments && (!per_pixel_sort || max_layers > TG_MAX_SAVED_LAYERS)) {
        set_error("tg_render_forward: fragments are saved only with per_pixel_sort and max_layers <= %d", TG_MAX_SAVED_LAYERS);
        return TG_E_ARG;
    }
    ForwardOut o{(real4 *)image, depthmap, final_weights, ends, last, last_depth, fragments, per_pixel_sort ? nullptr : hit_masks,
                 list_status};
    const TileLaunch tl = tile_launch(width, height, tile_w, tile_h, per_pixel_sort ? pixel_order_threads(kTileThreads) : kTileThreads);
    const dim3 grid = tl.grid;
    const int n_threads = tl.threads;
    hipStream_t s = (hipStream_t)stream;
    if (!per_pixel_sort) {
        TG_LAUNCH(forward_tile_order_kernel, grid, dim3(n_threads), 0, s, a, o);
        return check_launch("forward_tile_order_kernel");
    }
    const size_t lds = pixel_order_lds_bytes(n_threads, kSelectBatch);
    // Depth bounds make the batches jump in steps of kSelectBatch, so they go with the int positions.
    const bool split = !a.batch_bounds && n_threads >= kSelectBatchShort;
    static size_t lds_reserved[kMaxDevices] = {0}, lds_reserved_long[kMaxDevices] = {0};
    if (!split) {
        if (int e = reserve_lds("tg_render_forward", (const void *)forward_pixel_order_kernel<kSelectBatch, int>, lds, lds_reserved)) return e;
        TG_LAUNCH_AS("forward_pixel_order_kernel", (forward_pixel_order_kernel<kSelectBatch, int>), grid, dim3(n_threads), lds, s, a, o);
        return check_launch("forward_pixel_order_kernel");
    }
    const size_t lds_short = pixel_order_lds_bytes(n_threads, kSelectBatchShort, sizeof(uint16_t));
    static size_t lds_reserved_short[kMaxDevices] = {0};
    if (int e = reserve_lds("tg_render_forward", (const void *)forward_pixel_order_kernel<kSelectBatchShort, uint16_t>, lds_short,
                            lds_reserved_short))
        return e;
    TG_LAUNCH_AS("forward_pixel_order_kernel", (forward_pixel_order_kernel<kSelectBatchShort, uint16_t>), grid, dim3(n_threads),
                 lds_short, s, a, o);
    if (int e = check_launch("forward_pixel_order_kernel")) return e;
    if (int e = reserve_lds("tg_render_forward", (const void *)forward_pixel_order_long_lists_kernel, lds, lds_reserved_long)) return e;
    const int tiles = (int)(grid.x * grid.y);
    TG_LAUNCH(forward_pixel_order_long_lists_kernel, dim3(min(tiles, kLongListGroups), 1, grid.z), dim3(n_threads), lds, s, a, o,
              (int)grid.x, (int)grid.y);
    return check_launch("forward_pixel_order_long_lists_kernel");
}
