// tg_sort.hip -- stable LSD radix sort of (uint64 key, uint32 value) pairs, 8 bits per pass.
//
// HBM-bound: one read of the keys for all digit histograms (8 B/key), then per
// pass one read and one write of key + value (24 B/key).  Structure:
//
//   fill        zero the tickets and the look-back words (one launch)
//   histogram   every workgroup builds the 256-bin histogram of EVERY pass in
//               LDS (ds_add_u32) from one sweep over the keys and stores it as
//               a partial (no global atomics)
//   bases       per pass (one workgroup of 1024 threads): sum the partials,
//               exclusive scan over the 256 digits
//   sweep x P   each workgroup owns a tile of 4096 consecutive pairs:
//                 - wave64 match ranking: 8 ballots find the lanes that hold
//                   the same digit, mbcnt-style popcounts give the stable rank,
//                   a per-wave 256-entry LDS counter row carries it across the
//                   16 items of a lane;
//                 - the tile's 256 digit counts are published in look-back
//                   words (one uint32 per digit: bits 31..30 = 0 not ready,
//                   1 aggregate, 2 inclusive prefix; bits 29..0 = count) and
//                   thread d walks back over the predecessors' words of digit d,
//                   eight words in flight per step (decoupled look-back;
//                   relaxed agent-scope atomics suffice as flag and value
//                   share a word);
//                 - pairs are permuted into digit order through LDS, then each
//                   digit run is written contiguously.
//
// Tiles are numbered by an atomic ticket so that a workgroup only ever waits for
// workgroups that already run -- or, when the whole grid fits the device at once
// (then no workgroup has to finish for another to start), by the workgroup ids,
// which saves the serialised same-address atomics.  Waits are bounded
// (TG_STATUS_LOOKBACK_TIMEOUT).
#include "tg_common.hpp"

namespace tg {

constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kMaxPasses = 8;
constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortItems = 16;
constexpr int kSortTile = kSortThreads * kSortItems;  // 4096 pairs
constexpr int kHistBlocksMax = 256;
constexpr int kBasesThreads = 1024;
constexpr int kLookWindow = 4;  // predecessors read per round trip; wider windows only add L2 traffic (measured 1..64)
constexpr uint32_t kSortSpinLimit = 1u << 20;
constexpr uint32_t kLbAggregate = 1u << 30;
constexpr uint32_t kLbInclusive = 2u << 30;
constexpr uint32_t kLbValueMask = (1u << 30) - 1;
constexpr int64_t kSortMaxN = (1ll << 30) - 1;

struct SortLayout {
    int passes;
    int n_tiles;
    int hist_blocks;
    size_t off_tickets, off_partials, off_bases, off_lookback, total;
};

static SortLayout sort_layout(int64_t n, int end_bit) {
    SortLayout L;
    L.passes = end_bit <= 0 ? 0 : (end_bit + kRadixBits - 1) / kRadixBits;
    L.n_tiles = (int)ceil_div64(n, kSortTile);
    L.hist_blocks = L.n_tiles < kHistBlocksMax ? (L.n_tiles > 0 ? L.n_tiles : 1) : kHistBlocksMax;
    size_t o = 0;
    L.off_bases = o;    o += (size_t)kMaxPasses * kRadix * 4;
    L.off_partials = o; o += (size_t)kHistBlocksMax * kMaxPasses * kRadix * 4;
    L.off_tickets = o;  o += 256;  // kMaxPasses tickets, padded; zeroed together with the look-back words
    L.off_lookback = o; o += (size_t)kMaxPasses * (size_t)(L.n_tiles > 0 ? L.n_tiles : 1) * kRadix * 4;
    L.total = o;
    return L;
}

__global__ void fill_zero_kernel(uint32_t *p, size_t n_words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_words; i += stride) p[i] = 0;
}

// Also clears `zero_words` words from `zero` on (the tickets and look-back words of the sweeps that
// follow), a slice per workgroup: a launch of its own for that costs more than the stores.
__global__ __launch_bounds__(kSortThreads) void sort_histogram_kernel(const uint64_t *__restrict__ keys, int64_t n, int passes,
                                                                      uint32_t *__restrict__ partials, uint32_t *__restrict__ zero,
                                                                      size_t zero_words) {
    for (size_t i = (size_t)blockIdx.x * kSortThreads + threadIdx.x; i < zero_words; i += (size_t)gridDim.x * kSortThreads) zero[i] = 0;
    // one set of counters per wave: the upper passes see few distinct digits (the tile bits), and LDS
    // atomics to one address serialise
    __shared__ uint32_t s_hist_wave[kSortWaves][kMaxPasses][kRadix];
    const int tid = threadIdx.x;
    uint32_t (*s_hist)[kRadix] = s_hist_wave[tid / kWave];
    for (int w = 0; w < kSortWaves; w++)
        for (int p = 0; p < passes; p++) s_hist_wave[w][p][tid] = 0;
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * kSortThreads * 4;
    for (int64_t i = (int64_t)blockIdx.x * kSortThreads * 4 + tid; i < n; i += stride) {
        uint64_t k[4];
#pragma unroll
        for (int u = 0; u < 4; u++) k[u] = (i + u * kSortThreads < n) ? keys[i + u * kSortThreads] : 0;
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i + u * kSortThreads < n)
                for (int p = 0; p < passes; p++) atomicAdd(&s_hist[p][(k[u] >> (p * kRadixBits)) & (kRadix - 1)], 1u);
    }
    __syncthreads();
    uint32_t *out = partials + (size_t)blockIdx.x * kMaxPasses * kRadix;
    for (int p = 0; p < passes; p++) {
        uint32_t sum = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) sum += s_hist_wave[w][p][tid];
        out[p * kRadix + tid] = sum;
    }
}

// One workgroup per pass: digit totals over all partials (four groups of 256
// threads share the partials), then exclusive scan over the 256 digits.
__global__ __launch_bounds__(kBasesThreads) void sort_bases_kernel(const uint32_t *__restrict__ partials, int hist_blocks,
                                                                   uint32_t *__restrict__ bases, uint32_t *status) {
    __shared__ uint32_t s_part[kBasesThreads / kRadix][kRadix];
    __shared__ uint32_t s_scan[kRadix];
    const int tid = threadIdx.x;
    const int digit = tid & (kRadix - 1), group = tid / kRadix;
    const int p = blockIdx.x;
    if (p == 0 && tid == 0 && status) *status = TG_STATUS_OK;
    uint32_t sum = 0;
#pragma unroll 8
    for (int b = group; b < hist_blocks; b += kBasesThreads / kRadix) sum += partials[((size_t)b * kMaxPasses + p) * kRadix + digit];
    s_part[group][digit] = sum;
    __syncthreads();
    uint32_t total = 0;
    if (tid < kRadix) {
#pragma unroll
        for (int k = 0; k < kBasesThreads / kRadix; k++) total += s_part[k][tid];
        s_scan[tid] = total;
    }
    __syncthreads();
    for (int off = 1; off < kRadix; off <<= 1) {  // Hillis-Steele over 256 entries
        uint32_t v = (tid < kRadix && tid >= off) ? s_scan[tid - off] : 0u;
        __syncthreads();
        if (tid < kRadix) s_scan[tid] += v;
        __syncthreads();
    }
    if (tid < kRadix) bases[p * kRadix + tid] = s_scan[tid] - total;
}

__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
    // number of set bits of `mask` in lanes lower than the caller
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__global__ __launch_bounds__(kSortThreads) void sort_sweep_kernel(const uint64_t *__restrict__ keys_in,
                                                                  const uint32_t *__restrict__ vals_in,
                                                                  uint64_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
                                                                  int64_t n, int shift, const uint32_t *__restrict__ bases,
                                                                  uint32_t *lookback, uint32_t *ticket, uint32_t *status) {
    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_global_delta[kRadix];
    __shared__ uint32_t s_scan_wave[kSortWaves];
    // The ranking counters are dead once every pair knows its place in the tile,
    // so they share LDS with the permutation buffer (51 KB: three workgroups per CU).
    __shared__ __align__(16) unsigned char s_raw[kSortTile * 12];
    uint32_t (*s_wave_count)[kRadix] = reinterpret_cast<uint32_t (*)[kRadix]>(s_raw);
    uint32_t *s_local_start = reinterpret_cast<uint32_t *>(s_raw) + kSortWaves * kRadix;
    uint64_t *s_keys = reinterpret_cast<uint64_t *>(s_raw);
    uint32_t *s_vals = reinterpret_cast<uint32_t *>(s_raw + kSortTile * 8);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    if (tid == 0) s_tile = ticket ? atomicAdd(ticket, 1u) : blockIdx.x;  // no ticket: the whole grid is resident
    for (int w = 0; w < kSortWaves; w++) s_wave_count[w][tid] = 0;
    __syncthreads();
    const int tile = (int)s_tile;
    const int64_t tile_base = (int64_t)tile * kSortTile;
    const int n_valid = (int)((n - tile_base) < kSortTile ? (n - tile_base) : kSortTile);

    // Wave-striped loads keep memory order = (wave, item, lane) order.
    uint64_t key[kSortItems];
    uint32_t val[kSortItems];
    uint32_t rank[kSortItems];
    const int lane_base = wave * (kWave * kSortItems) + lane;
#pragma unroll
    for (int i = 0; i < kSortItems; i++) {
        const int local = lane_base + i * kWave;
        if (local < n_valid) {
            key[i] = keys_in[tile_base + local];
            val[i] = vals_in[tile_base + local];
        } else {
            key[i] = ~0ull;  // padding ranks after every real pair of the tile
            val[i] = 0;
        }
    }

    // Stable rank of each pair among the pairs of its wave with the same digit.
    // Match: 8 ballots leave in `peers` the lanes that hold the same digit.  The
    // lowest lane of each group adds the group size to the wave's counter row
    // with a returning LDS atomic; LDS serves a wave's instructions in order, so
    // item i sees the counts of items < i, and the 16 atomics are in flight
    // together.  The group reads its leader's result with ds_bpermute.
    uint32_t *wave_row = s_wave_count[wave];
    uint32_t below[kSortItems];
    uint32_t leader[kSortItems];
    uint32_t before[kSortItems];
#pragma unroll
    for (int i = 0; i < kSortItems; i++) {
        const uint32_t d = (uint32_t)(key[i] >> shift) & (kRadix - 1);
        uint64_t peers = ~0ull;
#pragma unroll
        for (int b = 0; b < kRadixBits; b++) {
            const bool bit = (d >> b) & 1u;
            const uint64_t vote = __builtin_amdgcn_ballot_w64(bit);
            peers &= bit ? vote : ~vote;
        }
        below[i] = lanes_below(peers);
        leader[i] = (uint32_t)__builtin_ctzll(peers);
        before[i] = 0;
        if (below[i] == 0) before[i] = __hip_atomic_fetch_add(wave_row + d, (uint32_t)__builtin_popcountll(peers), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
#pragma unroll
    for (int i = 0; i < kSortItems; i++)
        rank[i] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(leader[i] << 2), (int)before[i]) + below[i];
    __syncthreads();

    // Thread d owns digit d: per-wave exclusive offsets, tile count, look-back.
    uint32_t digit_count = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) {
        const uint32_t c = s_wave_count[w][tid];
        s_wave_count[w][tid] = digit_count;
        digit_count += c;
    }
    // real pairs only: padding always carries digit 255
    const uint32_t published = (tid == kRadix - 1) ? digit_count - (uint32_t)(kSortTile - n_valid) : digit_count;
    uint32_t *my_words = lookback + tid;
    __hip_atomic_store(my_words + (size_t)tile * kRadix, (tile == 0 ? kLbInclusive : kLbAggregate) | published, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);

    // exclusive scan of the tile's digit counts (padding included: it sits at the end)
    {
        uint32_t v = digit_count;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const uint32_t up = __shfl_up(v, off, kWave);
            if (lane >= off) v += up;
        }
        if (lane == kWave - 1) s_scan_wave[wave] = v;
        __syncthreads();
        uint32_t wave_prefix = 0;
        for (int w = 0; w < wave; w++) wave_prefix += s_scan_wave[w];
        s_local_start[tid] = wave_prefix + v - digit_count;
    }

    // Place of every pair inside the tile, then permute into digit order in LDS
    // (the buffer overlays the counters) and write digit runs contiguously.
    const uint32_t local_start = s_local_start[tid];
    __syncthreads();  // s_local_start is complete
#pragma unroll
    for (int i = 0; i < kSortItems; i++) {
        const uint32_t d = (uint32_t)(key[i] >> shift) & (kRadix - 1);
        rank[i] += s_local_start[d] + s_wave_count[wave][d];
    }
    __syncthreads();  // every pair knows its place: the counters may be overwritten
#pragma unroll
    for (int i = 0; i < kSortItems; i++) {
        s_keys[rank[i]] = key[i];
        s_vals[rank[i]] = val[i];
    }
    // While the pairs settle in LDS the predecessors publish their counts.
    uint32_t prefix = 0;
    bool timed_out = false;
    for (int look = tile - 1; look >= 0 && !timed_out;) {
        uint32_t words[kLookWindow];
#pragma unroll
        for (int k = 0; k < kLookWindow; k++)
            words[k] = (look - k >= 0)
                           ? __hip_atomic_load(my_words + (size_t)(look - k) * kRadix, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                           : kLbInclusive;  // before the first tile: inclusive prefix 0
        bool done = false;
#pragma unroll
        for (int k = 0; k < kLookWindow; k++) {
            if (done || timed_out) continue;
            uint32_t word = words[k];
            uint32_t spins = 0;
            while ((word >> 30) == 0 && spins < kSortSpinLimit) {
                __builtin_amdgcn_s_sleep(1);
                word = __hip_atomic_load(my_words + (size_t)(look - k) * kRadix, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                spins++;
            }
            if ((word >> 30) == 0) { timed_out = true; continue; }
            prefix += word & kLbValueMask;
            if ((word >> 30) == 2) done = true;
        }
        if (done) break;
        look -= kLookWindow;
    }
    if (tile != 0)
        __hip_atomic_store(my_words + (size_t)tile * kRadix, kLbInclusive | ((prefix + published) & kLbValueMask), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    if (timed_out && status) *status = TG_STATUS_LOOKBACK_TIMEOUT;
    s_global_delta[tid] = bases[tid] + prefix - local_start;

    __syncthreads();
#pragma unroll
    for (int i = 0; i < kSortItems; i++) {
        const int pos = i * kSortThreads + tid;
        if (pos < n_valid) {
            const uint64_t k = s_keys[pos];
            const uint32_t d = (uint32_t)(k >> shift) & (kRadix - 1);
            const uint32_t g = s_global_delta[d] + (uint32_t)pos;
            keys_out[g] = k;
            vals_out[g] = s_vals[pos];
        }
    }
}

}  // namespace tg

using namespace tg;

extern "C" size_t tg_sort_workspace_bytes(int64_t n) {
    if (n < 0 || n > kSortMaxN) return 0;
    return sort_layout(n, 64).total;
}

extern "C" int tg_sort_pairs_u64_u32(uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int64_t n,
                                     int end_bit, void *workspace, size_t workspace_bytes, uint32_t *status, int *result_in_alt,
                                     void *stream) {
    if (n < 0 || n > kSortMaxN || end_bit < 0 || end_bit > 64 || !result_in_alt) {
        set_error("tg_sort_pairs_u64_u32: n must be in [0, 2^30), end_bit in [0, 64]");
        return TG_E_ARG;
    }
    *result_in_alt = 0;
    hipStream_t s = (hipStream_t)stream;
    if (n == 0 || end_bit == 0) {
        if (status) {
            TG_LAUNCH(fill_zero_kernel, dim3(1), dim3(64), 0, s, status, (size_t)1);
            if (int e = check_launch("fill_zero_kernel")) return e;
        }
        return 0;
    }
    if (!keys || !values || !keys_alt || !values_alt || !workspace) {
        set_error("tg_sort_pairs_u64_u32: null pointer");
        return TG_E_ARG;
    }
    if (((uintptr_t)keys & 7) || ((uintptr_t)keys_alt & 7) || ((uintptr_t)workspace & 255)) {
        set_error("tg_sort_pairs_u64_u32: keys must be 8-byte aligned, workspace 256-byte aligned");
        return TG_E_ARG;
    }
    const SortLayout L = sort_layout(n, end_bit);
    if (workspace_bytes < L.total) {
        set_error("tg_sort_pairs_u64_u32: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
        return TG_E_WORKSPACE;
    }
    char *ws = (char *)workspace;
    uint32_t *tickets = (uint32_t *)(ws + L.off_tickets);
    uint32_t *bases = (uint32_t *)(ws + L.off_bases);
    uint32_t *partials = (uint32_t *)(ws + L.off_partials);
    uint32_t *lookback = (uint32_t *)(ws + L.off_lookback);

    // tickets and look-back words (adjacent) start at zero; bases and partials are fully overwritten
    const size_t fill_words = 64 + (size_t)L.passes * L.n_tiles * kRadix;
    TG_LAUNCH(sort_histogram_kernel, dim3(L.hist_blocks), dim3(kSortThreads), 0, s, keys, n, L.passes, partials, tickets, fill_words);
    if (int e = check_launch("sort_histogram_kernel")) return e;
    TG_LAUNCH(sort_bases_kernel, dim3(L.passes), dim3(kBasesThreads), 0, s, partials, L.hist_blocks, bases, status);
    if (int e = check_launch("sort_bases_kernel")) return e;

    uint64_t *kin = keys, *kout = keys_alt;
    uint32_t *vin = values, *vout = values_alt;
    // 534 same-address ticket atomics cost 6 us per pass; a grid that fits the device whole takes its
    // tile numbers from the workgroup ids instead
    static int resident_cache[kMaxDevices] = {0};
    const bool whole_grid_resident = L.n_tiles <= resident_workgroups((const void *)sort_sweep_kernel, kSortThreads, resident_cache);
    {
        // one pair of timing events around all passes: a pair per launch would add its own two
        // microseconds to every 24 us kernel
        ProfileScope timed("sort_sweep_kernel", s, L.passes);
        for (int p = 0; p < L.passes; p++) {
            hipLaunchKernelGGL(sort_sweep_kernel, dim3(L.n_tiles), dim3(kSortThreads), 0, s, kin, vin, kout, vout, n, p * kRadixBits,
                               bases + p * kRadix, lookback + (size_t)p * L.n_tiles * kRadix,
                               whole_grid_resident ? (uint32_t *)nullptr : tickets + p, status);
            if (int e = check_launch("sort_sweep_kernel")) return e;
            uint64_t *tk = kin; kin = kout; kout = tk;
            uint32_t *tv = vin; vin = vout; vout = tv;
        }
    }
    *result_in_alt = (L.passes & 1);
    return 0;
}
