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
#include "tg_scan.hpp"
#include "tg_sort_plan.hpp"

namespace tg {

__global__ void fill_zero_kernel(uint32_t *p, size_t n_words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_words; i += stride) p[i] = 0;
}

// Also clears `zero_words` words from `zero` on (the tickets and look-back words of the sweeps that
// follow), a slice per workgroup: a launch of its own for that costs more than the stores.
// 1024 threads a workgroup (one per CU at most 256 workgroups: the partials stay few) keep the LDS atomics of
// sixteen waves in flight; the counters exist once per pair of waves, because the upper passes see few
// distinct digits (the tile bits) and LDS atomics to one address serialise.
constexpr int kHistThreads = 1024;
constexpr int kHistSets = kHistThreads / kWave / 2;
__global__ __launch_bounds__(kHistThreads) void sort_histogram_kernel(const uint64_t *__restrict__ keys, int64_t n, PassPlan plan,
                                                                      uint32_t *__restrict__ partials, uint32_t *__restrict__ zero,
                                                                      size_t zero_words) {
    for (size_t i = (size_t)blockIdx.x * kHistThreads + threadIdx.x; i < zero_words; i += (size_t)gridDim.x * kHistThreads) zero[i] = 0;
    __shared__ uint32_t s_hist_set[kHistSets][kMaxPasses][kRadix];
    const int tid = threadIdx.x;
    const int passes = plan.passes;
    uint32_t (*s_hist)[kRadix] = s_hist_set[tid / (2 * kWave)];
    for (int j = tid; j < kHistSets * kMaxPasses * kRadix; j += kHistThreads) s_hist_set[0][0][j] = 0;
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * kHistThreads * 4;
    for (int64_t i = (int64_t)blockIdx.x * kHistThreads * 4 + tid; i < n; i += stride) {
        uint64_t k[4];
#pragma unroll
        for (int u = 0; u < 4; u++) k[u] = (i + u * kHistThreads < n) ? keys[i + u * kHistThreads] : 0;
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i + u * kHistThreads < n)
                for (int p = 0; p < passes; p++) atomicAdd(&s_hist[p][(uint32_t)(k[u] >> plan.shift[p]) & ((1u << plan.bits[p]) - 1)], 1u);
    }
    __syncthreads();
    uint32_t *out = partials + (size_t)blockIdx.x * kMaxPasses * kRadix;
    for (int j = tid; j < passes * kRadix; j += kHistThreads) {
        uint32_t sum = 0;
#pragma unroll
        for (int w = 0; w < kHistSets; w++) sum += s_hist_set[w][0][j];
        out[j] = sum;
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

// Stable rank of each of a lane's ITEMS digits among the equal digits of its wave, items in order, lanes in
// order within an item.  Match: every lane ORs its lane bit into the 64-bit LDS word of its digit and reads the
// word back: the lanes that hold the same digit (LDS serves a wave's instructions in order, so the read sees
// all 64 ORs of the instruction before it).  The lowest lane of each group adds the group size to the wave's
// counter row with a returning LDS atomic -- item i so sees the counts of items < i -- and clears the mask
// word; the group reads its leader's result with ds_bpermute.  Two sets of mask words take turns, so that the
// next item's OR and read are under way while this item's words are still in use.
// masks: 2 * kRadix words, zero on entry and zero again on return.  Afterwards wave_row[d] = the wave's
// number of digits d.
constexpr int kMaskWords = 2 * kRadix;
template <int ITEMS>
__device__ __forceinline__ void wave_match_rank(const uint32_t (&digit)[ITEMS], uint32_t *wave_row, unsigned long long *masks,
                                                uint32_t (&rank)[ITEMS]) {
    constexpr int kGroup = ITEMS < 16 ? ITEMS : 16;  // returning atomics in flight before their results are used
    static_assert(ITEMS % kGroup == 0, "whole groups");
    const unsigned long long me = 1ull << (threadIdx.x & (kWave - 1));
    (void)__hip_atomic_fetch_or(masks + digit[0], me, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    unsigned long long next = __hip_atomic_load(masks + digit[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
    for (int g = 0; g < ITEMS; g += kGroup) {
        uint32_t below[kGroup];
        uint32_t leader[kGroup];
        uint32_t before[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const int i = g + j;
            const unsigned long long peers = next;
            unsigned long long *mine = masks + (i & 1) * kRadix + digit[i];
            if (i + 1 < ITEMS) {
                unsigned long long *ahead = masks + ((i + 1) & 1) * kRadix + digit[i + 1];
                (void)__hip_atomic_fetch_or(ahead, me, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                next = __hip_atomic_load(ahead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            below[j] = lanes_below(peers);
            leader[j] = (uint32_t)__builtin_ctzll(peers);
            before[j] = 0;
            if (below[j] == 0) {
                before[j] = __hip_atomic_fetch_add(wave_row + digit[i], (uint32_t)__builtin_popcountll(peers), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_store(mine, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
#pragma unroll
        for (int j = 0; j < kGroup; j++)
            rank[g + j] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(leader[j] << 2), (int)before[j]) + below[j];
    }
}

// The same ranks with the match done by ballots instead of mask words: BITS ballots leave in `peers` the lanes
// that hold the same digit (about six vector instructions per bit).  No working memory; the segment sorts use
// it, whose waves keep the LDS busier than the vector units (measured: mask words 41 against ballots 37 us on
// the 8160 lists of the headline frame; the sweeps gain from the mask words, 21.6 -> 20 us a pass).
template <int BITS, int ITEMS>
__device__ __forceinline__ void wave_match_rank_ballots(const uint32_t (&digit)[ITEMS], uint32_t *wave_row, uint32_t (&rank)[ITEMS]) {
    constexpr int kGroup = ITEMS < 16 ? ITEMS : 16;  // atomics in flight together
    static_assert(ITEMS % kGroup == 0, "whole groups");
#pragma unroll
    for (int g = 0; g < ITEMS; g += kGroup) {
        uint32_t below[kGroup];
        uint32_t leader[kGroup];
        uint32_t before[kGroup];
#pragma unroll
        for (int i = 0; i < kGroup; i++) {
            const uint32_t d = digit[g + i];
            uint64_t peers = ~0ull;
#pragma unroll
            for (int b = 0; b < BITS; b++) {
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
        for (int i = 0; i < kGroup; i++)
            rank[g + i] = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(leader[i] << 2), (int)before[i]) + below[i];
    }
}

// One pass over digit (key >> shift) & mask, mask < 2^BITS.  `bases`: the exclusive scan of the digit totals,
// or, with totals_given, the totals themselves (scanned here).
template <int BITS>
__global__ __launch_bounds__(kSweepThreads) void sort_sweep_kernel(const uint64_t *__restrict__ keys_in,
                                                                  const uint32_t *__restrict__ vals_in,
                                                                  uint64_t *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
                                                                  int64_t n, int shift, uint32_t mask,
                                                                  const uint32_t *__restrict__ bases, int totals_given,
                                                                  uint32_t *lookback, uint32_t *ticket, uint32_t *status,
                                                                  int unpad_bits, int tiles_x, uint32_t *tile_count) {
    constexpr int kDigits = 1 << BITS;
    __shared__ uint32_t s_tile;
    __shared__ uint32_t s_global_delta[kRadix];
    __shared__ uint32_t s_scan_wave[kSweepWaves];
    __shared__ uint32_t s_base_wave[kSweepWaves];
    __shared__ uint32_t s_several_tiles[kRadix];  // with tile_count: the digit's pairs of this sort tile belong to more than one tile
    // The ranking counters are dead once every pair knows its place in the tile,
    // so they share LDS with the permutation buffer (51 KB: three workgroups per CU).
    __shared__ __align__(16) unsigned char s_raw[kSortTile * 12];
    uint32_t (*s_wave_count)[kRadix] = reinterpret_cast<uint32_t (*)[kRadix]>(s_raw);
    uint32_t *s_local_start = reinterpret_cast<uint32_t *>(s_raw) + kSweepWaves * kRadix;
    constexpr int kMaskOffset = (kSweepWaves + 1) * kRadix * 4;
    static_assert(kMaskOffset % 8 == 0 && kMaskOffset + kSweepWaves * kMaskWords * 8 <= kSortTile * 12, "counters and mask words fit the permutation buffer");
    unsigned long long *s_masks = reinterpret_cast<unsigned long long *>(s_raw + kMaskOffset);  // kSweepWaves sets of kMaskWords
    uint64_t *s_keys = reinterpret_cast<uint64_t *>(s_raw);
    uint32_t *s_vals = reinterpret_cast<uint32_t *>(s_raw + kSortTile * 8);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const bool owns_digit = tid < kDigits;
    if (tid == 0) s_tile = ticket ? atomicAdd(ticket, 1u) : blockIdx.x;  // no ticket: the whole grid is resident
    for (int j = tid; j < kSweepWaves * kRadix; j += kSweepThreads) s_wave_count[0][j] = 0;
    for (int j = tid; j < kSweepWaves * kMaskWords; j += kSweepThreads) s_masks[j] = 0;
    // this digit's first output position: given, or the exclusive scan of the totals
    uint32_t base = owns_digit ? bases[totals_given ? tid * kTotalsStride : tid] : 0u;
    uint32_t base_incl = 0;
    if (totals_given) {
        base_incl = wave_inclusive_scan_u32(base);
        if (lane == kWave - 1) s_base_wave[wave] = base_incl;
    }
    __syncthreads();
    if (totals_given) {
        uint32_t wave_prefix = 0;
        for (int w = 0; w < wave; w++) wave_prefix += s_base_wave[w];
        base = wave_prefix + base_incl - base;
    }
    const int tile = (int)s_tile;
    const int64_t tile_base = (int64_t)tile * kSortTile;
    const int n_valid = (int)((n - tile_base) < kSortTile ? (n - tile_base) : kSortTile);

    // Wave-striped loads keep memory order = (wave, item, lane) order.
    uint64_t key[kSweepItems];
    uint32_t val[kSweepItems];
    uint32_t digit[kSweepItems];
    uint32_t rank[kSweepItems];
    const int lane_base = wave * (kWave * kSweepItems) + lane;
#pragma unroll
    for (int i = 0; i < kSweepItems; i++) {
        const int local = lane_base + i * kWave;
        if (local < n_valid) {
            key[i] = keys_in[tile_base + local];
            val[i] = vals_in[tile_base + local];
        } else {
            key[i] = ~0ull;  // padding ranks after every real pair of the tile
            val[i] = 0;
        }
        digit[i] = (uint32_t)(key[i] >> shift) & mask;
    }
    wave_match_rank<kSweepItems>(digit, s_wave_count[wave], s_masks + wave * kMaskWords, rank);
    __syncthreads();

    // Thread d owns digit d: per-wave exclusive offsets, tile count, look-back.
    uint32_t digit_count = 0;
    if (tid < kRadix) {
#pragma unroll
        for (int w = 0; w < kSweepWaves; w++) {
            const uint32_t c = s_wave_count[w][tid];
            s_wave_count[w][tid] = digit_count;
            digit_count += c;
        }
    }
    // real pairs only: padding always carries the largest digit
    const uint32_t published = ((uint32_t)tid == mask) ? digit_count - (uint32_t)(kSortTile - n_valid) : digit_count;
    uint32_t *my_words = lookback + tid;
    if (owns_digit)
        __hip_atomic_store(my_words + (size_t)tile * kDigits, kLbAggregate | published, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // exclusive scan of the tile's digit counts (padding included: it sits at the end)
    {
        const uint32_t v = wave_inclusive_scan_u32(digit_count);
        if (lane == kWave - 1) s_scan_wave[wave] = v;
        __syncthreads();
        uint32_t wave_prefix = 0;
        for (int w = 0; w < wave; w++) wave_prefix += s_scan_wave[w];
        if (tid < kRadix) s_local_start[tid] = wave_prefix + v - digit_count;
    }

    // Place of every pair inside the tile, then permute into digit order in LDS
    // (the buffer overlays the counters) and write digit runs contiguously.
    __syncthreads();  // s_local_start is complete
    const uint32_t local_start = s_local_start[tid & (kRadix - 1)];
#pragma unroll
    for (int i = 0; i < kSweepItems; i++) rank[i] += s_local_start[digit[i]] + s_wave_count[wave][digit[i]];
    __syncthreads();  // every pair knows its place: the counters may be overwritten
#pragma unroll
    for (int i = 0; i < kSweepItems; i++) {
        s_keys[rank[i]] = key[i];
        s_vals[rank[i]] = val[i];
    }
    // While the pairs settle in LDS the predecessors publish their counts.  Two levels keep the chain of waits
    // short: the tiles of a group of kLookGroup read each other's counts directly (all published at about
    // the same time, so one round of loads), the tile that closes a group publishes the group's total, and
    // the look-back proper (aggregate / inclusive words, a window of loads per round trip) runs over groups.
    const int group = tile / kLookGroup, group_first = group * kLookGroup;
    uint32_t *group_words = lookback + (size_t)gridDim.x * kDigits + tid;
    uint32_t in_group = 0, group_prefix = 0;
    bool timed_out = false;
    if (owns_digit) {
        for (int j0 = group_first; j0 < tile && !timed_out; j0 += kLookWindow) {
            uint32_t words[kLookWindow];
#pragma unroll
            for (int k = 0; k < kLookWindow; k++)
                words[k] = (j0 + k < tile) ? __hip_atomic_load(my_words + (size_t)(j0 + k) * kDigits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                           : kLbAggregate;
#pragma unroll
            for (int k = 0; k < kLookWindow; k++) {
                if (timed_out) continue;
                uint32_t word = words[k];
                uint32_t spins = 0;
                while ((word >> 30) == 0 && spins < kSortSpinLimit) {
                    __builtin_amdgcn_s_sleep(1);
                    word = __hip_atomic_load(my_words + (size_t)(j0 + k) * kDigits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    spins++;
                }
                if ((word >> 30) == 0) { timed_out = true; continue; }
                in_group += word & kLbValueMask;
            }
        }
        const bool closes_group = tile == group_first + kLookGroup - 1 || tile == (int)gridDim.x - 1;
        if (closes_group)
            __hip_atomic_store(group_words + (size_t)group * kDigits, (group == 0 ? kLbInclusive : kLbAggregate) | ((in_group + published) & kLbValueMask),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int look = group - 1; look >= 0 && !timed_out;) {
            uint32_t words[kLookWindow];
#pragma unroll
            for (int k = 0; k < kLookWindow; k++)
                words[k] = (look - k >= 0)
                               ? __hip_atomic_load(group_words + (size_t)(look - k) * kDigits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                               : kLbInclusive;  // before the first group: inclusive prefix 0
            bool done = false;
#pragma unroll
            for (int k = 0; k < kLookWindow; k++) {
                if (done || timed_out) continue;
                uint32_t word = words[k];
                uint32_t spins = 0;
                while ((word >> 30) == 0 && spins < kSortSpinLimit) {
                    __builtin_amdgcn_s_sleep(1);
                    word = __hip_atomic_load(group_words + (size_t)(look - k) * kDigits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    spins++;
                }
                if ((word >> 30) == 0) { timed_out = true; continue; }
                group_prefix += word & kLbValueMask;
                if ((word >> 30) == 2) done = true;
            }
            if (done) break;
            look -= kLookWindow;
        }
        if (closes_group && group != 0)
            __hip_atomic_store(group_words + (size_t)group * kDigits, kLbInclusive | ((group_prefix + in_group + published) & kLbValueMask),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const uint32_t prefix = group_prefix + in_group;
    if (timed_out && status) *status = TG_STATUS_LOOKBACK_TIMEOUT;
    if (tid < kRadix) s_global_delta[tid] = base + prefix - local_start;

    __syncthreads();
    if (tile_count) {
        if (tid < kRadix) {
            // the last pass of a sort by tile column and row: the pairs of a row lie together in LDS, ordered by column.
            // Mostly they are one tile's (a sort tile spans few columns): then the row's count is that tile's.
            uint32_t several = 0;
            if (owns_digit && published > 0) {
                const uint32_t hi_first = (uint32_t)(s_keys[local_start] >> 32), hi_last = (uint32_t)(s_keys[local_start + published - 1] >> 32);
                if (hi_first == hi_last)
                    atomicAdd(&tile_count[(hi_first >> unpad_bits) * (uint32_t)tiles_x + (hi_first & ((1u << unpad_bits) - 1))], published);
                else
                    several = 1;
            }
            s_several_tiles[tid] = several;
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < kSweepItems; i++) {
        const int pos = i * kSweepThreads + tid;
        if (pos < n_valid) {
            uint64_t k = s_keys[pos];
            const uint32_t d = (uint32_t)(k >> shift) & mask;
            const uint32_t g = s_global_delta[d] + (uint32_t)pos;
            if (unpad_bits) {
                // the last pass of a sort by tile column and row: the high word ty << unpad_bits | tx becomes the tile
                // number.  Where a row's pairs here belong to several tiles, each run of one tile adds its length to
                // the tile's count (its first and its last pair add what they know of it).
                const uint32_t hi = (uint32_t)(k >> 32);
                const uint32_t tile_id = (hi >> unpad_bits) * (uint32_t)tiles_x + (hi & ((1u << unpad_bits) - 1));
                k = ((uint64_t)tile_id << 32) | (uint32_t)k;
                if (tile_count && s_several_tiles[d]) {
                    const uint32_t before = pos > 0 ? (uint32_t)(s_keys[pos - 1] >> 32) : ~hi;
                    const uint32_t after = pos + 1 < n_valid ? (uint32_t)(s_keys[pos + 1] >> 32) : ~hi;
                    const bool first = before != hi, last = after != hi;
                    if (first && last) atomicAdd(&tile_count[tile_id], 1u);
                    else if (first) atomicAdd(&tile_count[tile_id], 0u - (uint32_t)pos);
                    else if (last) atomicAdd(&tile_count[tile_id], (uint32_t)pos + 1u);
                }
            }
            keys_out[g] = k;
            vals_out[g] = s_vals[pos];
        }
    }
}

// ---- sorting the segments of a key array that is ordered by its high word ----------------------------
//
// After the passes over the tile bits every tile's pairs lie together, in emission order.  One workgroup
// then sorts a segment by its low key word (the depth bits) without leaving the CU: the pairs sit in
// registers, four 8-bit passes rank them with the same wave match as the sweeps and exchange them through
// LDS, and a pass whose digit is the same for the whole segment is left out.  A segment longer than the
// LDS holds is sorted by its workgroup through memory, pass by pass, between the two buffer pairs.

constexpr int kSegWaveItemsMax = 8;                                // segments up to 512 pairs: one wave each, no barriers
constexpr int kSegWaveCap = kWave * kSegWaveItemsMax;
constexpr int kSegLargeItems = 32;                                 // up to 8192 pairs in LDS (64 KB: two workgroups per CU)
constexpr int kSegLargeCap = kSortThreads * kSegLargeItems;
constexpr int kSegStreamItems = 8;                                 // chunk of the pass through memory
constexpr int kSegLargeGrid = 512;

struct SegLds {
    uint32_t count[kSortWaves][kRadix];
    uint32_t start[kRadix];
    uint32_t wave_total[kSortWaves];
    uint32_t varying;
};

__device__ __forceinline__ uint32_t wave_or_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v |= (uint32_t)__shfl_xor((int)v, off, kWave);
    return v;
}

// Ranks the workgroup's 256 * ITEMS digits (wave-striped order: wave, item, lane) and leaves in place[i]
// the position of item i in digit order.  Barriers inside; the caller separates calls by one more.
template <int ITEMS>
__device__ __forceinline__ void workgroup_digit_places(const uint32_t (&digit)[ITEMS], SegLds &lds, uint32_t (&place)[ITEMS]) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    for (int w = 0; w < kSortWaves; w++) lds.count[w][tid] = 0;
    __syncthreads();
    wave_match_rank_ballots<kRadixBits, ITEMS>(digit, lds.count[wave], place);
    __syncthreads();
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) {
        const uint32_t c = lds.count[w][tid];
        lds.count[w][tid] = run;
        run += c;
    }
    const uint32_t incl = wave_inclusive_scan_u32(run);
    if (lane == kWave - 1) lds.wave_total[wave] = incl;
    __syncthreads();
    uint32_t wave_prefix = 0;
    for (int w = 0; w < wave; w++) wave_prefix += lds.wave_total[w];
    lds.start[tid] = wave_prefix + incl - run;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; i++) place[i] += lds.start[digit[i]] + lds.count[wave][digit[i]];
}

// Sorts keys[start, start + n) / vals by the low key word, in place; n <= 256 * ITEMS.
template <int ITEMS>
__device__ __forceinline__ void segment_sort_in_lds(uint64_t *keys, uint32_t *vals, int64_t start, int n, SegLds &lds,
                                                    uint32_t *ex_keys, uint32_t *ex_vals) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    constexpr int kWaveSpan = kWave * ITEMS;
    uint32_t key[ITEMS], val[ITEMS];
    const uint64_t first = keys[start];
    uint32_t varying = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        const int pos = wave * kWaveSpan + i * kWave + lane;
        if (pos < n) {
            key[i] = (uint32_t)keys[start + pos];
            val[i] = vals[start + pos];
            varying |= key[i] ^ (uint32_t)first;
        } else {
            key[i] = ~0u;  // padding: behind every real pair, and a stable sort keeps it there
            val[i] = 0;
        }
    }
    if (tid == 0) lds.varying = 0;
    __syncthreads();
    varying = wave_or_u32(varying);
    if (lane == 0 && varying) atomicOr(&lds.varying, varying);
    __syncthreads();
    varying = lds.varying;
    if (varying == 0) return;  // all keys equal: the order stays
    const int last_pass = (31 - __builtin_clz(varying)) >> 3;
#pragma unroll 1
    for (int p = 0; p <= last_pass; p++) {
        const int shift = p * kRadixBits;
        if (((varying >> shift) & (kRadix - 1)) == 0) continue;  // the whole segment shares this digit
        uint32_t digit[ITEMS], place[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; i++) digit[i] = (key[i] >> shift) & (kRadix - 1);
        workgroup_digit_places<ITEMS>(digit, lds, place);
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            ex_keys[place[i]] = key[i];
            ex_vals[place[i]] = val[i];
        }
        __syncthreads();
        if (p == last_pass) break;
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            const int pos = wave * kWaveSpan + i * kWave + lane;
            key[i] = ex_keys[pos];
            val[i] = ex_vals[pos];
        }
        __syncthreads();  // everything is read before the next pass writes the exchange buffer
    }
    const uint64_t high = first & 0xffffffff00000000ull;
    for (int pos = tid; pos < n; pos += kSortThreads) {
        keys[start + pos] = high | ex_keys[pos];
        vals[start + pos] = ex_vals[pos];
    }
}

// ---- one wave per segment ----
struct WaveSegLds {
    uint32_t count[kRadix];
    uint32_t ex_keys[kSegWaveCap], ex_vals[kSegWaveCap];
};

// Orders the LDS traffic of one wave: LDS serves a wave's instructions in order, so a lane sees what another
// lane of its wave wrote by an earlier instruction; this keeps the compiler from moving accesses across.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The calling wave sorts keys[start, start + n) / vals by the low key word, in place; n <= 64 * ITEMS.
template <int ITEMS>
__device__ __forceinline__ void segment_sort_in_wave(uint64_t *keys, uint32_t *vals, int64_t start, int n, WaveSegLds &lds) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t key[ITEMS], val[ITEMS];
    const uint64_t first = keys[start];
    uint32_t varying = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        const int pos = i * kWave + lane;
        if (pos < n) {
            key[i] = (uint32_t)keys[start + pos];
            val[i] = vals[start + pos];
            varying |= key[i] ^ (uint32_t)first;
        } else {
            key[i] = ~0u;  // padding: behind every real pair, and a stable sort keeps it there
            val[i] = 0;
        }
    }
    varying = wave_or_u32(varying);
    if (varying == 0) return;  // all keys equal: the order stays
    const int last_pass = (31 - __builtin_clz(varying)) >> 3;
#pragma unroll 1
    for (int p = 0; p <= last_pass; p++) {
        const int shift = p * kRadixBits;
        if (((varying >> shift) & (kRadix - 1)) == 0) continue;  // the whole segment shares this digit
        uint32_t digit[ITEMS], place[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; i++) digit[i] = (key[i] >> shift) & (kRadix - 1);
#pragma unroll
        for (int j = 0; j < kRadix / kWave; j++) lds.count[j * kWave + lane] = 0;
        wave_lds_sync();
        wave_match_rank_ballots<kRadixBits, ITEMS>(digit, lds.count, place);
        wave_lds_sync();
        // exclusive scan of the 256 digit counts: four neighbouring digits per lane
        {
            uint32_t c[kRadix / kWave];
            uint32_t sum = 0;
#pragma unroll
            for (int j = 0; j < kRadix / kWave; j++) { c[j] = lds.count[lane * (kRadix / kWave) + j]; sum += c[j]; }
            uint32_t run = wave_inclusive_scan_u32(sum) - sum;
#pragma unroll
            for (int j = 0; j < kRadix / kWave; j++) { lds.count[lane * (kRadix / kWave) + j] = run; run += c[j]; }
        }
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            place[i] += lds.count[digit[i]];
            lds.ex_keys[place[i]] = key[i];
            lds.ex_vals[place[i]] = val[i];
        }
        wave_lds_sync();
        if (p == last_pass) break;
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            key[i] = lds.ex_keys[i * kWave + lane];
            val[i] = lds.ex_vals[i * kWave + lane];
        }
        wave_lds_sync();
    }
    const uint64_t high = first & 0xffffffff00000000ull;
#pragma unroll
    for (int i = 0; i < ITEMS; i++) {
        const int pos = i * kWave + lane;
        if (pos < n) {
            keys[start + pos] = high | lds.ex_keys[pos];
            vals[start + pos] = lds.ex_vals[pos];
        }
    }
}

// One workgroup per four segments.  A segment of up to kSegWaveCap pairs is sorted by one wave of its own;
// then the workgroup takes those of up to kSegMediumCap pairs together, one after the other.  Longer ones are
// left to segment_sort_large_kernel.
constexpr int kSegMediumItems = 8;
constexpr int kSegMediumCap = kSortThreads * kSegMediumItems;  // 2048 pairs: as much LDS as the four waves' own buffers
struct MediumSegLds {
    SegLds lds;
    uint32_t ex_keys[kSegMediumCap], ex_vals[kSegMediumCap];
};
// Where the segments lie: either `offsets` holds their bounds (tile_ranges_kernel wrote them), or -- tile_count given --
// the last sweep of a sort by tile column and row left every tile's number of pairs, and the bounds are made here:
// a tile's first pair comes behind all pairs of the rows above it (row_totals, the digit totals of the sweep over
// the rows) and of the tiles to its left in its row.  The kernel then writes `offsets`.
__global__ __launch_bounds__(kSortThreads) void segment_sort_small_kernel(uint64_t *keys, uint32_t *vals, int32_t *offsets,
                                                                          int n_segments, const uint32_t *__restrict__ tile_count,
                                                                          const uint32_t *__restrict__ row_totals, int tiles_x,
                                                                          uint32_t n_pairs) {
    __shared__ union SmallLds {
        WaveSegLds wave[kSortWaves];
        MediumSegLds medium;
    } s;
    __shared__ int s_bounds[kSortWaves + 1];
    const int wave = threadIdx.x / kWave;
    const int first = blockIdx.x * kSortWaves;
    int bounds[kSortWaves + 1];
    if (tile_count) {
        const int lane = threadIdx.x & (kWave - 1);
        const int t = first + wave;
        if (t < n_segments) {
            const int ty = t / tiles_x, tx = t - ty * tiles_x;
            uint32_t sum = 0;
            for (int d = lane; d < ty; d += kWave) sum += row_totals[d];
            for (int x = lane; x < tx; x += kWave) sum += tile_count[t - tx + x];
            sum = wave_sum(sum);
            if (lane == 0) {
                // counts of a sort whose wait expired (the status word says so) may be anything: stay inside the arrays
                sum = sum < n_pairs ? sum : n_pairs;
                const uint32_t length = tile_count[t];
                s_bounds[wave] = (int)sum;
                offsets[t] = (int32_t)sum;
                const int end = (int)(length < n_pairs - sum ? sum + length : n_pairs);
                if (wave == kSortWaves - 1 || t == n_segments - 1) s_bounds[wave + 1] = end;
                if (t == n_segments - 1) offsets[n_segments] = end;
            }
        }
        __syncthreads();
        const int last = min(kSortWaves, n_segments - first);  // segments of this workgroup
#pragma unroll
        for (int w = 0; w <= kSortWaves; w++) bounds[w] = s_bounds[min(w, last)];
    } else {
#pragma unroll
        for (int w = 0; w <= kSortWaves; w++) bounds[w] = offsets[min(first + w, n_segments)];
    }
    bool any_medium = false;
    int start = 0, n = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) {
        const int len = bounds[w + 1] - bounds[w];
        any_medium = any_medium || (len > kSegWaveCap && len <= kSegMediumCap);
        if (w == wave) { start = bounds[w]; n = len; }
    }
    if (n > 1 && n <= kSegWaveCap) {
        WaveSegLds &lds = s.wave[wave];
        switch ((n + kWave - 1) / kWave) {
        case 1: segment_sort_in_wave<1>(keys, vals, start, n, lds); break;
        case 2: segment_sort_in_wave<2>(keys, vals, start, n, lds); break;
        case 3: segment_sort_in_wave<3>(keys, vals, start, n, lds); break;
        case 4: segment_sort_in_wave<4>(keys, vals, start, n, lds); break;
        case 5: segment_sort_in_wave<5>(keys, vals, start, n, lds); break;
        case 6: segment_sort_in_wave<6>(keys, vals, start, n, lds); break;
        default: segment_sort_in_wave<8>(keys, vals, start, n, lds); break;
        }
    }
    if (!any_medium) return;  // the same for the whole workgroup
#pragma unroll 1
    for (int w = 0; w < kSortWaves; w++) {
        const int len = bounds[w + 1] - bounds[w];
        if (len <= kSegWaveCap || len > kSegMediumCap) continue;
        __syncthreads();  // the waves are done with their own buffers, the previous segment with the shared one
        if (len <= kSortThreads * 4)
            segment_sort_in_lds<4>(keys, vals, bounds[w], len, s.medium.lds, s.medium.ex_keys, s.medium.ex_vals);
        else
            segment_sort_in_lds<kSegMediumItems>(keys, vals, bounds[w], len, s.medium.lds, s.medium.ex_keys, s.medium.ex_vals);
    }
}

// The workgroup sorts keys[start, start + n) by the low key word through memory: per 8-bit pass a histogram
// of the segment, then its chunks in order, every pair written to its final place of the pass in the other
// buffer pair.  The sorted segment ends in (keys, vals).
__device__ void segment_sort_through_memory(uint64_t *keys, uint32_t *vals, uint64_t *keys_alt, uint32_t *vals_alt, int64_t start,
                                            int n, SegLds &lds, uint32_t *hist /* [kRadix] */, uint32_t *next /* [kRadix] */) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    constexpr int kChunk = kSortThreads * kSegStreamItems;
    constexpr int kWaveSpan = kWave * kSegStreamItems;
    uint64_t *src_k = keys, *dst_k = keys_alt;
    uint32_t *src_v = vals, *dst_v = vals_alt;
#pragma unroll 1
    for (int p = 0; p < 4; p++) {
        const int shift = p * kRadixBits;
        hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < n; i += kSortThreads) atomicAdd(&hist[(uint32_t)(src_k[start + i] >> shift) & (kRadix - 1)], 1u);
        __syncthreads();
        const uint32_t mine = hist[tid];
        const bool uniform = __syncthreads_or(mine == (uint32_t)n);
        if (uniform) continue;  // one digit holds the whole segment: the pass would change nothing
        {
            const uint32_t incl = wave_inclusive_scan_u32(mine);
            if (lane == kWave - 1) lds.wave_total[wave] = incl;
            __syncthreads();
            uint32_t wave_prefix = 0;
            for (int w = 0; w < wave; w++) wave_prefix += lds.wave_total[w];
            next[tid] = wave_prefix + incl - mine;
        }
        __syncthreads();
        for (int c0 = 0; c0 < n; c0 += kChunk) {
            uint64_t key[kSegStreamItems];
            uint32_t val[kSegStreamItems], digit[kSegStreamItems], place[kSegStreamItems];
            int n_pad = 0;
#pragma unroll
            for (int i = 0; i < kSegStreamItems; i++) {
                const int pos = c0 + wave * kWaveSpan + i * kWave + lane;
                if (pos < n) {
                    key[i] = src_k[start + pos];
                    val[i] = src_v[start + pos];
                    digit[i] = (uint32_t)(key[i] >> shift) & (kRadix - 1);
                } else {
                    key[i] = 0;
                    val[i] = 0;
                    digit[i] = kRadix - 1;  // padding: last in the chunk, so behind every real pair of its digit
                }
            }
            n_pad = (c0 + kChunk > n) ? c0 + kChunk - n : 0;
            workgroup_digit_places<kSegStreamItems>(digit, lds, place);
            // place = position in the chunk's digit order; the pass position is the digit's running start plus
            // the rank among the chunk's pairs of that digit
#pragma unroll
            for (int i = 0; i < kSegStreamItems; i++) {
                const int pos = c0 + wave * kWaveSpan + i * kWave + lane;
                if (pos < n) {
                    const int64_t to = start + next[digit[i]] + (place[i] - lds.start[digit[i]]);
                    dst_k[to] = key[i];
                    dst_v[to] = val[i];
                }
            }
            __syncthreads();
            // the chunk's count of digit d = start[d + 1] - start[d]
            const uint32_t end = (tid == kRadix - 1) ? (uint32_t)kChunk - (uint32_t)n_pad : lds.start[tid + 1];
            const uint32_t begin = lds.start[tid];
            __syncthreads();
            next[tid] += (end > begin) ? end - begin : 0u;
            __syncthreads();
        }
        // the next pass reads what this one wrote
        __threadfence();
        __syncthreads();
        __threadfence();
        uint64_t *tk = src_k; src_k = dst_k; dst_k = tk;
        uint32_t *tv = src_v; src_v = dst_v; dst_v = tv;
    }
    if (src_k != keys) {
        for (int i = tid; i < n; i += kSortThreads) {
            keys[start + i] = src_k[start + i];
            vals[start + i] = src_v[start + i];
        }
    }
}

// Segments longer than kSegMediumCap: few or none, so a workgroup looks through the lengths of its share of the
// segments, one segment per thread at a time, and takes the long ones in turn.
__global__ __launch_bounds__(kSortThreads, 2) void segment_sort_large_kernel(uint64_t *keys, uint32_t *vals, uint64_t *keys_alt,
                                                                             uint32_t *vals_alt, const int32_t *__restrict__ offsets,
                                                                             int n_segments) {
    __shared__ SegLds lds;
    __shared__ uint32_t ex_keys[kSegLargeCap], ex_vals[kSegLargeCap];
    __shared__ uint64_t s_votes[kSortWaves];
    // workgroup b looks at the segments b, b + gridDim.x, ...: long segments that are neighbours go to different workgroups
    const int grid = (int)gridDim.x;
    for (int base = 0; (int64_t)base * grid < n_segments; base += kSortThreads) {
        const int mine = (base + (int)threadIdx.x) * grid + (int)blockIdx.x;
        const bool is_long = mine < n_segments && offsets[mine + 1] - offsets[mine] > kSegMediumCap;
        const uint64_t vote = __builtin_amdgcn_ballot_w64(is_long);
        __syncthreads();  // the round before is done with the votes, the segment before with the LDS
        if ((threadIdx.x & (kWave - 1)) == 0) s_votes[threadIdx.x / kWave] = vote;
        __syncthreads();
        for (int w = 0; w < kSortWaves; w++) {
            uint64_t todo = s_votes[w];
            while (todo) {  // the same for the whole workgroup
                const int seg = (base + w * kWave + __builtin_ctzll(todo)) * grid + (int)blockIdx.x;
                todo &= todo - 1;
                const int64_t start = offsets[seg];
                const int n = offsets[seg + 1] - offsets[seg];
                if (n <= kSortThreads * 16)
                    segment_sort_in_lds<16>(keys, vals, start, n, lds, ex_keys, ex_vals);
                else if (n <= kSegLargeCap)
                    segment_sort_in_lds<kSegLargeItems>(keys, vals, start, n, lds, ex_keys, ex_vals);
                else
                    segment_sort_through_memory(keys, vals, keys_alt, vals_alt, start, n, lds, ex_keys, ex_keys + kRadix);
                __syncthreads();  // the next segment reuses the LDS
            }
        }
    }
}

__global__ __launch_bounds__(kSortThreads) void tile_ranges_kernel(const uint64_t *__restrict__ sorted_keys, int64_t n_keys,
                                                                   int n_tiles, int32_t *__restrict__ offsets) {
    const int64_t i = (int64_t)blockIdx.x * kSortThreads + threadIdx.x;
    if (i > n_keys) return;
    const int cur = (i < n_keys) ? (int)(sorted_keys[i] >> 32) : n_tiles;
    const int prev = (i > 0) ? (int)(sorted_keys[i - 1] >> 32) : -1;
    for (int t = prev + 1; t <= cur && t <= n_tiles; t++) offsets[t] = (int32_t)i;
}

template <int BITS>
static void launch_sweep(dim3 grid, hipStream_t s, const uint64_t *kin, const uint32_t *vin, uint64_t *kout, uint32_t *vout,
                         int64_t n, int shift, uint32_t mask, const uint32_t *bases, int totals_given, uint32_t *lookback,
                         uint32_t *ticket, uint32_t *status, int unpad_bits, int tiles_x, uint32_t *tile_count) {
    hipLaunchKernelGGL(sort_sweep_kernel<BITS>, grid, dim3(kSweepThreads), 0, s, kin, vin, kout, vout, n, shift, mask, bases,
                       totals_given, lookback, ticket, status, unpad_bits, tiles_x, tile_count);
}

// The sweeps of `plan` over (keys, values) <-> (keys_alt, values_alt).  bases: per pass kRadix words, the
// exclusive scan of the digit totals or (totals_given) the totals; lookback: per pass n_sort_tiles * kRadix
// words, zero; tickets: one word per pass, zero.
// unpad_bits, tiles_x, tile_count: for the last pass of a sort by tile column and row (see the kernel), else 0.
static int run_sweeps(const char *fn, const PassPlan &plan, int n_sort_tiles, const uint32_t *bases, int totals_given,
                      uint32_t *lookback, uint32_t *tickets, uint64_t *keys, uint32_t *values, uint64_t *keys_alt,
                      uint32_t *values_alt, int64_t n, uint32_t *status, hipStream_t s, int unpad_bits = 0, int tiles_x = 0,
                      uint32_t *tile_count = nullptr) {
    uint64_t *kin = keys, *kout = keys_alt;
    uint32_t *vin = values, *vout = values_alt;
    // 534 same-address ticket atomics cost 6 us per pass; a grid that fits the device whole takes its
    // tile numbers from the workgroup ids instead
    static int resident_cache[kMaxDevices] = {0};
    const bool whole_grid_resident = n_sort_tiles <= resident_workgroups((const void *)sort_sweep_kernel<kRadixBits>, kSweepThreads, resident_cache);
    // one pair of timing events around all passes: a pair per launch would add its own two
    // microseconds to every 24 us kernel
    ProfileScope timed("sort_sweep_kernel", s, plan.passes);
    for (int p = 0; p < plan.passes; p++) {
        const dim3 grid(n_sort_tiles);
        const uint32_t mask = (1u << plan.bits[p]) - 1;
        uint32_t *lb = lookback + (size_t)p * lookback_words_per_pass(n_sort_tiles);
        uint32_t *ticket = whole_grid_resident ? (uint32_t *)nullptr : tickets + p;
        const uint32_t *b = bases + (size_t)p * kRadix * (totals_given ? kTotalsStride : 1);
        const bool last = p == plan.passes - 1;
        const int ub = last ? unpad_bits : 0;
        uint32_t *tc = last ? tile_count : (uint32_t *)nullptr;
        switch (plan.bits[p]) {
        case 8: launch_sweep<8>(grid, s, kin, vin, kout, vout, n, plan.shift[p], mask, b, totals_given, lb, ticket, status, ub, tiles_x, tc); break;
        case 7: launch_sweep<7>(grid, s, kin, vin, kout, vout, n, plan.shift[p], mask, b, totals_given, lb, ticket, status, ub, tiles_x, tc); break;
        case 6: launch_sweep<6>(grid, s, kin, vin, kout, vout, n, plan.shift[p], mask, b, totals_given, lb, ticket, status, ub, tiles_x, tc); break;
        case 5: launch_sweep<5>(grid, s, kin, vin, kout, vout, n, plan.shift[p], mask, b, totals_given, lb, ticket, status, ub, tiles_x, tc); break;
        default: launch_sweep<4>(grid, s, kin, vin, kout, vout, n, plan.shift[p], mask, b, totals_given, lb, ticket, status, ub, tiles_x, tc); break;
        }
        if (int e = check_launch(fn)) return e;
        uint64_t *tk = kin; kin = kout; kout = tk;
        uint32_t *tv = vin; vin = vout; vout = tv;
    }
    return 0;
}

// Histogram, bases and the sweeps of `plan`, everything in the workspace laid out by L.
static int run_passes(const char *fn, const PassPlan &plan, const SortLayout &L, char *ws, uint64_t *keys, uint32_t *values,
                      uint64_t *keys_alt, uint32_t *values_alt, int64_t n, uint32_t *status, hipStream_t s) {
    uint32_t *tickets = (uint32_t *)(ws + L.off_tickets);
    uint32_t *bases = (uint32_t *)(ws + L.off_bases);
    uint32_t *partials = (uint32_t *)(ws + L.off_partials);
    uint32_t *lookback = (uint32_t *)(ws + L.off_lookback);
    // tickets and look-back words (adjacent) start at zero; bases and partials are fully overwritten
    TG_LAUNCH(sort_histogram_kernel, dim3(L.hist_blocks), dim3(kHistThreads), 0, s, keys, n, plan, partials, tickets, L.zero_words);
    if (int e = check_launch("sort_histogram_kernel")) return e;
    TG_LAUNCH(sort_bases_kernel, dim3(plan.passes), dim3(kBasesThreads), 0, s, partials, L.hist_blocks, bases, status);
    if (int e = check_launch("sort_bases_kernel")) return e;
    return run_sweeps(fn, plan, L.n_tiles, bases, 0, lookback, tickets, keys, values, keys_alt, values_alt, n, status, s);
}

// Tile ranges of keys that are ordered by tile, then every tile's segment sorted by its depth bits in place.
// With tile_count (the last sweep counted every tile's pairs) the ranges come from the counts, inside the segment kernel.
static int ranges_and_segments(uint64_t *k, uint32_t *v, uint64_t *k_other, uint32_t *v_other, int64_t n, int n_tiles,
                               int32_t *offsets, hipStream_t s, const uint32_t *tile_count = nullptr,
                               const uint32_t *row_totals = nullptr, int tiles_x = 0) {
    if (!tile_count) {
        TG_LAUNCH(tile_ranges_kernel, dim3((unsigned)ceil_div64(n + 1, kSortThreads)), dim3(kSortThreads), 0, s, k, n, n_tiles, offsets);
        if (int e = check_launch("tile_ranges_kernel")) return e;
    }
    TG_LAUNCH(segment_sort_small_kernel, dim3(ceil_div(n_tiles, kSortWaves)), dim3(kSortThreads), 0, s, k, v, offsets, n_tiles,
              tile_count, row_totals, tiles_x, (uint32_t)n);
    if (int e = check_launch("segment_sort_small_kernel")) return e;
    TG_LAUNCH(segment_sort_large_kernel, dim3(n_tiles < kSegLargeGrid ? n_tiles : kSegLargeGrid), dim3(kSortThreads), 0, s, k, v,
              k_other, v_other, offsets, n_tiles);
    return check_launch("segment_sort_large_kernel");
}

static int check_sort_buffers(const char *fn, const void *keys, const void *values, const void *keys_alt, const void *values_alt,
                              const void *workspace) {
    if (!keys || !values || !keys_alt || !values_alt || !workspace) {
        set_error("%s: null pointer", fn);
        return TG_E_ARG;
    }
    if (((uintptr_t)keys & 7) || ((uintptr_t)keys_alt & 7) || ((uintptr_t)workspace & 255)) {
        set_error("%s: keys must be 8-byte aligned, workspace 256-byte aligned", fn);
        return TG_E_ARG;
    }
    return 0;
}

}  // namespace tg

using namespace tg;

extern "C" size_t tg_sort_workspace_bytes(int64_t n) {
    if (n < 0 || n > kSortMaxN) return 0;
    return sort_layout(n, kMaxPasses).total;
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
    if (int e = check_sort_buffers("tg_sort_pairs_u64_u32", keys, values, keys_alt, values_alt, workspace)) return e;
    const PassPlan plan = plan_passes(0, end_bit);
    const SortLayout L = sort_layout(n, plan.passes);
    if (workspace_bytes < L.total) {
        set_error("tg_sort_pairs_u64_u32: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
        return TG_E_WORKSPACE;
    }
    if (int e = run_passes("tg_sort_pairs_u64_u32", plan, L, (char *)workspace, keys, values, keys_alt, values_alt, n, status, s))
        return e;
    *result_in_alt = (plan.passes & 1);
    return 0;
}

extern "C" int tg_tile_ranges(const uint64_t *sorted_keys, int64_t n_keys, int n_tiles, int32_t *offsets, void *stream) {
    if (n_keys < 0 || n_keys > 0x7fffffffll || n_tiles <= 0 || !offsets || (n_keys > 0 && !sorted_keys)) {
        set_error("tg_tile_ranges: null pointer or size out of range");
        return TG_E_ARG;
    }
    TG_LAUNCH(tile_ranges_kernel, dim3((unsigned)ceil_div64(n_keys + 1, kSortThreads)), dim3(kSortThreads), 0,
                       (hipStream_t)stream, sorted_keys, n_keys, n_tiles, offsets);
    return check_launch("tile_ranges_kernel");
}

extern "C" size_t tg_tile_list_sort_workspace_bytes(int64_t n, int n_tiles) {
    if (n < 0 || n > kSortMaxN || n_tiles <= 0) return 0;
    return sort_layout(n, kMaxPasses / 2).total;
}

// (keys, values): n > 0 pairs in any order -> tile passes with a histogram of their own, ranges, segments.
static int sort_tile_lists_run(const char *fn, uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int64_t n,
                               int n_tiles, int32_t *offsets, void *workspace, size_t workspace_bytes, uint32_t *status,
                               int *result_in_alt, hipStream_t s) {
    if (int e = check_sort_buffers(fn, keys, values, keys_alt, values_alt, workspace)) return e;
    const PassPlan plan = tile_pass_plan(n_tiles);
    const SortLayout L = sort_layout(n, plan.passes);
    if (workspace_bytes < L.total) {
        set_error("%s: workspace of %zu bytes, need %zu", fn, workspace_bytes, L.total);
        return TG_E_WORKSPACE;
    }
    char *ws = (char *)workspace;
    if (int e = run_passes(fn, plan, L, ws, keys, values, keys_alt, values_alt, n, status, s)) return e;
    uint64_t *k = (plan.passes & 1) ? keys_alt : keys, *k_other = (plan.passes & 1) ? keys : keys_alt;
    uint32_t *v = (plan.passes & 1) ? values_alt : values, *v_other = (plan.passes & 1) ? values : values_alt;
    *result_in_alt = (plan.passes & 1);
    return ranges_and_segments(k, v, k_other, v_other, n, n_tiles, offsets, s);
}

extern "C" int tg_sort_tile_lists(uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int64_t n,
                                  int n_tiles, int32_t *offsets, void *workspace, size_t workspace_bytes, uint32_t *status,
                                  int *result_in_alt, void *stream) {
    if (n < 0 || n > kSortMaxN || n_tiles <= 0 || !offsets || !result_in_alt) {
        set_error("tg_sort_tile_lists: n must be in [0, 2^30), n_tiles positive, offsets and result_in_alt given");
        return TG_E_ARG;
    }
    *result_in_alt = 0;
    hipStream_t s = (hipStream_t)stream;
    if (n == 0) {
        // no keys: the thread of key position 0 writes offsets[t] = 0 for every t
        TG_LAUNCH(tile_ranges_kernel, dim3(1), dim3(kSortThreads), 0, s, keys, n, n_tiles, offsets);
        if (int e = check_launch("tile_ranges_kernel")) return e;
        if (status) {
            TG_LAUNCH(fill_zero_kernel, dim3(1), dim3(64), 0, s, status, (size_t)1);
            if (int e = check_launch("fill_zero_kernel")) return e;
        }
        return 0;
    }
    return sort_tile_lists_run("tg_sort_tile_lists", keys, values, keys_alt, values_alt, n, n_tiles, offsets, workspace,
                               workspace_bytes, status, result_in_alt, s);
}

// ---- emission + tile lists of a frame -----------------------------------------------------------------
static size_t build_lookback_bytes(int64_t n_keys, int n_tiles) {
    const PassPlan plan = tile_pass_plan(n_tiles);
    const int64_t n_sort_tiles = ceil_div64(n_keys, kSortTile);
    return (size_t)plan.passes * lookback_words_per_pass(n_sort_tiles > 0 ? n_sort_tiles : 1) * 4;
}

constexpr size_t kFrameSortHeadBytes = 256;  // tg_build_frame_lists: the sweeps' tickets in front of the look-back words
extern "C" size_t tg_build_tile_lists_workspace_bytes(int64_t n_keys, int n_tiles) {
    if (n_keys < 0 || n_keys > kSortMaxN || n_tiles <= 0) return 0;
    if (!binning_counts_digits(n_tiles)) return tg_tile_list_sort_workspace_bytes(n_keys, n_tiles);
    return build_lookback_bytes(n_keys, n_tiles) + kFrameSortHeadBytes;
}

extern "C" int tg_build_tile_lists(const real *records, const uint32_t *tri_offsets, int32_t n_triangles, int64_t n_keys,
                                   uint32_t head_capacity, const uint32_t *heads, void *frame, int width, int height, int tile_w,
                                   int tile_h, uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt,
                                   int32_t *offsets, void *workspace, size_t workspace_bytes, uint32_t *status, int emit_only,
                                   int *result_in_alt, void *stream) {
    if (n_keys < 0 || n_keys > kSortMaxN || n_triangles < 0 || width <= 0 || height <= 0 || tile_w <= 0 || tile_h <= 0 || !frame ||
        !result_in_alt || (!emit_only && !offsets)) {
        set_error("tg_build_tile_lists: n_keys must be in [0, 2^30), sizes positive, frame state, offsets and result_in_alt given");
        return TG_E_ARG;
    }
    *result_in_alt = 0;
    hipStream_t s = (hipStream_t)stream;
    const int n_tiles = ceil_div(width, tile_w) * ceil_div(height, tile_h);
    if (n_keys == 0) {
        if (status) {
            TG_LAUNCH(fill_zero_kernel, dim3(1), dim3(64), 0, s, status, (size_t)1);
            if (int e = check_launch("fill_zero_kernel")) return e;
        }
        if (emit_only) return 0;
        TG_LAUNCH(tile_ranges_kernel, dim3(1), dim3(kSortThreads), 0, s, keys, n_keys, n_tiles, offsets);
        return check_launch("tile_ranges_kernel");
    }
    if (!records || !tri_offsets || !keys || !values || ((uintptr_t)keys & 7) || ((uintptr_t)records & (4 * sizeof(real) - 1))) {
        set_error("tg_build_tile_lists: null or misaligned records, offsets, keys or values");
        return TG_E_ARG;
    }
    if (emit_only)
        return launch_emit_records("bin_emit_records_kernel", records, tri_offsets, n_triangles, n_keys, head_capacity, heads, frame,
                                   width, height, tile_w, tile_h, keys, values, nullptr, 0, status, s);
    if (sizeof(real) != 4) {
        set_error("tg_build_tile_lists: the double build's depth keys take all 64 key bits; emit only, then sort by depth and by tile");
        return TG_E_ARG;
    }
    if (!binning_counts_digits(n_tiles)) {
        if (int e = launch_emit_records("bin_emit_records_kernel", records, tri_offsets, n_triangles, n_keys, head_capacity, heads,
                                        frame, width, height, tile_w, tile_h, keys, values, nullptr, 0, status, s))
            return e;
        return sort_tile_lists_run("tg_build_tile_lists", keys, values, keys_alt, values_alt, n_keys, n_tiles, offsets, workspace,
                                   workspace_bytes, status, result_in_alt, s);
    }
    if (int e = check_sort_buffers("tg_build_tile_lists", keys, values, keys_alt, values_alt, workspace)) return e;
    const size_t lookback_bytes = build_lookback_bytes(n_keys, n_tiles);
    if (workspace_bytes < lookback_bytes) {
        set_error("tg_build_tile_lists: workspace of %zu bytes, need %zu", workspace_bytes, lookback_bytes);
        return TG_E_WORKSPACE;
    }
    uint32_t *lookback = (uint32_t *)workspace;
    // the emission clears the look-back words and the status word; the digit totals are the binning kernel's
    if (int e = launch_emit_records("bin_emit_records_kernel", records, tri_offsets, n_triangles, n_keys, head_capacity, heads, frame,
                                    width, height, tile_w, tile_h, keys, values, lookback, lookback_bytes / 4, status, s))
        return e;
    const PassPlan plan = tile_pass_plan(n_tiles);
    const int tiles_x = ceil_div(width, tile_w), tiles_y = ceil_div(height, tile_h);
    uint32_t *tickets = frame_tickets(frame);
    if (int e = run_sweeps("tg_build_tile_lists", plan, (int)ceil_div64(n_keys, kSortTile), frame_totals(frame, n_triangles, tiles_x, tiles_y),
                           1, lookback, tickets + kSweepTicketWord, keys, values, keys_alt, values_alt, n_keys, status, s))
        return e;
    uint64_t *k = (plan.passes & 1) ? keys_alt : keys, *k_other = (plan.passes & 1) ? keys : keys_alt;
    uint32_t *v = (plan.passes & 1) ? values_alt : values, *v_other = (plan.passes & 1) ? values : values_alt;
    *result_in_alt = (plan.passes & 1);
    return ranges_and_segments(k, v, k_other, v_other, n_keys, n_tiles, offsets, s);
}

// ---- the tile lists of a frame whose keys tg_bin_frame emitted ------------------------------------------
// Workspace: the sweeps' tickets, their look-back words, then one count per tile (and one to spare).
static size_t frame_lists_count_offset(int64_t n_keys, int n_tiles) { return kFrameSortHeadBytes + build_lookback_bytes(n_keys, n_tiles); }

extern "C" size_t tg_build_frame_lists_workspace_bytes(int64_t n_keys, int tiles_x, int tiles_y) {
    if (n_keys < 0 || n_keys > kSortMaxN || tiles_x <= 0 || tiles_y <= 0 || (int64_t)tiles_x * tiles_y > 0x7fffffff) return 0;
    const int n_tiles = tiles_x * tiles_y;
    if (!grid_plan(tiles_x, tiles_y).on) return tg_tile_list_sort_workspace_bytes(n_keys, n_tiles);
    // two passes of at most 256 digits each
    return kFrameSortHeadBytes + 2 * lookback_words_per_pass(ceil_div64(n_keys > 0 ? n_keys : 1, kSortTile)) * 4 + (size_t)(n_tiles + 1) * 4;
}

extern "C" int tg_build_frame_lists(void *frame, uint32_t epoch, int64_t n_keys, int tiles_x, int tiles_y, uint64_t *keys,
                                    uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int32_t *offsets, void *workspace,
                                    size_t workspace_bytes, uint32_t *status, int *result_in_alt, void *stream) {
    if (n_keys < 0 || n_keys > kSortMaxN || tiles_x <= 0 || tiles_y <= 0 || (int64_t)tiles_x * tiles_y > 0x7fffffff || !frame ||
        !result_in_alt || !offsets) {
        set_error("tg_build_frame_lists: n_keys must be in [0, 2^30), tile counts positive, frame state, offsets and result_in_alt given");
        return TG_E_ARG;
    }
    *result_in_alt = 0;
    hipStream_t s = (hipStream_t)stream;
    if (sizeof(real) != 4) {
        set_error("tg_build_frame_lists: float build only");
        return TG_E_ARG;
    }
    const int n_tiles = tiles_x * tiles_y;
    if (n_keys == 0) {
        TG_LAUNCH(tile_ranges_kernel, dim3(1), dim3(kSortThreads), 0, s, keys, n_keys, n_tiles, offsets);
        return check_launch("tile_ranges_kernel");
    }
    const GridPlan grid = grid_plan(tiles_x, tiles_y);
    if (!grid.on)
        return sort_tile_lists_run("tg_build_frame_lists", keys, values, keys_alt, values_alt, n_keys, n_tiles, offsets, workspace,
                                   workspace_bytes, status, result_in_alt, s);
    if (int e = check_sort_buffers("tg_build_frame_lists", keys, values, keys_alt, values_alt, workspace)) return e;
    const int n_sort_tiles = (int)ceil_div64(n_keys, kSortTile);
    const size_t lookback_bytes = 2 * lookback_words_per_pass(n_sort_tiles) * 4;
    const size_t need = kFrameSortHeadBytes + lookback_bytes + (size_t)(n_tiles + 1) * 4;
    if (workspace_bytes < need) {
        set_error("tg_build_frame_lists: workspace of %zu bytes, need %zu", workspace_bytes, need);
        return TG_E_WORKSPACE;
    }
    uint32_t *tickets = (uint32_t *)workspace;
    uint32_t *lookback = (uint32_t *)((char *)workspace + kFrameSortHeadBytes);
    uint32_t *tile_count = (uint32_t *)((char *)workspace + kFrameSortHeadBytes + lookback_bytes);
    const uint32_t *totals = fused_frame_totals(frame, epoch);
    if (int e = run_sweeps("tg_build_frame_lists", grid.plan, n_sort_tiles, totals, 1, lookback, tickets, keys, values, keys_alt,
                           values_alt, n_keys, status, s, grid.column_bits, tiles_x, tile_count))
        return e;
    // two passes: the sorted pairs are back in (keys, values)
    return ranges_and_segments(keys, values, keys_alt, values_alt, n_keys, n_tiles, offsets, s, tile_count, totals + kRadix, tiles_x);
}
