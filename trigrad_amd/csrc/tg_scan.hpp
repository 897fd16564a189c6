// tg_scan.hpp -- the decoupled look-back of the single-pass prefix sums (the scan of counts, and the
// binning kernel that counts and scans in one launch).
#pragma once
#include "tg_common.hpp"

namespace tg {

constexpr int kScanThreads = 512;
constexpr int kScanTile = kScanThreads * 4;
constexpr uint32_t kSpinLimit = 1u << 20;

constexpr uint64_t kFlagAggregate = 1ull << 62;
constexpr uint64_t kFlagInclusive = 2ull << 62;

__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
    v = wave_inclusive_scan_u32(v);
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// Called by the first wave of the workgroup that owns `tile` (all 64 lanes), after the tile's total is known:
// publishes it, sums the totals of all earlier tiles from their state words (64 predecessors per step),
// publishes the inclusive prefix and returns the exclusive one (in every lane).  The last tile also writes
// the grand total.  A wait that expires is recorded in *status and the sum carries on with what it has.
__device__ __forceinline__ uint32_t scan_tile_prefix(uint64_t *states, int tile, uint32_t tile_total, int n_tiles, uint32_t *total,
                                                     uint32_t *status) {
    const int lane = threadIdx.x & (kWave - 1);
    if (lane == 0) {
        uint64_t word = (tile == 0 ? kFlagInclusive : kFlagAggregate) | tile_total;
        __hip_atomic_store(&states[tile], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    uint32_t prefix = 0;
    bool timed_out = false;
    for (int look = tile - 1; look >= 0; look -= kWave) {
        const int idx = look - lane;
        uint64_t word = kFlagInclusive;  // before the first tile: inclusive prefix 0
        if (idx >= 0) {
            uint32_t spins = 0;
            word = __hip_atomic_load(&states[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            while ((word >> 62) == 0 && spins < kSpinLimit) {
                __builtin_amdgcn_s_sleep(1);
                word = __hip_atomic_load(&states[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                spins++;
            }
            if ((word >> 62) == 0) timed_out = true;
        }
        const uint64_t inclusive_lanes = __builtin_amdgcn_ballot_w64((word >> 62) == 2);
        const int first = inclusive_lanes ? __builtin_ctzll(inclusive_lanes) : kWave;
        prefix += wave_sum(lane <= first ? (uint32_t)word : 0u);
        if (inclusive_lanes) break;
    }
    if (__builtin_amdgcn_ballot_w64(timed_out) && lane == 0 && status) *status = TG_STATUS_LOOKBACK_TIMEOUT;
    if (lane == 0) {
        if (tile != 0)
            __hip_atomic_store(&states[tile], kFlagInclusive | (uint64_t)(prefix + tile_total), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        if (tile == n_tiles - 1) *total = prefix + tile_total;
    }
    return prefix;
}

}  // namespace tg
