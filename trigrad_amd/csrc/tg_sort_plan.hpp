// tg_sort_plan.hpp -- digit positions and workspace layout of the radix sort, shared by the sort and by the key
// emission (which counts the tile digits of the keys it writes and clears the sweeps' look-back words).
#pragma once
#include "tg_common.hpp"

namespace tg {

constexpr int kRadixBits = 8;  // widest digit
constexpr int kRadix = 1 << kRadixBits;
constexpr int kMaxPasses = 8;
constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;
#ifndef TG_SORT_ITEMS
#define TG_SORT_ITEMS 16
#endif
constexpr int kSortItems = TG_SORT_ITEMS;
constexpr int kSortTile = kSortThreads * kSortItems;  // 4096 pairs
#ifndef TG_SWEEP_THREADS
#define TG_SWEEP_THREADS 512
#endif
constexpr int kSweepThreads = TG_SWEEP_THREADS;  // the sweep spreads a tile over more waves than it has digits to own
constexpr int kSweepWaves = kSweepThreads / kWave;
constexpr int kSweepItems = kSortTile / kSweepThreads;
constexpr int kHistBlocksMax = 256;
constexpr int kBasesThreads = 1024;
constexpr int kLookWindow = 8;  // look-back words a digit's thread reads per round trip
constexpr int kLookGroup = 32;  // sort tiles whose counts are read directly; the look-back proper runs over groups of them
constexpr uint32_t kSortSpinLimit = 1u << 20;
constexpr uint32_t kLbAggregate = 1u << 30;
constexpr uint32_t kLbInclusive = 2u << 30;
constexpr uint32_t kLbValueMask = (1u << 30) - 1;
constexpr int64_t kSortMaxN = (1ll << 30) - 1;

// The digit positions of a sort on key bits [begin_bit, end_bit): as few passes of at most 8 bits as
// cover them, of equal width up to one bit (45 bits: 8 8 8 7 7 7; the 13 tile bits of 1920x1080: 7 6).
struct PassPlan {
    int passes;
    int shift[kMaxPasses];
    int bits[kMaxPasses];
};

inline PassPlan plan_passes(int begin_bit, int end_bit) {
    PassPlan plan;
    const int n_bits = end_bit - begin_bit;
    plan.passes = n_bits <= 0 ? 0 : (n_bits + kRadixBits - 1) / kRadixBits;
    int at = begin_bit;
    for (int p = 0; p < kMaxPasses; p++) {
        const int width = p < plan.passes ? n_bits / plan.passes + (p < n_bits % plan.passes ? 1 : 0) : 0;
        plan.shift[p] = at;
        plan.bits[p] = width;
        at += width;
    }
    return plan;
}

// Look-back words of one pass: a row of kRadix per sort tile, then a row per group of tiles.
inline size_t lookback_words_per_pass(int64_t n_sort_tiles) {
    return (size_t)(n_sort_tiles + ceil_div64(n_sort_tiles, kLookGroup)) * kRadix;
}

struct SortLayout {
    int n_tiles;
    int hist_blocks;
    size_t off_tickets, off_partials, off_bases, off_lookback, total;
    size_t zero_words;  // words from off_tickets on that must be zero before the sweeps start
};

inline SortLayout sort_layout(int64_t n, int passes) {
    SortLayout L;
    L.n_tiles = (int)ceil_div64(n, kSortTile);
    L.hist_blocks = L.n_tiles < kHistBlocksMax ? (L.n_tiles > 0 ? L.n_tiles : 1) : kHistBlocksMax;
    size_t o = 0;
    L.off_bases = o;    o += (size_t)kMaxPasses * kRadix * 4;
    L.off_partials = o; o += (size_t)kHistBlocksMax * kMaxPasses * kRadix * 4;
    L.off_tickets = o;  o += 256;  // kMaxPasses tickets; zeroed with the look-back words
    L.off_lookback = o; o += (size_t)passes * lookback_words_per_pass(L.n_tiles > 0 ? L.n_tiles : 1) * 4;
    L.zero_words = (o - L.off_tickets) / 4;
    L.total = o;
    return L;
}
constexpr int kSweepTicketWord = 8;  // the sweeps' tickets inside the frame state of tg_bin_setup
constexpr int kTotalsStride = 1;  // words between two digit totals (a cache line each was tried: the atomics got no faster)


// Key bits that hold a tile number below n_tiles (at least one).
inline int tile_bits_of(int n_tiles) {
    int bits = 1;
    while (bits < 32 && (1ll << bits) < (int64_t)n_tiles) bits++;
    return bits;
}
inline PassPlan tile_pass_plan(int n_tiles) { return plan_passes(32, 32 + tile_bits_of(n_tiles)); }

// The binning counts the digits of at most this many tile passes (65536 tiles) for the sort; with more tiles,
// and in the double build (whose depth keys take all 64 bits), the sort makes its own histogram.
constexpr int kEmitDigitPasses = 2;
inline bool binning_counts_digits(int n_tiles) { return sizeof(real) == 4 && tile_pass_plan(n_tiles).passes <= kEmitDigitPasses; }


// Key emission from the triangle records of the frame's binning (tg_binning.hip); it clears zero_words words
// at `zero` and *clear_word.  The frame state's digit totals come from the binning kernel.
int launch_emit_records(const char *fn, const real *records, const uint32_t *tri_offsets, int32_t n_triangles, int64_t n_keys,
                        uint32_t owner_capacity, const uint32_t *owner_heads, void *frame, int width, int height, int tile_w,
                        int tile_h, uint64_t *keys, uint32_t *payload, uint32_t *zero, size_t zero_words, uint32_t *clear_word,
                        hipStream_t s);
uint32_t *frame_totals(void *frame, int32_t n_triangles, int tiles_x, int tiles_y);
uint32_t *frame_tickets(void *frame);
// The digit totals that tg_bin_frame(frame, epoch) counted.
uint32_t *fused_frame_totals(void *frame, uint32_t epoch);

// The sort of a frame whose binning is tg_bin_frame.  A tile number ty * tiles_x + tx orders like the pair (ty, tx),
// so two stable passes, by tile column and then by tile row, sort by tile.  The keys carry the pair as
// ty << column_bits | tx in their high word until the second pass, which writes the tile number in its place.
// The digits are then coordinates of the triangle's tile rectangle: every column of it holds as many keys as the
// rectangle has rows, so the binning counts a pass's digits with two additions per triangle to a difference
// array instead of one per key.  Up to 256 tile columns and rows; other frames sort on the bits of the tile
// number with a histogram of their own.
struct GridPlan {
    bool on;
    int column_bits, row_bits;
    PassPlan plan;
};
inline GridPlan grid_plan(int tiles_x, int tiles_y) {
    GridPlan g;
    g.column_bits = tile_bits_of(tiles_x);
    g.row_bits = tile_bits_of(tiles_y);
    g.on = sizeof(real) == 4 && g.column_bits <= kRadixBits && g.row_bits <= kRadixBits;
    g.plan = plan_passes(32, 32);
    g.plan.passes = 2;
    g.plan.shift[0] = 32; g.plan.bits[0] = g.column_bits;
    g.plan.shift[1] = 32 + g.column_bits; g.plan.bits[1] = g.row_bits;
    return g;
}

}  // namespace tg
