// tg_backward.hip -- backward of the tile compositor, one workgroup per tile.
//
// Fragments are visited in exact reverse blend order; the transmittance in front
// of a fragment is reconstructed by dividing the running value by (1 - opacity),
// as the reference does (render.cu:492).
//
// Each fragment yields 21 gradient terms (3 vertices x {x, y, w, r, g, b,
// opacity}; the z gradient is identically zero, render.cu:531-533).  Terms of
// the same list entry are added up inside a wave before they reach memory, so
// the kernels issue one global floating-point atomic per (wave, run of equal
// entries, term) instead of 24 per (pixel, entry).
//
// per_pixel_sort = 0 (backward_tile_order_kernel): all pixels of a tile share
//   the list order, so the tile's list is walked backwards in LDS-staged
//   batches of 64 entries.
// per_pixel_sort = 1, max_layers <= 32 (backward_saved_order_kernel): every
//   pixel walks the blend order the forward pass saved for it, backwards.
// per_pixel_sort = 1, max_layers > 32 (backward_pixel_order_kernel): the pixel
//   re-selects its fragments from the far end (32 at a time, below the (depth,
//   position) of the last blended fragment saved by the forward pass).
#include "tg_raster.hpp"

namespace tg {

struct BackwardArgs {
    const real4 *grad_image;
    const real *grad_depthmap;
    const real4 *image;
    const real *depthmap;
    const real *weights;
    const int32_t *ends;
    const int32_t *last;
    const real *last_depth;
    const uint16_t *fragments;  // saved by the forward pass (low halves, then high halves for long lists), or null
    const uint64_t *hit_masks; // saved by the tile-order forward pass, or null
    real *grad_vertices;
    real *grad_colors;
    real *grad_opacities;
    int vertex_stride, color_stride, opacity_stride;  // scalars from one vertex to the next in the three arrays
};

// process_backward's inputs for one list entry.
struct alignas(16) BackRecord {
    real m[9];
    real w[3];
    real iw[3];
    real iw2[3];  // 1 / (w * w)
    real op[3];
    real col[9];
    real xy[6];   // ax, ay, bx, by, cx, cy
    int id[3];
};
constexpr int kBackReals = 36;  // scalars in front of the ids
static_assert(offsetof(BackRecord, id) == kBackReals * sizeof(real), "BackRecord layout");

// 1 / x to within one unit in the last place: the hardware estimate and one Newton step where
// the estimate is an ordinary number (zero, infinity and NaN pass through as they are).  Used
// where the reference divides in its backward pass and the quotient is no carried state.
__device__ __forceinline__ float reciprocal(float x) {
    const float r = __builtin_amdgcn_rcpf(x);
    const float refined = __builtin_fmaf(__builtin_fmaf(-x, r, 1.0f), r, r);
    return __builtin_amdgcn_classf(r, 0x198) ? refined : r;  // +-normal, +-denormal
}
__device__ __forceinline__ double reciprocal(double x) { return 1.0 / x; }

__device__ __forceinline__ void gather_back(const RasterArgs &a, int j, BackRecord &r) {
    const TriIds t = load_ids(a, j);
    const real *m = a.bary + 9 * (int64_t)t.tri;
#pragma unroll
    for (int k = 0; k < 9; k++) r.m[k] = m[k];
    const real4 va = a.vertices[t.ia], vb = a.vertices[t.ib], vc = a.vertices[t.ic];
    r.w[0] = va.w; r.w[1] = vb.w; r.w[2] = vc.w;
    // gradients only: 1 / w to within one unit in the last place, and its square for 1 / (w * w)
    r.iw[0] = reciprocal(va.w); r.iw[1] = reciprocal(vb.w); r.iw[2] = reciprocal(vc.w);
    r.iw2[0] = r.iw[0] * r.iw[0]; r.iw2[1] = r.iw[1] * r.iw[1]; r.iw2[2] = r.iw[2] * r.iw[2];
    r.op[0] = a.opacities[t.ia]; r.op[1] = a.opacities[t.ib]; r.op[2] = a.opacities[t.ic];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        r.col[k] = a.colors[3 * (int64_t)t.ia + k];
        r.col[3 + k] = a.colors[3 * (int64_t)t.ib + k];
        r.col[6 + k] = a.colors[3 * (int64_t)t.ic + k];
    }
    r.xy[0] = va.x; r.xy[1] = va.y; r.xy[2] = vb.x; r.xy[3] = vb.y; r.xy[4] = vc.x; r.xy[5] = vc.y;
    r.id[0] = t.ia; r.id[1] = t.ib; r.id[2] = t.ic;
}


// Reverse-traversal state of one pixel (render.cu:647-653).
struct BackState {
    real final_alpha, alpha, s0, s1, s2, oa, zoa, final_weight, final_depth;
    real inv_final_weight;  // the reference divides two terms of every fragment by the pixel's final weight
    real g0, g1, g2, g3, gd;  // upstream gradient of this pixel
};

constexpr int kTerms = 21;  // per vertex v: [7v+0] x, [7v+1] y, [7v+2] w, [7v+3..5] rgb, [7v+6] opacity

// util.h:299-317 scalar interpolate3_backward.
__device__ __forceinline__ void interp_backward_scalar(real g, const real b[3], const real v[3], const real w[3],
                                                       real gb[3], real gv[3], real gw[3]) {
    const real nom = (b[0] * w[0] * v[0] + b[1] * w[1] * v[1]) + b[2] * w[2] * v[2];
    const real denom = (b[0] * w[0] + b[1] * w[1]) + b[2] * w[2];
    // all zero where the reference returns early (util.h:303); written as selections, because a branch
    // around the assignments of three arrays makes the compiler keep them in scratch memory
    const bool dead = denom * denom < kEffZero;
    const real inv = reciprocal(denom);  // the reference divides nine times, by denom and by its square
    const real inv2 = inv * inv;
#pragma unroll
    for (int k = 0; k < 3; k++) {
        gb[k] = dead ? 0.0f : g * ((v[k] * w[k] * denom - nom * w[k]) * inv2);
        gv[k] = dead ? 0.0f : g * b[k] * w[k] * inv;
        gw[k] = dead ? 0.0f : g * (b[k] * v[k] * denom - nom * b[k]) * inv2;
    }
}

// process_backward (render.cu:455-538) is evaluated in two parts.  The part that
// carries state from one fragment of a pixel to the next (transmittance and the
// running sums) has to follow the reverse blend order of that pixel; it reduces
// the fragment to five numbers.  Everything else is a function of those five
// numbers, the pixel position and the triangle, and can be evaluated in any
// order.

// What the ordered part hands over for one fragment.
struct FragSeed {
    real d_do;    // derivative w.r.t. the interpolated opacity (:502)
    real gc[3];   // derivative w.r.t. the interpolated colour (:510)
    real dd_dz;   // derivative w.r.t. the interpolated view depth (:517)
};

// The fragment itself: interpolated opacity, colour and view depth (no state involved).
struct FragValue {
    real o, color[3], z;
};

__device__ __forceinline__ FragValue fragment_value(const BackRecord &r, real b0, real b1, real b2) {
    const real w[3] = {r.w[0], r.w[1], r.w[2]};
    FragValue v;
    // The opacity is recomputed exactly as the forward pass computed it: 1 - o can be small, and the
    // transmittance is reconstructed by dividing by it.  The three colour quotients over the same
    // denominator (util.h:245-250) share its reciprocal.
    v.o = clampf(interp_w(b0, b1, b2, r.op[0], r.op[1], r.op[2], w[0], w[1], w[2]), 0.0f, kMaxOpacity);
    const real inv_denom = reciprocal(b0 * w[0] + b1 * w[1] + b2 * w[2]);
#pragma unroll
    for (int k = 0; k < 3; k++)
        v.color[k] = (b0 * r.col[k] * w[0] + b1 * r.col[3 + k] * w[1] + b2 * r.col[6 + k] * w[2]) * inv_denom;
    v.z = interp_1(b0, b1, b2, r.iw[0], r.iw[1], r.iw[2]);
    return v;
}

// The step from one fragment of a pixel to the next one in reverse blend order (render.cu:487-517).
__device__ __forceinline__ FragSeed fragment_chain_step(BackState &st, const FragValue &v) {
    const real o = v.o, z = v.z;
    const real color[3] = {v.color[0], v.color[1], v.color[2]};
    const real om = 1.0f - o;
    const real inv_om = reciprocal(om);  // the reference divides six derivative terms by om
    const real g[3] = {st.g0, st.g1, st.g2};
    real s[3] = {st.s0, st.s1, st.s2};
    real t3[3];
#pragma unroll
    for (int k = 0; k < 3; k++) t3[k] = (color[k] * st.alpha - s[k]) * inv_om * g[k];
    const real drgb_do = ((t3[0] + t3[1]) + t3[2]) + st.g3 * (-st.final_alpha * inv_om);  // :491
    st.alpha /= om;                                                                        // :492 (state: kept exact)
#pragma unroll
    for (int k = 0; k < 3; k++) s[k] += color[k] * o * st.alpha;                       // :493
    st.s0 = s[0]; st.s1 = s[1]; st.s2 = s[2];
    const real ddw_do = st.alpha - st.oa * inv_om;                                    // :494
    const real dud_do = st.alpha * z - st.zoa * inv_om;                               // :495
    st.oa = st.oa + o * st.alpha;                                                      // :496
    st.zoa = st.zoa + z * o * st.alpha;                                                // :497
    real dd_do = (dud_do - st.final_depth * ddw_do) * st.inv_final_weight * st.gd;    // :499
    if (st.final_weight < kEffZero) dd_do = 0.0f;
    FragSeed f;
    f.d_do = drgb_do + dd_do;
    const real ao = st.alpha * o;
    f.gc[0] = ao * g[0]; f.gc[1] = ao * g[1]; f.gc[2] = ao * g[2];                     // :510
    f.dd_dz = ao * st.gd * st.inv_final_weight;                                        // :517
    if (st.final_weight < kEffZero) f.dd_dz = 0.0f;
    return f;
}

__device__ __forceinline__ FragSeed fragment_state_step(BackState &st, const BackRecord &r, real b0, real b1, real b2) {
    return fragment_chain_step(st, fragment_value(r, b0, b1, b2));
}

// The order-free part: the 21 gradient terms of one fragment.
__device__ __forceinline__ void fragment_terms(const FragSeed &f, const BackRecord &r, real b0, real b1, real b2, real px,
                                               real py, real out[kTerms]) {
    const real b[3] = {b0, b1, b2};
    const real w[3] = {r.w[0], r.w[1], r.w[2]};
    const real ones[3] = {1.0f, 1.0f, 1.0f};
    real gb_o[3], gv_o[3], gw_o[3];
    interp_backward_scalar(f.d_do, b, r.op, w, gb_o, gv_o, gw_o);

    // vector interpolate3_backward for the colour (util.h:319-355)
    const real *gc = f.gc;
    real gb_c[3], gw_c[3], scale[3];
    {
        real nom[3];
#pragma unroll
        for (int k = 0; k < 3; k++) nom[k] = (b[0] * w[0] * r.col[k] + b[1] * w[1] * r.col[3 + k]) + b[2] * w[2] * r.col[6 + k];
        const real denom = b[0] * w[0] + b[1] * w[1] + b[2] * w[2];
        const bool dead = denom * denom < kEffZero;  // util.h:326: all zero (selections, not a branch: see above)
        const real inv = reciprocal(denom);
        const real inv2 = inv * inv;
#pragma unroll
        for (int v = 0; v < 3; v++) {
            real dfb[3], dfw[3];
#pragma unroll
            for (int k = 0; k < 3; k++) {
                const real a = r.col[3 * v + k];
                dfb[k] = w[v] * (a * denom - nom[k]) * inv2;
                dfw[k] = (b[v] * a * denom - nom[k] * b[v]) * inv2;
            }
            gb_c[v] = dead ? 0.0f : (gc[0] * dfb[0] + gc[1] * dfb[1]) + gc[2] * dfb[2];
            gw_c[v] = dead ? 0.0f : (gc[0] * dfw[0] + gc[1] * dfw[1]) + gc[2] * dfw[2];
            scale[v] = dead ? 0.0f : b[v] * w[v] * inv;
        }
    }

    real gb_z[3], gv_z[3], gw_z[3];
    interp_backward_scalar(f.dd_dz, b, r.iw, ones, gb_z, gv_z, gw_z);

    real gbary[3];
#pragma unroll
    for (int k = 0; k < 3; k++) gbary[k] = gb_o[k] + gb_c[k] + gb_z[k];  // :527

    // util.h:405-455 barycentric_backward (vertex part)
    const real ax = r.xy[0], ay = r.xy[1], bx = r.xy[2], by = r.xy[3], cx = r.xy[4], cy = r.xy[5];
    real dxy[3][2];
    {
        // The reference divides each of the 21 numerators below by T or d (util.h:405-455).  Here the two
        // reciprocals are formed once and multiplied in: every quotient is within two units in the last
        // place of the reference's, and 19 of the fragment's 50 divisions go away.  The numerators keep the
        // reference's form: its differences of screen coordinates cancel, and for a sliver that rounding
        // is larger than the tolerance of the comparison, so the shorter closed form
        // (-l_v * row k of the matrix) does not reproduce the reference's numbers.
        // Nor are they fused: a fused multiply-add moves l0..l2 by as much as the reference's own rounding
        // does, which the numerators amplify for a sliver (measured: 11 rounding steps of the terms' magnitudes
        // where 2 are allowed), and the same holds for v * denom - nom in interp_backward_scalar (2.6 steps).
        const real T = (bx - ax) * (cy - ay) - (by - ay) * (cx - ax);
        const real inv_T = reciprocal(T);
        const real l0 = ((bx - px) * (cy - py) - (by - py) * (cx - px)) * inv_T;
        const real l1 = ((cx - px) * (ay - py) - (cy - py) * (ax - px)) * inv_T;
        const real l2 = ((ax - px) * (by - py) - (ay - py) * (bx - px)) * inv_T;
        const real d = ax * (by - cy) + bx * (-ay + cy) + cx * (ay - by);
        const bool flat = abs_real(d) < kEffZero;  // util.h:421: zero (selection, not a branch: see above)
        {
            const real inv_d = reciprocal(d);
            real J[3][2][3];
            J[0][0][0] = l0 * (-by + cy) * inv_d;
            J[0][0][1] = (-cy - l1 * (by - cy) + py) * inv_d;
            J[0][0][2] = (by - l2 * (by - cy) - py) * inv_d;
            J[0][1][0] = l0 * (bx - cx) * inv_d;
            J[0][1][1] = (cx + l1 * (bx - cx) - px) * inv_d;
            J[0][1][2] = (-bx + l2 * (bx - cx) + px) * inv_d;
            J[1][0][0] = (cy + l0 * (ay - cy) - py) * inv_d;
            J[1][0][1] = l1 * (ay - cy) * inv_d;
            J[1][0][2] = (-ay + l2 * (ay - cy) + py) * inv_d;
            J[1][1][0] = (-cx - l0 * (ax - cx) + px) * inv_d;
            J[1][1][1] = l1 * (-ax + cx) * inv_d;
            J[1][1][2] = (ax - l2 * (ax - cx) - px) * inv_d;
            J[2][0][0] = (-by - l0 * (ay - by) + py) * inv_d;
            J[2][0][1] = (ay - l1 * (ay - by) - py) * inv_d;
            J[2][0][2] = l2 * (-ay + by) * inv_d;
            J[2][1][0] = (bx + l0 * (ax - bx) - px) * inv_d;
            J[2][1][1] = (-ax + l1 * (ax - bx) + px) * inv_d;
            J[2][1][2] = l2 * (ax - bx) * inv_d;
#pragma unroll
            for (int v = 0; v < 3; v++)
#pragma unroll
                for (int c = 0; c < 2; c++) dxy[v][c] = flat ? 0.0f : gbary[0] * J[v][c][0] + gbary[1] * J[v][c][1] + gbary[2] * J[v][c][2];
        }
    }
#pragma unroll
    for (int v = 0; v < 3; v++) {
        const real dd_dw = -gv_z[v] * r.iw2[v];        // :523-525
        const real dw = gw_o[v] + gw_c[v] + gw_z[v];   // :530
        out[7 * v + 0] = dxy[v][0];
        out[7 * v + 1] = dxy[v][1];
        out[7 * v + 2] = dw + dd_dw;
        out[7 * v + 3] = gc[0] * scale[v];
        out[7 * v + 4] = gc[1] * scale[v];
        out[7 * v + 5] = gc[2] * scale[v];
        out[7 * v + 6] = gv_o[v];
    }
}

// One fragment start to finish (used where every pixel has its own order).
__device__ __forceinline__ void fragment_backward(BackState &st, const BackRecord &r, real b0, real b1, real b2, real px,
                                                  real py, real out[kTerms]) {
    const FragSeed f = fragment_state_step(st, r, b0, b1, b2);
    fragment_terms(f, r, b0, b1, b2, px, py, out);
}

// Layout of the three gradient arrays, a template parameter of the kernels so that the two layouts
// in use address with constants: dense (4, 3, 1 scalars per vertex), one (V,8) block (8, 8, 8), or
// the strides given at run time.
enum GradLayout { kGradDense = 0, kGradBlock8 = 1, kGradStrided = 2 };

template <int kLayout>
__device__ __forceinline__ int term_stride(const BackwardArgs &g, int c) {
    if (c < 3) return kLayout == kGradDense ? 4 : kLayout == kGradBlock8 ? 8 : g.vertex_stride;
    if (c < 6) return kLayout == kGradDense ? 3 : kLayout == kGradBlock8 ? 8 : g.color_stride;
    return kLayout == kGradDense ? 1 : kLayout == kGradBlock8 ? 8 : g.opacity_stride;
}

template <int kLayout>
__device__ __forceinline__ real *term_address(const BackwardArgs &g, int vertex_id, int c) {
    const int64_t at = term_stride<kLayout>(g, c) * (int64_t)vertex_id;
    if (c < 2) return g.grad_vertices + at + c;
    if (c == 2) return g.grad_vertices + at + 3;
    if (c < 6) return g.grad_colors + at + (c - 3);
    return g.grad_opacities + at;
}

__device__ __forceinline__ BackState load_back_state(const BackwardArgs &g, const PixelCoord &p) {
    BackState st;
    const real4 gi = g.grad_image[p.index];
    st.g0 = gi.x; st.g1 = gi.y; st.g2 = gi.z; st.g3 = gi.w;
    st.gd = g.grad_depthmap ? g.grad_depthmap[p.index] : 0.0f;  // null: the depth map took no part in the loss
    st.final_alpha = g.image[p.index].w;
    st.alpha = st.final_alpha;
    st.s0 = st.s1 = st.s2 = 0.0f;
    st.oa = st.zoa = 0.0f;
    st.final_weight = g.weights[p.index];
    st.inv_final_weight = 1.0f / st.final_weight;
    st.final_depth = g.depthmap[p.index];
    return st;
}


constexpr int kBackBatch = 64;    // list entries staged per batch
constexpr int kBackWords = kBackBatch / kWave;  // words of a lane's hit mask per batch
constexpr int kWaveSlots = 64;    // hit slots per wave and round: one per lane of the order-free part
constexpr int kTermStride = 65;   // row stride of the per-wave term matrix (odd: conflict-free columns)
constexpr int kMaxWaves = kTileThreads / kWave;

// The run sums' view of a lane: lane = 21 * group + q adds up gradient term q over the group's third
// of the slots.  What depends on q only is worked out once per kernel.
struct TermLane {
    int group;   // 0..2; 3 for the one lane left over
    int q;
    int vertex;  // q / 7: which of the entry's three vertices the term belongs to
    int stride;  // scalars per vertex in the term's array
    real *base;  // the term's element of vertex 0
};

template <int kLayout>
__device__ __forceinline__ TermLane term_lane(const BackwardArgs &g, int lane) {
    TermLane t;
    t.group = lane / kTerms;
    t.q = lane - t.group * kTerms;
    t.vertex = t.q / 7;
    const int c = t.q - 7 * t.vertex;
    t.stride = term_stride<kLayout>(g, c);
    t.base = term_address<kLayout>(g, 0, c);
    return t;
}

// Orders the LDS traffic of one wave: what lanes wrote before is visible to the
// lanes that read after (LDS serves a wave's instructions in order; this keeps
// the compiler from moving accesses across the point).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Adds up the runs of equal list entry among the first n slots of a wave's term matrix (row q = term
// q, rows kTermStride apart; slots of one entry are neighbours) and adds every non-zero run sum to the
// gradient arrays.  Bit c of `heads` is set where slot c starts a run.  Lane (group, q) owns a fixed third of
// row q -- slots [0, 22), [22, 44) or [44, 64) -- and turns it into running sums that start over at each head:
// straight-line code, no branch, no look at the entries; slots from n on hold what an earlier round left, which
// a running sum carries to later slots only, never into a slot below n.  The last slot of a run, and of a third,
// then holds a sum to deliver, and every lane walks the ones of its own third.  vertex_at(c, v): vertex id v of
// the entry in slot c.
constexpr int kRunSpan = 22;  // slots of a third (the last one has kWave - 2 * kRunSpan = 20)
template <typename VertexAt>
__device__ __forceinline__ void add_run_sums(real *terms, int n, uint64_t heads, const TermLane &t, VertexAt vertex_at) {
    if (t.group >= 3) return;  // the one lane left over; nothing below synchronises the wave
    const int c0 = t.group * kRunSpan;
    real *row = terms + t.q * kTermStride + c0;
    const bool full = t.group < 2;  // a third of kRunSpan slots
    {
        const uint32_t mine = (uint32_t)(heads >> c0);
        real v[kRunSpan];
#pragma unroll
        for (int k = 0; k < kRunSpan; k++) v[k] = (k < kWave - 2 * kRunSpan || full) ? row[k] : 0.0f;
        real sum = 0.0f;
#pragma unroll
        for (int k = 0; k < kRunSpan; k++) {
            sum = ((mine >> k) & 1) ? v[k] : sum + v[k];
            if (k < kWave - 2 * kRunSpan || full) row[k] = sum;
        }
    }
    // what a lane reads below it wrote itself above: LDS serves a wave's instructions in order
    uint64_t tails = (heads >> 1) | (1ull << (n - 1)) | (1ull << (kRunSpan - 1)) | (1ull << (2 * kRunSpan - 1));
    if (n < kWave) tails &= (1ull << n) - 1;
    uint32_t mine = (uint32_t)(tails >> c0) & ((1u << (full ? kRunSpan : kWave - 2 * kRunSpan)) - 1);
    while (mine) {
        // two slots per turn, so that two chains of LDS reads are in flight
        const int k0 = __builtin_ctz(mine);
        mine &= mine - 1;
        const int k1 = mine ? __builtin_ctz(mine) : k0;
        const bool two = mine != 0;
        mine &= mine - 1;  // 0 & anything = 0
        const real sum0 = row[k0], sum1 = two ? row[k1] : 0.0f;
        const int vertex0 = vertex_at(c0 + k0, t.vertex), vertex1 = vertex_at(c0 + k1, t.vertex);
        if (sum0 != 0.0f) unsafeAtomicAdd(t.base + (int64_t)t.stride * vertex0, sum0);
        if (sum1 != 0.0f) unsafeAtomicAdd(t.base + (int64_t)t.stride * vertex1, sum1);
    }
}

__device__ __forceinline__ int top_bit(uint64_t m) { return 63 - __builtin_clzll(m); }

// Transposes the 64 x 64 bit matrix whose row i is the word x of lane i: afterwards bit i of
// lane b's word is what bit b of lane i's word was.  Six exchange steps between lanes 32, 16, ... 1
// apart, each swapping the off-diagonal blocks of that size.
__device__ __forceinline__ uint64_t transpose_bits(uint64_t x, int lane) {
    constexpr uint64_t kHigh[6] = {0xFFFFFFFF00000000ull, 0xFFFF0000FFFF0000ull, 0xFF00FF00FF00FF00ull,
                                   0xF0F0F0F0F0F0F0F0ull, 0xCCCCCCCCCCCCCCCCull, 0xAAAAAAAAAAAAAAAAull};
#pragma unroll
    for (int s = 0; s < 6; s++) {
        const int j = 32 >> s;
        const uint32_t lo = __shfl_xor((uint32_t)x, j, kWave), hi = __shfl_xor((uint32_t)(x >> 32), j, kWave);
        const uint64_t y = ((uint64_t)hi << 32) | lo;
        x = (lane & j) ? (x & kHigh[s]) | ((y >> j) & ~kHigh[s]) : (x & ~kHigh[s]) | ((y << j) & kHigh[s]);
    }
    return x;
}

__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ uint32_t lanes_below_mask(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Tile-order backward.  LDS floating-point atomics cost about three cycles per lane on
// gfx950 and direct global atomics collide on the shared vertices, so the
// per-entry sums are formed with plain LDS stores and loads.  The kernel is bound by
// latency (LDS round trips, dependent loads), so its LDS and register budgets are set
// for four workgroups per CU: the records of 64 list entries are staged per batch by
// the whole workgroup; after that every wave works on its own 64 pixels without
// workgroup barriers:
//   1. which entries cover which pixel: the lane's 64-bit mask the forward pass saved
//      (or the inside tests again, same record for all lanes: LDS broadcast); the
//      wave's ballot per entry is the transpose of the lanes' masks;
//   2. the ballots become slot numbers: entries from the far end, lanes in
//      order inside an entry, so every (pixel, entry) hit of the wave owns one
//      slot, slots are grouped by entry, and a lane's own hits have increasing
//      numbers in the order it must visit them (reverse blend order);
//   3. ordered part, in rounds of 64 slots: every lane walks its own hits and
//      advances the pixel's transmittance and running sums; each hit leaves
//      five numbers in its slot;
//   4. order-free part with every lane busy: lane = slot evaluates the 21 gradient
//      terms of its hit and writes them to a term matrix; three groups of 21 lanes
//      add up the runs of equal entry and issue one global floating-point atomic
//      per run and term.
template <int kLayout>
__global__ __launch_bounds__(kTileThreads) void backward_tile_order_kernel(RasterArgs a, BackwardArgs g) {
    __shared__ BackRecord s_rec[kBackBatch];
    __shared__ uint64_t s_ballot[kMaxWaves][kBackBatch];
    __shared__ uint32_t s_base[kMaxWaves][kBackBatch];
    __shared__ int s_tag[kMaxWaves][kWaveSlots];  // (entry | source lane << 8) of a slot
    __shared__ real s_term[kMaxWaves][kTerms * kTermStride];
    __shared__ uint8_t s_touch[kBackBatch];
    __shared__ WaveRect s_rects[kMaxTileWaves];
    __shared__ int s_last;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int n_waves = blockDim.x / kWave;
    const TileId tile_id = tile_of_workgroup<kTileBandBackward>();
    const int tile = tile_id.index;
    const int start = a.offsets[tile];
    const PixelCoord p = pixel_of_thread(a, tile_id);
    const TermLane tl = term_lane<kLayout>(g, lane);
    uint64_t *ballots = s_ballot[wave];
    uint32_t *bases = s_base[wave];
    int *tags = s_tag[wave];
    real *terms = s_term[wave];

    // With the forward pass's masks comes the number of list entries this workgroup has to walk; else
    // it is the largest `last` of its pixels.  The pixel's own loads are issued first either way: the
    // barriers and the staging of the first batch cover their latency.
    const bool saved_masks = g.hit_masks != nullptr;
    const uint64_t *const masks = saved_masks ? g.hit_masks + hit_mask_head_words() : nullptr;
    const int my_last = p.valid ? g.last[p.index] : 0;  // entries [0, my_last) of the list may hold my fragments
    BackState st;
    if (p.valid) st = load_back_state(g, p);
    int tile_last;
    if (saved_masks) {
        tile_last = (int)g.hit_masks[hit_mask_head_index(tile)];
    } else {
        if (tid == 0) s_last = 0;
        publish_wave_rect(p, s_rects);  // only the repeated inside tests cull by wave rectangle
        __syncthreads();
        if (my_last > 0) atomicMax(&s_last, my_last);
        __syncthreads();
        tile_last = s_last;
    }

    // Batches are aligned to multiples of kBackBatch from the start of the list (the last one may be
    // short), so that a batch is whole words of the saved hit masks.
    const int64_t mask_slots = (int64_t)gridDim.z * blockDim.x, mask_slot = (int64_t)blockIdx.z * blockDim.x + tid;
    const int hi0 = (tile_last + kBackBatch - 1) / kBackBatch * kBackBatch;
    for (int hi = hi0; hi > 0; hi -= kBackBatch) {
        const int lo = hi - kBackBatch;
        const int nb = min(hi, tile_last) - lo;
        const int mine = my_last - lo;  // records [0, mine) of this batch are within my range
        // my saved masks of the batch: asked for here, used after the staging
        uint64_t m[kBackWords] = {};
        if (saved_masks) {
            const int64_t chunk = hit_mask_chunk(start, tile, lo);
#pragma unroll
            for (int wd = 0; wd < kBackWords; wd++)
                if (64 * wd < mine) {
                    m[wd] = masks[(chunk + wd) * mask_slots + mask_slot];
                    if (mine < 64 * wd + 64) m[wd] &= (1ull << (mine - 64 * wd)) - 1;  // entries past my last one
                }
        }
        __syncthreads();  // every wave is done with the previous batch
        for (int e = tid; e < nb; e += blockDim.x) {
            gather_back(a, start + lo + e, s_rec[e]);
            if (!saved_masks) s_touch[e] = (uint8_t)waves_touched(s_rec[e].m, s_rects, n_waves);
        }
        __syncthreads();

        // 1. which entries cover which pixel: read back what the forward pass saved, or test again
        //    (then only the entries that can touch this wave's pixels)
        if (__builtin_amdgcn_ballot_w64(mine > 0) == 0) continue;  // nothing for this wave in the batch
        if (saved_masks) {
            // per-entry ballots = the transpose of the lanes' masks
#pragma unroll
            for (int wd = 0; wd < kBackWords; wd++) ballots[wd * kWave + lane] = transpose_bits(m[wd], lane);
        } else {
#pragma unroll
            for (int wd = 0; wd < kBackWords; wd++) ballots[wd * kWave + lane] = 0;
            wave_lds_sync();
#pragma unroll
            for (int wd = 0; wd < kBackWords; wd++) {
                uint64_t bits = 0;
                uint64_t todo = wave_candidates(s_touch, 64 * wd, nb, wave);
                while (todo) {
                    const int bit = __builtin_ctzll(todo);
                    todo &= todo - 1;
                    const BackRecord &r = s_rec[64 * wd + bit];
                    real b0, b1, b2;
                    bary_apply(r.m, p.px, p.py, b0, b1, b2);
                    const bool hit = bary_inside(b0, b1, b2) && 64 * wd + bit < mine;
                    const uint64_t vote = __builtin_amdgcn_ballot_w64(hit);
                    if (hit) bits |= 1ull << bit;
                    if (lane == 0) ballots[64 * wd + bit] = vote;
                }
                m[wd] = bits;
            }
        }
        wave_lds_sync();

        // 2. slot numbers of this wave
        uint32_t n_hits;
        {
            // lane l takes entries nb - 1 - kBackWords * l and the kBackWords - 1 before it
            uint32_t cnt[kBackWords], mine_total = 0;
#pragma unroll
            for (int k = 0; k < kBackWords; k++) {
                const int e = nb - 1 - kBackWords * lane - k;
                cnt[k] = e >= 0 ? (uint32_t)__builtin_popcountll(ballots[e]) : 0u;
                mine_total += cnt[k];
            }
            const uint32_t incl = wave_inclusive_scan_u32(mine_total);
            uint32_t base = incl - mine_total;
#pragma unroll
            for (int k = 0; k < kBackWords; k++) {
                const int e = nb - 1 - kBackWords * lane - k;
                if (e >= 0) bases[e] = base;
                base += cnt[k];
            }
            n_hits = (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        }
        wave_lds_sync();

        for (uint32_t round0 = 0; round0 < n_hits; round0 += kWaveSlots) {
            const int n_slots = (int)min((uint32_t)kWaveSlots, n_hits - round0);
            // 3. ordered part, lane by lane over its own hits
            while (true) {
                int e = -1;
                uint32_t slot = 0;
#pragma unroll
                for (int wd = kBackWords - 1; wd >= 0; wd--)
                    if (e < 0 && m[wd]) e = 64 * wd + top_bit(m[wd]);
                if (e >= 0) {
                    slot = bases[e] + lanes_below_mask(ballots[e]) - round0;
                    if (slot >= (uint32_t)kWaveSlots) e = -1;
                }
                const bool active = e >= 0;
                if (__builtin_amdgcn_ballot_w64(active) == 0) break;
                if (active) {
#pragma unroll
                    for (int wd = 0; wd < kBackWords; wd++)
                        if ((e >> 6) == wd) m[wd] &= ~(1ull << (e & 63));
                    const BackRecord &r = s_rec[e];
                    real b0, b1, b2;
                    bary_apply(r.m, p.px, p.py, b0, b1, b2);
                    const FragSeed f = fragment_state_step(st, r, b0, b1, b2);
                    // the five numbers wait in the slot's column of the term matrix, which is free until
                    // the slot's own lane replaces them by the terms
                    terms[0 * kTermStride + slot] = f.d_do;
                    terms[1 * kTermStride + slot] = f.gc[0];
                    terms[2 * kTermStride + slot] = f.gc[1];
                    terms[3 * kTermStride + slot] = f.gc[2];
                    terms[4 * kTermStride + slot] = f.dd_dz;
                    tags[slot] = e | (lane << 8);
                }
            }
            wave_lds_sync();

            // 4. order-free part: lane = slot
            int tag = -1;
            if (lane < n_slots) tag = tags[lane] & 0xff;
            // the pixel of the slot, from the lane that owns it
            const int src = (lane < n_slots) ? tags[lane] >> 8 : lane;
            const real px = __shfl(p.px, src, kWave), py = __shfl(p.py, src, kWave);
            if (lane < n_slots) {
                FragSeed f;
                f.d_do = terms[0 * kTermStride + lane];
                f.gc[0] = terms[1 * kTermStride + lane];
                f.gc[1] = terms[2 * kTermStride + lane];
                f.gc[2] = terms[3 * kTermStride + lane];
                f.dd_dz = terms[4 * kTermStride + lane];
                const BackRecord &r = s_rec[tag];
                real b0, b1, b2;
                bary_apply(r.m, px, py, b0, b1, b2);
                real term[kTerms];
                fragment_terms(f, r, b0, b1, b2, px, py, term);
#pragma unroll
                for (int q = 0; q < kTerms; q++) terms[q * kTermStride + lane] = term[q];
            }
            const int tag_before = __shfl_up(tag, 1, kWave);
            const uint64_t heads = __builtin_amdgcn_ballot_w64(lane < n_slots && (lane == 0 || tag != tag_before));
            wave_lds_sync();
            add_run_sums(terms, n_slots, heads, tl, [&](int c, int v) { return s_rec[tags[c] & 0xff].id[v]; });
            wave_lds_sync();
        }
    }
}

// list positions whose gradient sums are kept in LDS by the per-pixel-order kernel (the double build has
// half the room per scalar and twice the candidate lists)
constexpr int kAccWindow = sizeof(real) == 4 ? 512 : 128;

// The order the reverse selection walks: by pixel depth, a NaN depth behind every number (that is where the
// forward selection leaves such a fragment, render.cu:338-373: every comparison with it is false), equal
// depths (two NaNs count as equal) by list position.
__device__ __forceinline__ bool depth_before(real a, real b) { return a < b || (b != b && a == a); }
__device__ __forceinline__ bool depth_same(real a, real b) { return a == b || (a != a && b != b); }

// Candidate insertion for the reverse selection: keeps the `cap` LARGEST
// (depth, position) pairs in descending order.  Positions arrive in ascending
// order, so a candidate whose depth equals a stored one has the larger position
// and goes in front of it.
__device__ __forceinline__ void topk_insert_desc(const TopK &tk, int cap, int &n, real d, int j) {
    if (n == cap && depth_before(d, tk.d(cap - 1))) return;
    int i = (n < cap) ? n : cap - 1;
    while (i > 0 && !depth_before(d, tk.d(i - 1))) {
        tk.d(i) = tk.d(i - 1);
        tk.j(i) = tk.j(i - 1);
        i--;
    }
    tk.d(i) = d;
    tk.j(i) = j;
    if (n < cap) n++;
}

template <int kLayout>
__global__ __launch_bounds__(kTileThreads) void backward_pixel_order_kernel(RasterArgs a, BackwardArgs g) {
    extern __shared__ __align__(16) unsigned char s_dyn[];
    const int n_threads = blockDim.x;
    DepthRecord *s_rec = reinterpret_cast<DepthRecord *>(s_dyn);
    TopK tk;
    tk.depth = reinterpret_cast<real *>(s_dyn + sizeof(DepthRecord) * kBatch);
    tk.pos = reinterpret_cast<int *>(tk.depth + kLayers * n_threads);
    tk.n_threads = n_threads;
    // Per-entry sums of the first kAccWindow list positions live in LDS and are
    // flushed once per tile; positions beyond the window go straight to memory.
    real *s_acc = reinterpret_cast<real *>(tk.pos + kLayers * n_threads);

    __shared__ uint8_t s_touch[kBatch];
    __shared__ WaveRect s_rects[kMaxTileWaves];
    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int n_waves = blockDim.x / kWave;
    const TileId tile_id = tile_of_workgroup<kTileBandBackward>();
    const int tile = tile_id.index;
    const int start = a.offsets[tile], end = a.offsets[tile + 1];
    const PixelCoord p = pixel_of_thread(a, tile_id);
    publish_wave_rect(p, s_rects);
    const int n_acc = min(end - start, kAccWindow);
    for (int i = tid; i < n_acc * kTerms; i += blockDim.x) s_acc[i] = 0.0f;

    BackState st;
    int remaining = 0;
    // exclusive upper bound of the fragments still to visit, in (depth, position) order
    real bound_depth = 0.0f;
    int bound_j = 0;
    if (p.valid) {
        st = load_back_state(g, p);
        remaining = min(g.ends[p.index], a.max_layers);  // render.cu:642
        bound_depth = g.last_depth[p.index];
        bound_j = start + g.last[p.index];  // one past the last blended entry
    }
    while (true) {
        const bool want = remaining > 0;
        if (!__syncthreads_or(want)) break;
        const int cap = min(kLayers, remaining);
        int found = 0;
        for (int batch = start; batch < end; batch += kBatch) {
            const int nb = min(kBatch, end - batch);
            __syncthreads();
            for (int e = tid; e < nb; e += blockDim.x) {
                gather_depth(a, batch + e, s_rec[e]);
                s_touch[e] = (uint8_t)waves_touched(s_rec[e].m, s_rects, n_waves);
            }
            __syncthreads();
            uint64_t m[kBatch / kWave];
            batch_hit_mask<kBatch / kWave>(s_rec, s_touch, nb, wave, p.px, p.py, m);
            if (!want) {
#pragma unroll
                for (int wd = 0; wd < kBatch / kWave; wd++) m[wd] = 0;
            }
            while (true) {
                const int e = pop_lowest<kBatch / kWave>(m);
                if (__builtin_amdgcn_ballot_w64(e >= 0) == 0) break;  // wave-uniform
                if (e < 0) continue;
                const DepthRecord &r = s_rec[e];
                real b0, b1, b2;
                bary_apply(r.m, p.px, p.py, b0, b1, b2);
                const real pd = interp_w(b0, b1, b2, r.z[0], r.z[1], r.z[2], r.w[0], r.w[1], r.w[2]);
                const int j = batch + e;
                if (depth_before(pd, bound_depth) || (depth_same(pd, bound_depth) && j < bound_j)) topk_insert_desc(tk, cap, found, pd, j);
            }
        }
        if (want) {
            for (int i = 0; i < found; i++) {
                BackRecord r;
                gather_back(a, tk.j(i), r);
                real b0, b1, b2;
                bary_apply(r.m, p.px, p.py, b0, b1, b2);
                if (!bary_inside(b0, b1, b2)) continue;  // cannot happen: the selection tested it
                real term[kTerms];
                fragment_backward(st, r, b0, b1, b2, p.px, p.py, term);
                const int rel = tk.j(i) - start;
                if (rel < kAccWindow) {
#pragma unroll
                    for (int q = 0; q < kTerms; q++) atomicAdd(s_acc + rel * kTerms + q, term[q]);
                } else {
#pragma unroll
                    for (int q = 0; q < kTerms; q++)
                        if (term[q] != 0.0f) unsafeAtomicAdd(term_address<kLayout>(g, r.id[q / 7], q % 7), term[q]);
                }
            }
            if (found < cap) {
                remaining = 0;  // list exhausted
            } else {
                remaining -= found;
                bound_depth = tk.d(found - 1);
                bound_j = tk.j(found - 1);
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < n_acc; e += blockDim.x) {
        const TriIds t = load_ids(a, start + e);
        const int id[3] = {t.ia, t.ib, t.ic};
#pragma unroll
        for (int q = 0; q < kTerms; q++) {
            const real v = s_acc[e * kTerms + q];
            if (v != 0.0f) unsafeAtomicAdd(term_address<kLayout>(g, id[q / 7], q % 7), v);
        }
    }
}

// Per-pixel order with the blend order saved by the forward pass
// (max_layers <= TG_MAX_SAVED_LAYERS): no re-selection.  Step s of a pixel is its
// fragment n - 1 - s, so every pixel starts at its own far end.  The pixels of a wave
// hold different numbers of fragments, so the wave takes its (pixel, step) pairs 64 at a
// time: a round's 64 slots keep every lane busy whatever the pixels' counts are.  A round
// takes the pending pairs nearest the far end of the tile's list (every pixel a prefix of
// its next steps, so its own slots come in the order it must visit them): the slots of a
// round then hold few different entries.  Per round:
//   1. lane = pixel: which of my next steps (their list positions are fetched from the
//      saved order four steps ahead) lie at or above the round's threshold; they get
//      consecutive slots;
//   2. lane = slot: gathers the record of its fragment from memory (neighbouring
//      pixels hold the same few entries, so the loads hit in cache; staging the tile's
//      records in LDS first was measured slower, for the workgroups per CU it costs)
//      and leaves the fragment's own opacity, colour and view depth in the slot;
//   3. lane = pixel: the ordered part over my slots of the round, which replaces the
//      five values by the five numbers the gradient terms are linear in;
//   4. lane = slot: the 21 gradient terms.  LDS floating-point atomics cost about three
//      cycles per lane on gfx950 and many slots of a round hold the same entry, so the
//      terms are grouped by entry first: slots with equal entries get consecutive
//      columns (ballot matching, groups in order of their lowest slot) of a term
//      matrix in LDS, three groups of 21 lanes add up the runs of equal entry and issue
//      one global floating-point atomic per run and term.
template <int kLayout>
__global__ __launch_bounds__(kTileThreads) void backward_saved_order_kernel(RasterArgs a, BackwardArgs g) {
    __shared__ real s_term[kMaxWaves][kTerms * kTermStride];
    __shared__ int s_rel[kMaxWaves][kWave];         // list position of a slot's fragment, from the tile's start
    __shared__ int s_tag[kMaxWaves][kWave];         // the same by column of the term matrix
    __shared__ int s_vertex[kMaxWaves][3 * kWave];  // the three vertex ids of a column's entry
    __shared__ uint8_t s_src[kMaxWaves][kWave];     // the pixel (lane) of a slot
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const TileId tile_id = tile_of_workgroup<kTileBandBackward>();
    const int tile = tile_id.index;
    const int start = a.offsets[tile], end = a.offsets[tile + 1];
    const PixelCoord p = pixel_of_thread(a, tile_id);
    const int rel_bits = 32 - __builtin_clz(max(end - start - 1, 1));  // bits that tell two list positions apart
    real *terms = s_term[wave];
    int *tags = s_tag[wave];
    int *vertices = s_vertex[wave];
    const TermLane tl = term_lane<kLayout>(g, lane);

    BackState st;
    int n = 0;
    if (p.valid) {
        st = load_back_state(g, p);
        n = min(g.ends[p.index], a.max_layers);  // render.cu:642
    }
    const int64_t plane = (int64_t)a.W * a.H;
    const bool long_list = end - start > 0xffff;  // then the positions' high halves were saved as well
    // The list positions of my steps, one after the other: step s is layer n - 1 - s, a plane further down each time.
    const uint16_t *next_layer = g.fragments + ((int64_t)(n - 1) * plane + (p.valid ? p.index : 0));
    const int64_t high_halves = (int64_t)a.max_layers * plane;
    int steps_read = 0;
    auto next_position = [&]() {
        int position = -1;  // no such step: below every threshold
        if (steps_read < n) {
            position = *next_layer;
            if (long_list) position |= (int)next_layer[high_halves] << 16;
        }
        next_layer -= plane;
        steps_read++;
        return position;
    };
    // the list positions of my next four steps
    int ahead0 = next_position(), ahead1 = next_position(), ahead2 = next_position(), ahead3 = next_position();
    int remaining = __builtin_amdgcn_readlane((int)wave_inclusive_scan_u32((uint32_t)n), kWave - 1);  // the wave's fragments not handed out yet

    // How many of my next steps lie at or above list position `threshold`: a prefix of them, so that I visit them in order.
    // -> the four masks of the lanes whose first, second, ... next step qualifies, and the slots that makes.
    auto slots_at = [&](int threshold) {
        const uint64_t first = __builtin_amdgcn_ballot_w64(ahead0 >= threshold);
        const uint64_t second = first & __builtin_amdgcn_ballot_w64(ahead1 >= threshold);
        const uint64_t third = second & __builtin_amdgcn_ballot_w64(ahead2 >= threshold);
        const uint64_t fourth = third & __builtin_amdgcn_ballot_w64(ahead3 >= threshold);
        return __builtin_popcountll(first) + __builtin_popcountll(second) + __builtin_popcountll(third) + __builtin_popcountll(fourth);
    };

    for (int round = 0; remaining > 0; round++) {
        // 1. the round's slots.  A round takes the wave's pending fragments from the far end of the tile's LIST, not step s
        //    of every pixel: a triangle is at another step in each pixel it covers, but at one list position, so the
        //    slots of a round then hold few different entries -- long runs, few atomics, and gathers whose lanes share
        //    their cache lines.  Every pixel gives a prefix of its next (at most four) steps, those at or above a
        //    threshold: the largest threshold that fills the 64 slots.  What overflows is cut off in lane order from a
        //    start lane that moves from round to round, and waits for the next round.
        int threshold = 0, offered = slots_at(0);
        if (offered > kWave) {
            int high = __builtin_amdgcn_readfirstlane(wave_max_i32(ahead0)) + 1;  // slots_at(threshold) >= 64 > slots_at(high) = 0
            while (high - threshold > 1) {
                const int middle = threshold + (high - threshold) / 2;
                const int slots = slots_at(middle);
                if (slots >= kWave) { threshold = middle; offered = slots; } else { high = middle; }
            }
        }
        const bool first = ahead0 >= threshold, second = first && ahead1 >= threshold, third = second && ahead2 >= threshold,
                   fourth = third && ahead3 >= threshold;
        const int mine_count = (int)first + (int)second + (int)third + (int)fourth;
        const int taken_incl = (int)wave_inclusive_scan_u32((uint32_t)mine_count);
        const int first_lane = (round * 23) & (kWave - 1);
        const int before_first = __builtin_amdgcn_readlane(taken_incl - mine_count, first_lane);
        int base = taken_incl - mine_count - before_first;
        if (lane < first_lane) base += offered;
        const int granted = max(0, min(mine_count, kWave - base));
        const int n_slots = min(kWave, offered);
        int *rels = s_rel[wave];
        uint8_t *srcs = s_src[wave];
        if (granted > 0) { rels[base] = ahead0; srcs[base] = (uint8_t)lane; }
        if (granted > 1) { rels[base + 1] = ahead1; srcs[base + 1] = (uint8_t)lane; }
        if (granted > 2) { rels[base + 2] = ahead2; srcs[base + 2] = (uint8_t)lane; }
        if (granted > 3) { rels[base + 3] = ahead3; srcs[base + 3] = (uint8_t)lane; }
        uint64_t mine = granted > 0 ? ((1ull << granted) - 1) << base : 0ull;  // my slots of the round: increasing slot = increasing step
#pragma unroll
        for (int k = 0; k < 4; k++)
            if (granted > k) {
                ahead0 = ahead1; ahead1 = ahead2; ahead2 = ahead3;
                ahead3 = next_position();
            }
        remaining -= n_slots;
        wave_lds_sync();

        // 2. lane = slot: the record, and the fragment's own values
        const int src = (lane < n_slots) ? srcs[lane] : lane;
        const real px = __shfl(p.px, src, kWave), py = __shfl(p.py, src, kWave);
        BackRecord r;
        real b0 = 0.0f, b1 = 0.0f, b2 = 0.0f;
        int rel = 0;
        if (lane < n_slots) {
            rel = rels[lane];
            gather_back(a, start + rel, r);
            bary_apply(r.m, px, py, b0, b1, b2);
            const FragValue v = fragment_value(r, b0, b1, b2);
            terms[0 * kTermStride + lane] = v.o;
            terms[1 * kTermStride + lane] = v.color[0];
            terms[2 * kTermStride + lane] = v.color[1];
            terms[3 * kTermStride + lane] = v.color[2];
            terms[4 * kTermStride + lane] = v.z;
        }
        wave_lds_sync();

        // 3. lane = pixel: the ordered part
        while (true) {
            const bool active = mine != 0;
            if (__builtin_amdgcn_ballot_w64(active) == 0) break;
            if (active) {
                const int c = __builtin_ctzll(mine);
                mine &= mine - 1;
                FragValue v;
                v.o = terms[0 * kTermStride + c];
                v.color[0] = terms[1 * kTermStride + c];
                v.color[1] = terms[2 * kTermStride + c];
                v.color[2] = terms[3 * kTermStride + c];
                v.z = terms[4 * kTermStride + c];
                const FragSeed f = fragment_chain_step(st, v);
                terms[0 * kTermStride + c] = f.d_do;
                terms[1 * kTermStride + c] = f.gc[0];
                terms[2 * kTermStride + c] = f.gc[1];
                terms[3 * kTermStride + c] = f.gc[2];
                terms[4 * kTermStride + c] = f.dd_dz;
            }
        }
        wave_lds_sync();

        // 4. lane = slot: the terms, in the column the matching gives the slot
        const bool active = lane < n_slots;
        FragSeed f;
        f.d_do = f.gc[0] = f.gc[1] = f.gc[2] = f.dd_dz = 0.0f;
        if (active) {
            f.d_do = terms[0 * kTermStride + lane];
            f.gc[0] = terms[1 * kTermStride + lane];
            f.gc[1] = terms[2 * kTermStride + lane];
            f.gc[2] = terms[3 * kTermStride + lane];
            f.dd_dz = terms[4 * kTermStride + lane];
        }
        uint64_t peers = __builtin_amdgcn_ballot_w64(active);
        for (int b = 0; b < rel_bits; b++) {  // wave-uniform
            const bool bit = (rel >> b) & 1;
            const uint64_t vote = __builtin_amdgcn_ballot_w64(bit);
            peers &= bit ? vote : ~vote;
        }
        const uint32_t rank = lanes_below_mask(peers);
        const bool leads = active && rank == 0;
        const uint32_t size = leads ? (uint32_t)__builtin_popcountll(peers) : 0u;
        const uint32_t incl = wave_inclusive_scan_u32(size);
        const int leader = active ? __builtin_ctzll(peers) : lane;
        const int column = __shfl((int)(incl - size), leader, kWave) + (int)rank;
        wave_lds_sync();  // every slot's five numbers are in registers before terms take their place
        if (active) {
            real term[kTerms];
            fragment_terms(f, r, b0, b1, b2, px, py, term);
#pragma unroll
            for (int q = 0; q < kTerms; q++) terms[q * kTermStride + column] = term[q];
            tags[column] = rel;
#pragma unroll
            for (int k = 0; k < 3; k++) vertices[k * kWave + column] = r.id[k];
        }
        wave_lds_sync();
        // a column starts a run where its entry differs from the column before
        const uint64_t heads = __builtin_amdgcn_ballot_w64(lane < n_slots && (lane == 0 || tags[lane] != tags[max(lane - 1, 0)]));
        add_run_sums(terms, n_slots, heads, tl, [&](int c, int v) { return vertices[v * kWave + c]; });
        wave_lds_sync();
    }
}

// The three gradient arrays out of the (V,8) block the per-pixel-order kernels accumulate into:
// one read of the block instead of the three strided ones that three separate copies make.
__global__ __launch_bounds__(256) void split_gradient_block_kernel(const real4 *__restrict__ block, int64_t n_vertices,
                                                                   real4 *__restrict__ grad_vertices, real *__restrict__ grad_colors,
                                                                   real *__restrict__ grad_opacities) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vertices) return;
    const real4 position = block[2 * v], rest = block[2 * v + 1];
    grad_vertices[v] = position;
    grad_colors[3 * v] = rest.x;
    grad_colors[3 * v + 1] = rest.y;
    grad_colors[3 * v + 2] = rest.z;
    grad_opacities[v] = rest.w;
}

size_t backward_pixel_order_lds_bytes(int n_threads) { return pixel_order_lds_bytes(n_threads, kBatch) + (size_t)kAccWindow * kTerms * sizeof(real); }

}  // namespace tg

using namespace tg;

extern "C" int tg_render_backward(const real *grad_image, const real *grad_depthmap, const real *vertices,
                                  const int32_t *indices, const real *colors, const real *opacities,
                                  const int32_t *sorted_ids, const int32_t *offsets, const real *bary, const real *image,
                                  const real *depthmap, const real *final_weights, const int32_t *ends, const int32_t *last,
                                  const real *last_depth, const uint16_t *fragments, const uint64_t *hit_masks, int width,
                                  int height, int tile_w,
                                  int tile_h, real early_stopping_threshold, int per_pixel_sort, int max_layers, real *grad_vertices,
                                  real *grad_colors, real *grad_opacities, int vertex_stride, int color_stride,
                                  int opacity_stride, void *stream) {
    if (int e = check_raster_args("tg_render_backward", width, height, tile_w, tile_h, max_layers)) return e;
    if (!grad_image || !vertices || !indices || !colors || !opacities || !offsets || !bary || !image ||
        !depthmap || !final_weights || !ends || !last || !grad_vertices || !grad_colors || !grad_opacities ||
        (per_pixel_sort && !last_depth && !fragments)) {
        set_error("tg_render_backward: null pointer");
        return TG_E_ARG;
    }
    if (vertex_stride < 4 || color_stride < 3 || opacity_stride < 1) {
        set_error("tg_render_backward: gradient strides must be at least 4, 3 and 1");
        return TG_E_ARG;
    }
    if (((uintptr_t)vertices & 15) || ((uintptr_t)image & 15) || ((uintptr_t)grad_image & 15)) {
        set_error("tg_render_backward: vertices, image and grad_image must be 16-byte aligned");
        return TG_E_ARG;
    }
    RasterArgs a{(const real4 *)vertices, indices, colors, opacities, sorted_ids, offsets, bary, nullptr, nullptr,
                 width, height, tile_w, tile_h, early_stopping_threshold, max_layers};
    BackwardArgs g{(const real4 *)grad_image, grad_depthmap, (const real4 *)image, depthmap, final_weights, ends, last,
                   last_depth, fragments, per_pixel_sort ? nullptr : hit_masks, grad_vertices, grad_colors, grad_opacities,
                   vertex_stride, color_stride, opacity_stride};
    hipStream_t s = (hipStream_t)stream;
    const int layout = (vertex_stride == 4 && color_stride == 3 && opacity_stride == 1)   ? kGradDense
                       : (vertex_stride == 8 && color_stride == 8 && opacity_stride == 8) ? kGradBlock8
                                                                                          : kGradStrided;
#define TG_LAUNCH_BACKWARD(kernel, grid, block, lds_bytes)                                                  \
    do {                                                                                                    \
        if (layout == kGradDense) TG_LAUNCH_AS(#kernel, kernel<kGradDense>, grid, block, lds_bytes, s, a, g);   \
        else if (layout == kGradBlock8) TG_LAUNCH_AS(#kernel, kernel<kGradBlock8>, grid, block, lds_bytes, s, a, g); \
        else TG_LAUNCH_AS(#kernel, kernel<kGradStrided>, grid, block, lds_bytes, s, a, g);                      \
    } while (0)
    if (!per_pixel_sort) {
        const TileLaunch tl = tile_launch(width, height, tile_w, tile_h, kTileThreads);
        TG_LAUNCH_BACKWARD(backward_tile_order_kernel, tl.grid, dim3(tl.threads), 0);
        return check_launch("backward_tile_order_kernel");
    }
    if (fragments) {
        if (max_layers > TG_MAX_SAVED_LAYERS) {
            set_error("tg_render_backward: saved fragments need max_layers <= %d", TG_MAX_SAVED_LAYERS);
            return TG_E_ARG;
        }
        const TileLaunch tl = tile_launch(width, height, tile_w, tile_h, kTileThreads);
        TG_LAUNCH_BACKWARD(backward_saved_order_kernel, tl.grid, dim3(tl.threads), 0);
        return check_launch("backward_saved_order_kernel");
    }
    const TileLaunch tl = tile_launch(width, height, tile_w, tile_h, pixel_order_threads(kTileThreads));
    const size_t lds = backward_pixel_order_lds_bytes(tl.threads);
    static size_t lds_reserved[3][kMaxDevices] = {{0}};
    int which = 0;
    for (const void *kernel : {(const void *)backward_pixel_order_kernel<kGradDense>, (const void *)backward_pixel_order_kernel<kGradBlock8>,
                               (const void *)backward_pixel_order_kernel<kGradStrided>})
        if (int e = reserve_lds("tg_render_backward", kernel, lds, lds_reserved[which++])) return e;
    TG_LAUNCH_BACKWARD(backward_pixel_order_kernel, tl.grid, dim3(tl.threads), lds);
    return check_launch("backward_pixel_order_kernel");
#undef TG_LAUNCH_BACKWARD
}

extern "C" int tg_split_gradient_block(const real *block, int64_t n_vertices, real *grad_vertices, real *grad_colors,
                                       real *grad_opacities, void *stream) {
    if (n_vertices < 0 || n_vertices > (int64_t)0x7fffffff * 256) {
        set_error("tg_split_gradient_block: n_vertices out of range");
        return TG_E_ARG;
    }
    if (n_vertices == 0) return 0;
    if (!block || !grad_vertices || !grad_colors || !grad_opacities) {
        set_error("tg_split_gradient_block: null pointer");
        return TG_E_ARG;
    }
    if (((uintptr_t)block & 15) || ((uintptr_t)grad_vertices & 15)) {
        set_error("tg_split_gradient_block: block and grad_vertices must be 16-byte aligned");
        return TG_E_ARG;
    }
    TG_LAUNCH(split_gradient_block_kernel, dim3((unsigned)ceil_div64(n_vertices, 256)), dim3(256), 0, (hipStream_t)stream,
              (const real4 *)block, n_vertices, (real4 *)grad_vertices, grad_colors, grad_opacities);
    return check_launch("split_gradient_block_kernel");
}
