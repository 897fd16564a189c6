// trigrad_oracle.cpp -- CPU restatement of trigrad's tile rasterizer (TEST INFRASTRUCTURE).
//
// This file is the parity oracle and the reported CPU baseline.  It is NOT part
// of the product: nothing under trigrad_amd/ may include, link or call it.  Only
// tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it.
//
// It restates, operation by operation, the arithmetic of the reference's CUDA
// source (paths relative to the reference tree):
//   src/trigrad/render.cu   binning, clipped-min-depth key, bary matrices,
//                           forward blend, backward
//   src/trigrad/util.h      interpolate3(+backward), barycentric(+backward)
//   src/trigrad/wrapper.py  max_layers<=0 -> M+1, empty scene
// under two declared conventions the CUDA build leaves to chance:
//   * strict IEEE-754 evaluation of the source expressions: no fused
//     multiply-add (build with -ffp-contract=off), correctly rounded division;
//   * the slot order inside a tile before the depth sort (decided by atomicAdd
//     races in render.cu:239) is ascending triangle id, i.e. the outcome of a
//     serial execution; equal keys then stay in triangle-id order because the
//     sort is stable (render.cu:280).  Keys are ordered by the total order of
//     their order-preserving bit pattern (-0.0 sorts before +0.0).
//
// Every function cites the reference lines it follows.  Everything is
// templated on the scalar type: float is the shipped precision
// (util.h:14-20), double is the DOUBLE_PRECISION build (util.h:6-13) that the
// reference's own gradcheck tests presuppose.
//
// Parity status of each part (what pins it, see tests/test_oracle_*.py):
//   tile rect / counts      closed forms for in-screen AABBs, brute force
//   emission / sort / ranges numpy lexsort, searchsorted, cumsum
//   clipped-min-depth key   dense float64 sampling of the plane over
//                           triangle-intersect-tile, constant-z triangles
//   bary matrices           numpy.linalg.inv
//   forward image/depth     independent float64 per-pixel renderer, closed
//                           forms (n constant layers, early-stop layer count)
//   backward                finite differences of the float64 instantiation
//                           (the reference's own method,
//                           tests/test_render_gradients.py) and autograd
//                           through the independent renderer
//   NaN depths/keys         parity unpinned (ordering of NaN is an accident of
//                           the CUDA build; never produced by finite input)
//
// Build: g++ -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

int g_threads = 1;

template <typename S> struct P2 { S x, y; };
template <typename S> struct P3 { S x, y, z; };

template <typename S> constexpr S eff_zero() { return std::numeric_limits<S>::min(); }  // util.h:24
template <typename S> constexpr S max_opacity() { return (S)0.9999; }                   // util.h:22

// std::min/std::max over three values, first wins ties (render.cu:68-71).
template <typename S> inline S min3(S a, S b, S c) { S m = a; if (b < m) m = b; if (c < m) m = c; return m; }
template <typename S> inline S max3(S a, S b, S c) { S m = a; if (m < b) m = b; if (m < c) m = c; return m; }
// std::clamp(v, lo, hi) (render.cu:72-75, :442).
template <typename S> inline S clampS(S v, S lo, S hi) { return (v < lo) ? lo : ((hi < v) ? hi : v); }

struct TileRect { int x0, y0, x1, y1; };  // y0 == -1 marks "no tiles"

// render.cu:51-76 touched_tiles.  The tile coordinate is evaluated in double
// because of the 0.5 literal at :72-75, rounded to the scalar type, clamped in
// the scalar type and truncated toward zero by the int assignment.
template <typename S>
inline TileRect touched_tiles(P2<S> a, P2<S> b, P2<S> c, int W, int H, int tw, int th, int tiles_x, int tiles_y) {
    S ux = b.x - a.x, uy = b.y - a.y, vx = c.x - a.x, vy = c.y - a.y;
    S v = ux * vy - uy * vx;  // util.h:384-388 cross2d(b-a, c-a)
    if (std::fabs(v) < eff_zero<S>() || std::isnan(v) || std::isinf(v)) return {0, -1, 0, -1};
    S minx = min3(a.x, b.x, c.x), miny = min3(a.y, b.y, c.y);
    S maxx = max3(a.x, b.x, c.x), maxy = max3(a.y, b.y, c.y);
    auto coord = [](S m, int extent, int tile, int ntiles) -> int {
        S one = (S)1;
        double t = (((double)(m + one) * 0.5) * (double)extent) / (double)tile;
        return (int)clampS((S)t, (S)0, (S)(ntiles - 1));
    };
    TileRect r;
    r.x0 = coord(minx, W, tw, tiles_x);
    r.y0 = coord(miny, H, th, tiles_y);
    r.x1 = coord(maxx, W, tw, tiles_x);
    r.y1 = coord(maxy, H, th, tiles_y);
    return r;
}

// render.cu:140-152 compute_plane: z = A x + B y + C through the three (x, y, z_ndc).
template <typename S>
inline void compute_plane(P3<S> a, P3<S> b, P3<S> c, S &A, S &B, S &C) {
    S det = a.x * (b.y - c.y) + b.x * (c.y - a.y) + c.x * (a.y - b.y);
    S id = (S)(1.0 / (double)det);  // :144, double literal
    A = (a.z * (b.y - c.y) + b.z * (c.y - a.y) + c.z * (a.y - b.y)) * id;
    B = (a.x * (b.z - c.z) + b.x * (c.z - a.z) + c.x * (a.z - b.z)) * id;
    C = (a.x * (b.y * c.z - c.y * b.z) + b.x * (c.y * a.z - a.y * c.z) + c.x * (a.y * b.z - b.y * a.z)) * id;
}

// render.cu:159-189 one Sutherland-Hodgman pass against nx*x + ny*y - d >= 0.
template <typename S>
inline int clip_halfspace(const P2<S> *in, int n_in, P2<S> *out, S nx, S ny, S d) {
    int n_out = 0;
    P2<S> p0 = in[n_in - 1];
    S d0 = nx * p0.x + ny * p0.y - d;
    bool in0 = d0 >= 0;
    for (int i = 0; i < n_in; i++) {
        P2<S> p1 = in[i];
        S d1 = nx * p1.x + ny * p1.y - d;
        bool in1 = d1 >= 0;
        // The reference's arrays hold 7 vertices, enough for a convex polygon; a
        // sliver whose in/out pattern alternates by rounding could exceed that
        // (undefined behaviour there).  Declared here: capacity 8, the rest dropped.
        if (in1 != in0 && n_out < 8) {
            S t = d0 / (d0 - d1);
            out[n_out].x = p0.x + t * (p1.x - p0.x);
            out[n_out].y = p0.y + t * (p1.y - p0.y);
            n_out++;
        }
        if (in1 && n_out < 8) out[n_out++] = p1;
        p0 = p1; d0 = d1; in0 = in1;
    }
    return n_out;
}

// render.cu:243-268: depth key of (triangle, tile) = min of the plane over the
// triangle clipped to the tile rectangle, 1e30 when the clip is empty.
template <typename S>
inline S tile_depth_key(P3<S> a, P3<S> b, P3<S> c, S A, S B, S C, int tx, int ty, int W, int H, int tw, int th) {
    S xmin = (S)(tx * tw) / W * 2 - 1;
    S xmax = (S)((tx + 1) * tw) / W * 2 - 1;
    S ymin = (S)(ty * th) / H * 2 - 1;
    S ymax = (S)((ty + 1) * th) / H * 2 - 1;
    P2<S> poly[8], buf[8];
    int n = 3;
    poly[0] = {a.x, a.y}; poly[1] = {b.x, b.y}; poly[2] = {c.x, c.y};
    const S nxs[4] = {(S)1, (S)-1, (S)0, (S)0};
    const S nys[4] = {(S)0, (S)0, (S)1, (S)-1};
    const S ds[4] = {xmin, -xmax, ymin, -ymax};
    for (int e = 0; e < 4; e++) {  // :254-257, order +x, -x, +y, -y
        n = clip_halfspace(poly, n, buf, nxs[e], nys[e], ds[e]);
        if (n <= 0) return (S)1e30;  // :259
        for (int i = 0; i < n; i++) poly[i] = buf[i];
    }
    S md = std::numeric_limits<S>::max();
    for (int i = 0; i < n; i++) {
        S pd = A * poly[i].x + B * poly[i].y + C;  // :154-157
        md = (pd < md) ? pd : md;                  // std::min(md, pd), :266
    }
    return md;
}

// Order-preserving map of a float's bits to an unsigned integer.
inline uint32_t orderable(float f) {
    uint32_t b; std::memcpy(&b, &f, 4);
    return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
inline uint64_t orderable(double f) {
    uint64_t b; std::memcpy(&b, &f, 8);
    return b ^ ((b >> 63) ? ~0ull : 0x8000000000000000ull);
}

template <typename S>
inline void load_tri(const S *verts, const int *idx, int t, P3<S> &a, P3<S> &b, P3<S> &c) {
    const S *va = verts + 4 * (size_t)idx[3 * t], *vb = verts + 4 * (size_t)idx[3 * t + 1], *vc = verts + 4 * (size_t)idx[3 * t + 2];
    a = {va[0], va[1], va[2]}; b = {vb[0], vb[1], vb[2]}; c = {vc[0], vc[1], vc[2]};
}

// ---- binning -----------------------------------------------------------------

// render.cu:90-139 count_per_tile: per-tile histogram over the tile AABB of each
// triangle; also the per-triangle overlap count (the quantity the key pipeline scans).
template <typename S>
void bin_count(const S *verts, const int *idx, int M, int W, int H, int tw, int th, int *tri_counts, int *tile_counts) {
    int tiles_x = (W + tw - 1) / tw, tiles_y = (H + th - 1) / th;
    if (tile_counts) std::fill(tile_counts, tile_counts + (size_t)tiles_x * tiles_y, 0);
    for (int t = 0; t < M; t++) {
        P3<S> a, b, c; load_tri(verts, idx, t, a, b, c);
        TileRect r = touched_tiles<S>({a.x, a.y}, {b.x, b.y}, {c.x, c.y}, W, H, tw, th, tiles_x, tiles_y);
        int n = 0;
        if (r.y0 != -1) {
            for (int i = r.x0; i <= r.x1; i++)
                for (int j = r.y0; j <= r.y1; j++) { if (tile_counts) tile_counts[j * tiles_x + i]++; n++; }
        }
        if (tri_counts) tri_counts[t] = n;
    }
}

// Emission in the order the key pipeline defines: triangle id ascending, then
// tile x outer, tile y inner (render.cu:235-236), one (tile, depth key, triangle)
// record per covered tile.  Returns K.  Any output may be null.
template <typename S>
long bin_emit(const S *verts, const int *idx, int M, int W, int H, int tw, int th,
              int *tile_of, S *depth_of, int *tri_of, uint64_t *keys64) {
    int tiles_x = (W + tw - 1) / tw, tiles_y = (H + th - 1) / th;
    long k = 0;
    for (int t = 0; t < M; t++) {
        P3<S> a, b, c; load_tri(verts, idx, t, a, b, c);
        TileRect r = touched_tiles<S>({a.x, a.y}, {b.x, b.y}, {c.x, c.y}, W, H, tw, th, tiles_x, tiles_y);
        if (r.y0 == -1) continue;
        S A, B, C; compute_plane(a, b, c, A, B, C);
        for (int tx = r.x0; tx <= r.x1; tx++)
            for (int ty = r.y0; ty <= r.y1; ty++) {
                S key = tile_depth_key(a, b, c, A, B, C, tx, ty, W, H, tw, th);
                int tile = ty * tiles_x + tx;
                if (tile_of) tile_of[k] = tile;
                if (depth_of) depth_of[k] = key;
                if (tri_of) tri_of[k] = t;
                if (keys64) {
                    if constexpr (sizeof(S) == 4) keys64[k] = ((uint64_t)(uint32_t)tile << 32) | orderable((float)key);
                    else keys64[k] = 0;
                }
                k++;
            }
    }
    return k;
}

// render.cu:286-308 per_tile_lists + render.cu:272-284 sort_depth_ranges: the
// observable after the segmented stable sort -- offsets[T+1], and per tile the
// triangle ids ordered by (depth key, triangle id), with their keys.
template <typename S>
long per_tile_lists(const S *verts, const int *idx, int M, int W, int H, int tw, int th,
                    int *offsets, int *sorted_ids, S *sorted_depths, long capacity) {
    int tiles_x = (W + tw - 1) / tw, tiles_y = (H + th - 1) / th, T = tiles_x * tiles_y;
    std::vector<int> counts(T);
    bin_count<S>(verts, idx, M, W, H, tw, th, nullptr, counts.data());
    offsets[0] = 0;
    for (int t = 0; t < T; t++) offsets[t + 1] = offsets[t] + counts[t];  // :290-295 exclusive scan
    long K = offsets[T];
    if (!sorted_ids || K > capacity) return K;
    std::vector<int> cursor(offsets, offsets + T);
    std::vector<int> ids(K);
    std::vector<S> keys(K);
    for (int t = 0; t < M; t++) {  // :202-270 fill, serial => slot order = triangle id
        P3<S> a, b, c; load_tri(verts, idx, t, a, b, c);
        TileRect r = touched_tiles<S>({a.x, a.y}, {b.x, b.y}, {c.x, c.y}, W, H, tw, th, tiles_x, tiles_y);
        if (r.y0 == -1) continue;
        S A, B, C; compute_plane(a, b, c, A, B, C);
        for (int tx = r.x0; tx <= r.x1; tx++)
            for (int ty = r.y0; ty <= r.y1; ty++) {
                int slot = cursor[ty * tiles_x + tx]++;
                ids[slot] = t;
                keys[slot] = tile_depth_key(a, b, c, A, B, C, tx, ty, W, H, tw, th);
            }
    }
#pragma omp parallel for schedule(dynamic, 16) num_threads(g_threads)
    for (int t = 0; t < T; t++) {  // :280 stable ascending sort inside each segment
        int s = offsets[t], e = offsets[t + 1];
        std::vector<int> perm(e - s);
        for (int i = 0; i < e - s; i++) perm[i] = s + i;
        std::stable_sort(perm.begin(), perm.end(), [&](int p, int q) { return orderable(keys[p]) < orderable(keys[q]); });
        for (int i = 0; i < e - s; i++) { sorted_ids[s + i] = ids[perm[i]]; if (sorted_depths) sorted_depths[s + i] = keys[perm[i]]; }
    }
    return K;
}

// Library-free statement of the key pipeline's remaining integer stages.
void sort_pairs_u64(const uint64_t *keys, const int *vals, long K, uint64_t *keys_out, int *vals_out) {
    std::vector<long> perm(K);
    for (long i = 0; i < K; i++) perm[i] = i;
    std::stable_sort(perm.begin(), perm.end(), [&](long p, long q) { return keys[p] < keys[q]; });
    for (long i = 0; i < K; i++) { keys_out[i] = keys[perm[i]]; vals_out[i] = vals[perm[i]]; }
}
void tile_ranges(const uint64_t *sorted_keys, long K, int T, int *offsets) {
    long i = 0;
    for (int t = 0; t <= T; t++) {
        while (i < K && (long)(sorted_keys[i] >> 32) < t) i++;
        offsets[t] = (int)i;
    }
}

// ---- bary matrices -----------------------------------------------------------

// render.cu:310-337 cartesian_to_bary_kernel.
template <typename S>
void bary_matrices(const S *verts, const int *idx, int M, S *out) {
    for (int t = 0; t < M; t++) {
        P3<S> a, b, c; load_tri(verts, idx, t, a, b, c);
        S denom = a.x * (b.y - c.y) + b.x * (c.y - a.y) + c.x * (a.y - b.y);
        if (std::fabs(denom) < eff_zero<S>()) denom = 1;
        S *m = out + 9 * (size_t)t;
        m[0] = (b.y - c.y) / denom; m[1] = (c.x - b.x) / denom; m[2] = (b.x * c.y - c.x * b.y) / denom;
        m[3] = (c.y - a.y) / denom; m[4] = (a.x - c.x) / denom; m[5] = (c.x * a.y - a.x * c.y) / denom;
        m[6] = (a.y - b.y) / denom; m[7] = (b.x - a.x) / denom; m[8] = (a.x * b.y - b.x * a.y) / denom;
    }
}

// ---- per-fragment math ---------------------------------------------------------

// render.cu:78-88 apply_cart_to_bary.
template <typename S> inline P3<S> apply_bary(const S *m, P2<S> p) {
    return {m[0] * p.x + m[1] * p.y + m[2], m[3] * p.x + m[4] * p.y + m[5], m[6] * p.x + m[7] * p.y + m[8]};
}
// util.h:245-250 scalar interpolate3 with weights.
template <typename S> inline S interp(P3<S> bc, S a, S b, S c, P3<S> w) {
    S denom = bc.x * w.x + bc.y * w.y + bc.z * w.z;
    return (bc.x * a * w.x + bc.y * b * w.y + bc.z * c * w.z) / denom;
}
template <typename S> inline bool outside(P3<S> bc) {  // render.cu:401,438,482
    return bc.x < eff_zero<S>() || bc.y < eff_zero<S>() || bc.z < eff_zero<S>();
}
// render.cu:561-562 pixel centre: evaluated in double, rounded once.
template <typename S> inline P2<S> pixel_centre(int ix, int iy, int W, int H) {
    return {(S)(((double)(S)ix + 0.5) / (double)(S)W * 2.0 - 1.0), (S)(((double)(S)iy + 0.5) / (double)(S)H * 2.0 - 1.0)};
}

template <typename S> struct Scene {
    const S *verts; const int *idx; const S *colors; const S *opac;
    const int *ids; const int *offsets; const S *bary;
    int W, H, tw, th;
    // backward pass only: > 0 makes every gradient array hold, behind its sums, the sums of the magnitudes of what was
    // added (so many vertices further on): the scale that the rounding of a float32 accumulation of the same terms is
    // proportional to.  Test infrastructure, not part of the reference.
    size_t magnitudes_at = 0;
};

template <typename S> struct Frag {  // everything process_forward/backward read for one list entry
    int ia, ib, ic; P3<S> ws;
};

template <typename S> inline bool frag_bary(const Scene<S> &sc, int j, P2<S> pos, int &tri, int &ia, int &ib, int &ic, P3<S> &ws, P3<S> &bc) {
    tri = sc.ids[j];
    ia = sc.idx[3 * tri]; ib = sc.idx[3 * tri + 1]; ic = sc.idx[3 * tri + 2];
    ws = {sc.verts[4 * (size_t)ia + 3], sc.verts[4 * (size_t)ib + 3], sc.verts[4 * (size_t)ic + 3]};
    bc = apply_bary(sc.bary + 9 * (size_t)tri, pos);
    return !outside(bc);
}

template <typename S> struct PixelAcc {
    S alpha = 1; S col[3] = {0, 0, 0}; S depth = 0; S weight = 0; int ends = 0; int blended = 0; int last = 0;
};

// render.cu:417-453 process_forward.
template <typename S>
inline void process_forward(const Scene<S> &sc, int j, int start, P2<S> pos, PixelAcc<S> &px) {
    int tri, ia, ib, ic; P3<S> ws, bc;
    if (!frag_bary(sc, j, pos, tri, ia, ib, ic, ws, bc)) return;
    S o = interp(bc, sc.opac[ia], sc.opac[ib], sc.opac[ic], ws);
    o = clampS(o, (S)0.0, max_opacity<S>());
    S color[3];
    for (int k = 0; k < 3; k++) color[k] = interp(bc, sc.colors[3 * (size_t)ia + k], sc.colors[3 * (size_t)ib + k], sc.colors[3 * (size_t)ic + k], ws);
    S iwx = (S)1.0 / ws.x, iwy = (S)1.0 / ws.y, iwz = (S)1.0 / ws.z;
    S z = interp(bc, iwx, iwy, iwz, P3<S>{1, 1, 1});
    S ao = px.alpha * o;
    px.depth = px.depth + ao * z;
    px.weight = px.weight + ao;
    for (int k = 0; k < 3; k++) px.col[k] = px.col[k] + ao * color[k];
    px.alpha *= (1 - o);
    px.ends++; px.blended++;
    px.last = j - start + 1;
}

// render.cu:338-373 insert_sorted_topk (the ignore_sort branch is never taken).
template <typename S>
inline void insert_topk(int layers, int *topk, S *topk_d, int &n, S d, int value) {
    if (n == layers && d >= topk_d[layers - 1]) return;
    int i = (n < layers) ? n : (layers - 1);
    while (i > 0 && d < topk_d[i - 1]) { topk_d[i] = topk_d[i - 1]; topk[i] = topk[i - 1]; i--; }
    topk_d[i] = d; topk[i] = value;
    if (n < layers) n++;
}

// render.cu:375-415 select_next_k_in_tile.
template <typename S>
inline int select_next_k(const Scene<S> &sc, int K, int *out_j, S *out_d, S lastDepth, int lastJ, int start, int end, P2<S> pos) {
    int n = 0;
    for (int i = 0; i < K; i++) out_d[i] = std::numeric_limits<S>::infinity();
    for (int j = start; j < end; j++) {
        int tri, ia, ib, ic; P3<S> ws, bc;
        if (!frag_bary(sc, j, pos, tri, ia, ib, ic, ws, bc)) continue;
        S pd = interp(bc, sc.verts[4 * (size_t)ia + 2], sc.verts[4 * (size_t)ib + 2], sc.verts[4 * (size_t)ic + 2], ws);
        if (pd < lastDepth) continue;
        if (pd == lastDepth && j <= lastJ) continue;
        insert_topk(K, out_j, out_d, n, pd, j);
    }
    return n;
}

constexpr int LAYERS = 32;  // render.cu:570, :655

// render.cu:540-619 render_forward_kernel, one pixel.
template <typename S>
inline void forward_pixel(const Scene<S> &sc, int ix, int iy, int tile, S thr, bool pps, int max_layers,
                          S *image, S *depthmap, S *weights, int *ends, int *last) {
    int index = iy * sc.W + ix;
    int start = sc.offsets[tile], end = sc.offsets[tile + 1];
    P2<S> pos = pixel_centre<S>(ix, iy, sc.W, sc.H);
    PixelAcc<S> px;
    if (!pps) {
        for (int j = start; j < end && px.alpha > thr && px.blended < max_layers; ++j) process_forward(sc, j, start, pos, px);
    } else {
        int bj[LAYERS]; S bd[LAYERS];
        S lastDepth = -std::numeric_limits<S>::infinity();
        int lastJ = -1;
        while (px.alpha > thr && px.blended < max_layers) {
            int batch = std::min(LAYERS, max_layers - px.blended);
            int found = select_next_k(sc, batch, bj, bd, lastDepth, lastJ, start, end, pos);
            if (found == 0) break;
            int todo = std::min(found, max_layers - px.blended);
            for (int i = 0; i < todo; i++) process_forward(sc, bj[i], start, pos, px);
            lastDepth = bd[todo - 1];
            lastJ = bj[todo - 1];
        }
    }
    if (px.weight > eff_zero<S>()) depthmap[index] = px.depth / px.weight;
    else { depthmap[index] = std::numeric_limits<S>::infinity(); px.weight = 0; }
    weights[index] = px.weight;
    ends[index] = px.ends;
    if (last) last[index] = px.last;
    image[4 * (size_t)index + 0] = px.col[0]; image[4 * (size_t)index + 1] = px.col[1];
    image[4 * (size_t)index + 2] = px.col[2]; image[4 * (size_t)index + 3] = px.alpha;
}

template <typename S>
void render_forward(const Scene<S> &sc, S thr, bool pps, int max_layers, S *image, S *depthmap, S *weights, int *ends, int *last) {
    int tiles_x = (sc.W + sc.tw - 1) / sc.tw, tiles_y = (sc.H + sc.th - 1) / sc.th;
#pragma omp parallel for schedule(dynamic, 1) num_threads(g_threads)
    for (int tile = 0; tile < tiles_x * tiles_y; tile++) {
        int bx = tile % tiles_x, by = tile / tiles_x;
        for (int ly = 0; ly < sc.th; ly++)
            for (int lx = 0; lx < sc.tw; lx++) {
                int ix = bx * sc.tw + lx, iy = by * sc.th + ly;
                if (iy >= sc.H || ix >= sc.W) continue;  // :554
                forward_pixel(sc, ix, iy, tile, thr, pps, max_layers, image, depthmap, weights, ends, last);
            }
    }
}

// util.h:299-317 scalar interpolate3_backward.
template <typename S>
inline void interp_bwd_scalar(S g, P3<S> bc, S a, S b, S c, P3<S> w, S gb[3], S gv[3], S gw[3]) {
    const S B[3] = {bc.x, bc.y, bc.z}, Wt[3] = {w.x, w.y, w.z}, V[3] = {a, b, c};
    S nom = (B[0] * Wt[0] * V[0] + B[1] * Wt[1] * V[1]) + B[2] * Wt[2] * V[2];
    S denom = (B[0] * Wt[0] + B[1] * Wt[1]) + B[2] * Wt[2];
    if (denom * denom < eff_zero<S>()) { for (int k = 0; k < 3; k++) gb[k] = gv[k] = gw[k] = 0; return; }
    S inv2 = (S)1 / (denom * denom);
    for (int k = 0; k < 3; k++) {
        S dfd = (V[k] * Wt[k] * denom - nom * Wt[k]) * inv2;
        gb[k] = g * dfd;
        gv[k] = g * B[k] * Wt[k] / denom;
        gw[k] = g * (B[k] * V[k] * denom - nom * B[k]) * inv2;
    }
}
// util.h:319-355 vector interpolate3_backward.
template <typename S>
inline void interp_bwd_vec(const S g[3], P3<S> bc, const S *a, const S *b, const S *c, P3<S> w,
                           S gb[3], S ga[3], S gbv[3], S gc[3], S gw[3]) {
    const S B[3] = {bc.x, bc.y, bc.z}, Wt[3] = {w.x, w.y, w.z};
    const S *V[3] = {a, b, c};
    S nom[3];
    for (int k = 0; k < 3; k++) nom[k] = (B[0] * Wt[0] * a[k] + B[1] * Wt[1] * b[k]) + B[2] * Wt[2] * c[k];
    S denom = B[0] * Wt[0] + B[1] * Wt[1] + B[2] * Wt[2];
    if (denom * denom < eff_zero<S>()) { for (int k = 0; k < 3; k++) gb[k] = ga[k] = gbv[k] = gc[k] = gw[k] = 0; return; }
    S inv2 = (S)(1.0 / (double)(denom * denom));
    for (int v = 0; v < 3; v++) {
        S dfb[3], dfw[3];
        for (int k = 0; k < 3; k++) {
            dfb[k] = Wt[v] * (V[v][k] * denom - nom[k]) * inv2;
            dfw[k] = (B[v] * V[v][k] * denom - nom[k] * B[v]) * inv2;
        }
        gb[v] = (g[0] * dfb[0] + g[1] * dfb[1]) + g[2] * dfb[2];
        gw[v] = (g[0] * dfw[0] + g[1] * dfw[1]) + g[2] * dfw[2];
    }
    S scale[3];
    for (int v = 0; v < 3; v++) scale[v] = B[v] * Wt[v] / denom;
    for (int k = 0; k < 3; k++) { ga[k] = g[k] * scale[0]; gbv[k] = g[k] * scale[1]; gc[k] = g[k] * scale[2]; }
}

template <typename S> inline S cross2(S ax, S ay, S bx, S by) { return ax * by - ay * bx; }  // util.h:384-388

// util.h:395-403 barycentric.
template <typename S> inline P3<S> barycentric(P2<S> v0, P2<S> v1, P2<S> v2, P2<S> p) {
    S T = cross2(v1.x - v0.x, v1.y - v0.y, v2.x - v0.x, v2.y - v0.y);
    S a = cross2(v1.x - p.x, v1.y - p.y, v2.x - p.x, v2.y - p.y) / T;
    S b = cross2(v2.x - p.x, v2.y - p.y, v0.x - p.x, v0.y - p.y) / T;
    S c = cross2(v0.x - p.x, v0.y - p.y, v1.x - p.x, v1.y - p.y) / T;
    return {a, b, c};
}

// util.h:405-455 barycentric_backward: J[v][axis][k] = d bary_k / d vertex_v.axis, v=3 is the point.
template <typename S>
inline bool barycentric_jacobian(P2<S> a, P2<S> b, P2<S> c, P2<S> p, S J[4][2][3]) {
    P3<S> l = barycentric(a, b, c, p);
    S d = a.x * (b.y - c.y) + b.x * (-a.y + c.y) + c.x * (a.y - b.y);
    if (std::fabs(d) < eff_zero<S>()) return false;
    J[0][0][0] = l.x * (-b.y + c.y) / d;
    J[0][0][1] = (-c.y - l.y * (b.y - c.y) + p.y) / d;
    J[0][0][2] = (b.y - l.z * (b.y - c.y) - p.y) / d;
    J[0][1][0] = l.x * (b.x - c.x) / d;
    J[0][1][1] = (c.x + l.y * (b.x - c.x) - p.x) / d;
    J[0][1][2] = (-b.x + l.z * (b.x - c.x) + p.x) / d;
    J[1][0][0] = (c.y + l.x * (a.y - c.y) - p.y) / d;
    J[1][0][1] = l.y * (a.y - c.y) / d;
    J[1][0][2] = (-a.y + l.z * (a.y - c.y) + p.y) / d;
    J[1][1][0] = (-c.x - l.x * (a.x - c.x) + p.x) / d;
    J[1][1][1] = l.y * (-a.x + c.x) / d;
    J[1][1][2] = (a.x - l.z * (a.x - c.x) - p.x) / d;
    J[2][0][0] = (-b.y - l.x * (a.y - b.y) + p.y) / d;
    J[2][0][1] = (a.y - l.y * (a.y - b.y) - p.y) / d;
    J[2][0][2] = l.z * (-a.y + b.y) / d;
    J[2][1][0] = (b.x + l.x * (a.x - b.x) - p.x) / d;
    J[2][1][1] = (-a.x + l.y * (a.x - b.x) + p.x) / d;
    J[2][1][2] = l.z * (a.x - b.x) / d;
    J[3][0][0] = (b.y - c.y) / d;
    J[3][0][1] = (-a.y + c.y) / d;
    J[3][0][2] = (a.y - b.y) / d;
    J[3][1][0] = (-b.x + c.x) / d;
    J[3][1][1] = (a.x - c.x) / d;
    J[3][1][2] = (-a.x + b.x) / d;
    return true;
}
template <typename S>
inline void barycentric_bwd(const S g[3], P2<S> a, P2<S> b, P2<S> c, P2<S> p, S out[4][2]) {
    S J[4][2][3];
    if (!barycentric_jacobian(a, b, c, p, J)) { for (int v = 0; v < 4; v++) out[v][0] = out[v][1] = 0; return; }
    for (int v = 0; v < 4; v++)
        for (int ax = 0; ax < 2; ax++) out[v][ax] = g[0] * J[v][ax][0] + g[1] * J[v][ax][1] + g[2] * J[v][ax][2];
}
// The scale of a position term (test infrastructure, not part of the reference).  A numerator such as
// -c.y - l.y (b.y - c.y) + p.y is a small difference of screen coordinates of order one: its float32 value is
// uncertain by 2^-24 of the SUM of its addends' magnitudes, whichever way it is evaluated (contracted into a fused
// multiply-add or not, with l off by an ulp or not).  So every Jacobian entry is taken with the magnitudes of its
// numerator's addends, and g with the magnitudes of the parts it is the sum of.
template <typename S>
inline void barycentric_bwd_magnitude(const S g[3], P2<S> a, P2<S> b, P2<S> c, P2<S> p, S out[4][2]) {
    for (int v = 0; v < 4; v++) out[v][0] = out[v][1] = 0;
    P3<S> l = barycentric(a, b, c, p);
    S d = a.x * (b.y - c.y) + b.x * (-a.y + c.y) + c.x * (a.y - b.y);
    if (std::fabs(d) < eff_zero<S>()) return;
    const S id = 1 / std::fabs(d);
    const auto sum3 = [&](S u, S m, S q) { return (std::fabs(u) + std::fabs(m) + std::fabs(q)) * id; };
    const auto prod = [&](S m) { return std::fabs(m) * id; };
    S J[3][2][3];
    J[0][0][0] = prod(l.x * (-b.y + c.y));
    J[0][0][1] = sum3(c.y, l.y * (b.y - c.y), p.y);
    J[0][0][2] = sum3(b.y, l.z * (b.y - c.y), p.y);
    J[0][1][0] = prod(l.x * (b.x - c.x));
    J[0][1][1] = sum3(c.x, l.y * (b.x - c.x), p.x);
    J[0][1][2] = sum3(b.x, l.z * (b.x - c.x), p.x);
    J[1][0][0] = sum3(c.y, l.x * (a.y - c.y), p.y);
    J[1][0][1] = prod(l.y * (a.y - c.y));
    J[1][0][2] = sum3(a.y, l.z * (a.y - c.y), p.y);
    J[1][1][0] = sum3(c.x, l.x * (a.x - c.x), p.x);
    J[1][1][1] = prod(l.y * (-a.x + c.x));
    J[1][1][2] = sum3(a.x, l.z * (a.x - c.x), p.x);
    J[2][0][0] = sum3(b.y, l.x * (a.y - b.y), p.y);
    J[2][0][1] = sum3(a.y, l.y * (a.y - b.y), p.y);
    J[2][0][2] = prod(l.z * (-a.y + b.y));
    J[2][1][0] = sum3(b.x, l.x * (a.x - b.x), p.x);
    J[2][1][1] = sum3(a.x, l.y * (a.x - b.x), p.x);
    J[2][1][2] = prod(l.z * (a.x - b.x));
    for (int v = 0; v < 3; v++)
        for (int ax = 0; ax < 2; ax++) out[v][ax] = g[0] * J[v][ax][0] + g[1] * J[v][ax][1] + g[2] * J[v][ax][2];
}

template <typename S> struct BackState {
    S final_alpha, alpha; S s[3] = {0, 0, 0}; S oa = 0, zoa = 0; S final_weight, final_depth;
};

// *p += v, and, if `behind` is not 0, p[behind] += magnitude (see Scene::magnitudes_at).
inline void accum(double *p, double v, size_t behind = 0, double magnitude = 0.0) {
#pragma omp atomic
    *p += v;
    if (behind) {
#pragma omp atomic
        p[behind] += magnitude;
    }
}

// render.cu:455-538 process_backward.  Gradients are accumulated in double: the
// oracle returns the exactly accumulated sum of the per-fragment terms, so a
// comparison with it measures only the summation error of the path under test.
template <typename S>
inline void process_backward(const Scene<S> &sc, int j, P2<S> pos, const S *gout, S gdepth, BackState<S> &st,
                             double *gV, double *gC, double *gO) {
    int tri, ia, ib, ic; P3<S> ws, bc;
    if (!frag_bary(sc, j, pos, tri, ia, ib, ic, ws, bc)) return;
    const int vid[3] = {ia, ib, ic};
    S o = interp(bc, sc.opac[ia], sc.opac[ib], sc.opac[ic], ws);
    o = clampS(o, (S)0.0, max_opacity<S>());
    S color[3];
    const S *ca = sc.colors + 3 * (size_t)ia, *cb = sc.colors + 3 * (size_t)ib, *cc = sc.colors + 3 * (size_t)ic;
    for (int k = 0; k < 3; k++) color[k] = interp(bc, ca[k], cb[k], cc[k], ws);
    S iw[3] = {(S)1.0 / ws.x, (S)1.0 / ws.y, (S)1.0 / ws.z};
    P3<S> ones = {1, 1, 1};
    S z = interp(bc, iw[0], iw[1], iw[2], ones);

    S om = 1 - o;
    S t3[3];
    for (int k = 0; k < 3; k++) t3[k] = (color[k] * st.alpha - st.s[k]) / om * gout[k];
    S drgb_do = ((t3[0] + t3[1]) + t3[2]) + gout[3] * (-st.final_alpha / om);  // :491
    st.alpha /= ((S)1.0 - o);                                                  // :492
    for (int k = 0; k < 3; k++) st.s[k] += color[k] * o * st.alpha;            // :493
    S ddw_do = st.alpha - st.oa / ((S)1.0 - o);                                // :494
    S dud_do = st.alpha * z - st.zoa / ((S)1.0 - o);                           // :495
    st.oa = st.oa + o * st.alpha;                                              // :496
    st.zoa = st.zoa + z * o * st.alpha;                                        // :497
    S dd_do = (dud_do - st.final_depth * ddw_do) / st.final_weight * gdepth;   // :499
    if (st.final_weight < eff_zero<S>()) dd_do = 0;
    S d_do = drgb_do + dd_do;

    S gb_o[3], gv_o[3], gw_o[3];
    interp_bwd_scalar(d_do, bc, sc.opac[ia], sc.opac[ib], sc.opac[ic], ws, gb_o, gv_o, gw_o);
    const size_t mag = sc.magnitudes_at;
    for (int v = 0; v < 3; v++) accum(gO + vid[v], (double)gv_o[v], mag, std::fabs((double)gv_o[v]));  // :506-508

    S ao = st.alpha * o;
    S gcol[3] = {ao * gout[0], ao * gout[1], ao * gout[2]};                    // :510
    S gb_c[3], ga[3], gbv[3], gc[3], gw_c[3];
    interp_bwd_vec(gcol, bc, ca, cb, cc, ws, gb_c, ga, gbv, gc, gw_c);
    for (int k = 0; k < 3; k++) {                                              // :514-516
        accum(gC + 3 * (size_t)ia + k, (double)ga[k], 3 * mag, std::fabs((double)ga[k]));
        accum(gC + 3 * (size_t)ib + k, (double)gbv[k], 3 * mag, std::fabs((double)gbv[k]));
        accum(gC + 3 * (size_t)ic + k, (double)gc[k], 3 * mag, std::fabs((double)gc[k]));
    }
    S dd_dz = ao * gdepth / st.final_weight;                                   // :517
    if (st.final_weight < eff_zero<S>()) dd_dz = 0;
    S gb_z[3], gv_z[3], gw_z[3];
    interp_bwd_scalar(dd_dz, bc, iw[0], iw[1], iw[2], ones, gb_z, gv_z, gw_z);
    const S wv[3] = {ws.x, ws.y, ws.z};
    S dd_dw[3];
    for (int v = 0; v < 3; v++) dd_dw[v] = -gv_z[v] / (wv[v] * wv[v]);         // :523-525

    S gbary[3];
    for (int k = 0; k < 3; k++) gbary[k] = gb_o[k] + gb_c[k] + gb_z[k];        // :527
    S dxy[4][2];
    const S *va = sc.verts + 4 * (size_t)ia, *vb = sc.verts + 4 * (size_t)ib, *vc = sc.verts + 4 * (size_t)ic;
    barycentric_bwd<S>(gbary, {va[0], va[1]}, {vb[0], vb[1]}, {vc[0], vc[1]}, pos, dxy);
    // a position term is a sum of three products that may cancel, and each of the three barycentric gradients is a sum
    // of three parts: its scale is that of the parts, which barycentric_bwd turns into with the magnitudes as input
    S dxy_mag[4][2] = {};
    if (mag) {
        S gbary_mag[3];
        for (int k = 0; k < 3; k++) gbary_mag[k] = std::fabs(gb_o[k]) + std::fabs(gb_c[k]) + std::fabs(gb_z[k]);
        barycentric_bwd_magnitude<S>(gbary_mag, {va[0], va[1]}, {vb[0], vb[1]}, {vc[0], vc[1]}, pos, dxy_mag);
    }
    for (int v = 0; v < 3; v++) {                                              // :530-537
        S dw = gw_o[v] + gw_c[v] + gw_z[v];
        accum(gV + 4 * (size_t)vid[v] + 0, (double)dxy[v][0], 4 * mag, (double)dxy_mag[v][0]);
        accum(gV + 4 * (size_t)vid[v] + 1, (double)dxy[v][1], 4 * mag, (double)dxy_mag[v][1]);
        accum(gV + 4 * (size_t)vid[v] + 3, (double)(dw + dd_dw[v]), 4 * mag,
              std::fabs((double)gw_o[v]) + std::fabs((double)gw_c[v]) + std::fabs((double)gw_z[v]) + std::fabs((double)dd_dw[v]));
    }
}

// render.cu:621-695 render_backward_kernel, one pixel.
//   literal != 0: the traversal exactly as written in the reference.
//   literal == 0: the declared policy -- fragments are visited in exact reverse
//     blend order.  Identical to the literal traversal when per_pixel_sort is on
//     and at most 32 fragments were blended (the reference's tested regime);
//     differs where the literal traversal is not the derivative of the forward
//     pass (per_pixel_sort off: forward-order walk over `ends` list slots,
//     :659-666; per_pixel_sort on with more than 32 blended: batches visited
//     front to back, :673-693).
template <typename S>
inline void backward_pixel(const Scene<S> &sc, int ix, int iy, int tile, bool pps, int max_layers, int literal,
                           const S *gimage, const S *gdepthmap, const S *image, const S *depthmap, const S *weights,
                           const int *ends, double *gV, double *gC, double *gO) {
    int index = iy * sc.W + ix;
    int start = sc.offsets[tile], tile_end = sc.offsets[tile + 1];
    int limit = std::min(ends[index], max_layers);  // :642
    P2<S> pos = pixel_centre<S>(ix, iy, sc.W, sc.H);
    BackState<S> st;
    st.final_alpha = image[4 * (size_t)index + 3];
    st.alpha = st.final_alpha;
    st.final_weight = weights[index];
    st.final_depth = depthmap[index];
    const S *gout = gimage + 4 * (size_t)index;
    S gd = gdepthmap[index];
    if (!pps) {
        if (literal) {
            for (int i = 0; i < limit; i++) process_backward(sc, start + i, pos, gout, gd, st, gV, gC, gO);
        } else {
            // the blended fragments are the first `limit` inside-hits in list order
            std::vector<int> hits; hits.reserve(limit);
            for (int j = start; j < tile_end && (int)hits.size() < limit; j++) {
                int tri, ia, ib, ic; P3<S> ws, bc;
                if (frag_bary(sc, j, pos, tri, ia, ib, ic, ws, bc)) hits.push_back(j);
            }
            for (int i = (int)hits.size() - 1; i >= 0; i--) process_backward(sc, hits[i], pos, gout, gd, st, gV, gC, gO);
        }
        return;
    }
    if (literal || limit <= LAYERS) {
        int bj[LAYERS]; S bd[LAYERS];
        S lastDepth = -std::numeric_limits<S>::infinity();
        int lastJ = -1, remaining = limit;
        while (remaining > 0) {
            int batch = std::min(LAYERS, remaining);
            int found = select_next_k(sc, batch, bj, bd, lastDepth, lastJ, start, tile_end, pos);
            if (found == 0) break;
            int todo = std::min(found, remaining);
            for (int i = todo - 1; i >= 0; --i) process_backward(sc, bj[i], pos, gout, gd, st, gV, gC, gO);
            lastDepth = bd[todo - 1]; lastJ = bj[todo - 1];
            remaining -= todo;
        }
        return;
    }
    // per-pixel order, more than 32 blended: full (depth, j) order, reversed.
    struct DJ { S d; int j; };
    std::vector<DJ> fr;
    for (int j = start; j < tile_end; j++) {
        int tri, ia, ib, ic; P3<S> ws, bc;
        if (!frag_bary(sc, j, pos, tri, ia, ib, ic, ws, bc)) continue;
        S pd = interp(bc, sc.verts[4 * (size_t)ia + 2], sc.verts[4 * (size_t)ib + 2], sc.verts[4 * (size_t)ic + 2], ws);
        fr.push_back({pd, j});
    }
    std::stable_sort(fr.begin(), fr.end(), [](const DJ &p, const DJ &q) { return p.d < q.d; });
    int n = std::min((int)fr.size(), limit);
    for (int i = n - 1; i >= 0; --i) process_backward(sc, fr[i].j, pos, gout, gd, st, gV, gC, gO);
}

template <typename S>
void render_backward(const Scene<S> &sc, bool pps, int max_layers, int literal,
                     const S *gimage, const S *gdepthmap, const S *image, const S *depthmap, const S *weights,
                     const int *ends, int V, double *gV, double *gC, double *gO) {
    const size_t copies = sc.magnitudes_at ? 2 : 1;  // sums, and behind them the magnitudes
    std::fill(gV, gV + copies * 4 * (size_t)V, 0.0); std::fill(gC, gC + copies * 3 * (size_t)V, 0.0);
    std::fill(gO, gO + copies * (size_t)V, 0.0);
    int tiles_x = (sc.W + sc.tw - 1) / sc.tw, tiles_y = (sc.H + sc.th - 1) / sc.th;
#pragma omp parallel for schedule(dynamic, 1) num_threads(g_threads)
    for (int tile = 0; tile < tiles_x * tiles_y; tile++) {
        int bx = tile % tiles_x, by = tile / tiles_x;
        for (int ly = 0; ly < sc.th; ly++)
            for (int lx = 0; lx < sc.tw; lx++) {
                int ix = bx * sc.tw + lx, iy = by * sc.th + ly;
                if (iy >= sc.H || ix >= sc.W) continue;
                backward_pixel(sc, ix, iy, tile, pps, max_layers, literal, gimage, gdepthmap, image, depthmap, weights, ends, gV, gC, gO);
            }
    }
}

}  // namespace

// ---- C entry points (ctypes) -----------------------------------------------------

#define TGO_INSTANTIATE(SUF, S)                                                                                            \
    extern "C" void tgo_bin_count_##SUF(const S *v, const int *i, int M, int W, int H, int tw, int th, int *tri_counts,    \
                                        int *tile_counts) {                                                                \
        bin_count<S>(v, i, M, W, H, tw, th, tri_counts, tile_counts);                                                      \
    }                                                                                                                      \
    extern "C" long tgo_bin_emit_##SUF(const S *v, const int *i, int M, int W, int H, int tw, int th, int *tile_of,        \
                                       S *depth_of, int *tri_of, uint64_t *keys64) {                                       \
        return bin_emit<S>(v, i, M, W, H, tw, th, tile_of, depth_of, tri_of, keys64);                                      \
    }                                                                                                                      \
    extern "C" long tgo_per_tile_lists_##SUF(const S *v, const int *i, int M, int W, int H, int tw, int th, int *offsets,  \
                                             int *sorted_ids, S *sorted_depths, long capacity) {                          \
        return per_tile_lists<S>(v, i, M, W, H, tw, th, offsets, sorted_ids, sorted_depths, capacity);                     \
    }                                                                                                                      \
    extern "C" void tgo_bary_##SUF(const S *v, const int *i, int M, S *out) { bary_matrices<S>(v, i, M, out); }            \
    extern "C" void tgo_forward_##SUF(const S *v, const int *i, const S *c, const S *o, const int *ids,                    \
                                      const int *offsets, const S *bary, int W, int H, int tw, int th, S thr, int pps,     \
                                      int max_layers, S *image, S *depthmap, S *weights, int *ends, int *last) {           \
        Scene<S> sc{v, i, c, o, ids, offsets, bary, W, H, tw, th};                                                         \
        render_forward<S>(sc, thr, pps != 0, max_layers, image, depthmap, weights, ends, last);                            \
    }                                                                                                                      \
    extern "C" void tgo_backward_##SUF(const S *gimage, const S *gdepth, const S *v, const int *i, const S *c, const S *o, \
                                       const int *ids, const int *offsets, const S *bary, const S *image,                  \
                                       const S *depthmap, const S *weights, const int *ends, int W, int H, int tw, int th, \
                                       int pps, int max_layers, int literal, int V, double *gV, double *gC, double *gO,    \
                                       int magnitudes) {                                                                   \
        Scene<S> sc{v, i, c, o, ids, offsets, bary, W, H, tw, th};                                                         \
        sc.magnitudes_at = magnitudes ? (size_t)V : 0;                                                                     \
        render_backward<S>(sc, pps != 0, max_layers, literal, gimage, gdepth, image, depthmap, weights, ends, V, gV, gC,   \
                           gO);                                                                                            \
    }                                                                                                                      \
    /* component hooks: src/trigrad/tests.cu:43-76 */                                                                      \
    extern "C" void tgo_barycentric_##SUF(const S *p0, const S *p1, const S *q0, const S *q1, S *out) {                    \
        P3<S> r = barycentric<S>({p0[0], p0[1]}, {p1[0], p1[1]}, {q0[0], q0[1]}, {q1[0], q1[1]});                          \
        out[0] = r.x; out[1] = r.y; out[2] = r.z;                                                                          \
    }                                                                                                                      \
    extern "C" void tgo_barycentric_backward_##SUF(const S *g, const S *a, const S *b, const S *c, const S *p, S *out) {   \
        S o[4][2];                                                                                                         \
        barycentric_bwd<S>(g, {a[0], a[1]}, {b[0], b[1]}, {c[0], c[1]}, {p[0], p[1]}, o);                                  \
        for (int v = 0; v < 4; v++) { out[2 * v] = o[v][0]; out[2 * v + 1] = o[v][1]; }                                    \
    }                                                                                                                      \
    extern "C" S tgo_interpolate3_scalar_##SUF(const S *bc, S a, S b, S c, const S *w) {                                   \
        return interp<S>({bc[0], bc[1], bc[2]}, a, b, c, {w[0], w[1], w[2]});                                              \
    }                                                                                                                      \
    extern "C" void tgo_interpolate3_scalar_backward_##SUF(S g, const S *bc, S a, S b, S c, const S *w, S *gb, S *gv,      \
                                                           S *gw) {                                                        \
        interp_bwd_scalar<S>(g, {bc[0], bc[1], bc[2]}, a, b, c, {w[0], w[1], w[2]}, gb, gv, gw);                           \
    }                                                                                                                      \
    extern "C" void tgo_interpolate3_vector_##SUF(const S *bc, const S *a, const S *b, const S *c, const S *w, S *out) {   \
        for (int k = 0; k < 3; k++) out[k] = interp<S>({bc[0], bc[1], bc[2]}, a[k], b[k], c[k], {w[0], w[1], w[2]});       \
    }                                                                                                                      \
    extern "C" void tgo_interpolate3_vector_backward_##SUF(const S *g, const S *bc, const S *a, const S *b, const S *c,    \
                                                           const S *w, S *gb, S *ga, S *gbv, S *gc, S *gw) {               \
        interp_bwd_vec<S>(g, {bc[0], bc[1], bc[2]}, a, b, c, {w[0], w[1], w[2]}, gb, ga, gbv, gc, gw);                     \
    }

TGO_INSTANTIATE(f32, float)
TGO_INSTANTIATE(f64, double)

extern "C" void tgo_sort_pairs_u64(const uint64_t *keys, const int *vals, long K, uint64_t *keys_out, int *vals_out) {
    sort_pairs_u64(keys, vals, K, keys_out, vals_out);
}
extern "C" void tgo_tile_ranges(const uint64_t *sorted_keys, long K, int T, int *offsets) { tile_ranges(sorted_keys, K, T, offsets); }
extern "C" void tgo_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
extern "C" int tgo_max_threads() {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
