"""Pins the binning / key / sort / ranges / bary parts of the CPU oracle against
closed forms, brute force and library routines (no GPU).  The reference's own
tests hold no expected values for these stages, so each check is chosen so that
a plausible slip (wrong rounding direction, swapped loop order, transposed
matrix, sign of a clip plane) fails it."""
import numpy as np
import pytest

import scenes as S

F = np.float32


def _tri_scene(xy, z=(1.0, 1.0, 1.0)):
    xy = np.asarray(xy, dtype=F).reshape(-1, 3, 2)
    n = xy.shape[0]
    zz = np.broadcast_to(np.asarray(z, dtype=F), (n, 3))
    v = np.concatenate([xy, zz[..., None], (1 / zz)[..., None]], axis=-1).reshape(3 * n, 4).astype(F)
    return v, np.arange(3 * n, dtype=np.int32).reshape(n, 3)


def test_tile_rect_closed_form_for_in_screen_boxes(oracle):
    """A triangle whose AABB is [x0,x1]x[y0,y1] in pixels, strictly inside the
    screen and off tile boundaries, covers (floor(x1/tw)-floor(x0/tw)+1) *
    (floor(y1/th)-floor(y0/th)+1) tiles."""
    rng = np.random.default_rng(0)
    W, H, tw, th = 640, 360, 16, 16
    n = 500
    x0 = rng.uniform(1, W - 2, n); x1 = rng.uniform(1, W - 2, n)
    y0 = rng.uniform(1, H - 2, n); y1 = rng.uniform(1, H - 2, n)
    x0, x1 = np.minimum(x0, x1), np.maximum(x0, x1) + 0.25
    y0, y1 = np.minimum(y0, y1), np.maximum(y0, y1) + 0.25
    for a in (x0, x1, y0, y1):  # stay clear of tile boundaries (float32 rounding of the NDC round trip)
        near = np.abs(a / 16 - np.round(a / 16)) < 1e-3
        a[near] += 0.37
    ndc = lambda p, e: p / e * 2 - 1
    xy = np.stack([np.stack([ndc(x0, W), ndc(y0, H)], -1), np.stack([ndc(x1, W), ndc(y0, H)], -1),
                   np.stack([ndc(x0, W), ndc(y1, H)], -1)], axis=1)
    v, idx = _tri_scene(xy)
    tri, tile = oracle.bin_count(v, idx, W, H, tw, th)
    want = (np.floor(x1 / tw) - np.floor(x0 / tw) + 1) * (np.floor(y1 / th) - np.floor(y0 / th) + 1)
    np.testing.assert_array_equal(tri, want.astype(np.int32))
    assert tile.sum() == tri.sum()


def test_tile_counts_brute_force_and_clamping(oracle):
    """Per-tile histogram = brute-force count of AABB/tile overlaps; off-screen
    triangles are clamped into border tiles, not culled (render.cu:72-75)."""
    W, H, tw, th = 100, 70, 16, 16  # partial last tile column and row
    s = S.random_soup(300, W, H, seed=5, sigma_px=20.0)
    v, idx = s["vertices"], s["indices"]
    tri, tile = oracle.bin_count(v, idx, W, H, tw, th)
    tiles_x, tiles_y = -(-W // tw), -(-H // th)
    want_tile = np.zeros(tiles_x * tiles_y, np.int64)
    want_tri = np.zeros(idx.shape[0], np.int64)
    P = v[idx][:, :, :2].astype(np.float64)
    for t in range(idx.shape[0]):
        lo, hi = P[t].min(0), P[t].max(0)
        tx0 = int(np.clip(np.trunc((np.float32(lo[0]) + np.float32(1)).astype(np.float64) * 0.5 * W / tw), 0, tiles_x - 1))
        tx1 = int(np.clip(np.trunc((np.float32(hi[0]) + np.float32(1)).astype(np.float64) * 0.5 * W / tw), 0, tiles_x - 1))
        ty0 = int(np.clip(np.trunc((np.float32(lo[1]) + np.float32(1)).astype(np.float64) * 0.5 * H / th), 0, tiles_y - 1))
        ty1 = int(np.clip(np.trunc((np.float32(hi[1]) + np.float32(1)).astype(np.float64) * 0.5 * H / th), 0, tiles_y - 1))
        for ty in range(ty0, ty1 + 1):
            for tx in range(tx0, tx1 + 1):
                want_tile[ty * tiles_x + tx] += 1
                want_tri[t] += 1
    np.testing.assert_array_equal(tile, want_tile)
    np.testing.assert_array_equal(tri, want_tri)
    # a triangle entirely right of the screen lands in the last tile column
    v2, idx2 = _tri_scene([[[3.0, -0.1], [3.2, -0.1], [3.0, 0.1]]])
    tri2, tile2 = oracle.bin_count(v2, idx2, W, H, tw, th)
    assert tri2[0] >= 1 and tile2.reshape(tiles_y, tiles_x)[:, :-1].sum() == 0


def test_degenerate_triangles_touch_no_tile(oracle):
    v, idx = _tri_scene([[[0, 0], [0.5, 0.5], [0.25, 0.25]],          # collinear
                         [[0.1, 0.1], [0.1, 0.1], [0.3, 0.2]],        # repeated vertex
                         [[np.nan, 0], [0.5, 0.5], [0.2, 0.1]],       # NaN
                         [[np.inf, 0], [0.5, 0.5], [0.2, 0.1]],       # infinite
                         [[0, 0], [0.5, 0], [0, 0.5]]])               # ordinary
    tri, _ = oracle.bin_count(v, idx, 64, 64, 16, 16)
    assert tri.tolist()[:4] == [0, 0, 0, 0] and tri[4] > 0


def test_emission_order_and_sort_match_library_routines(oracle):
    s = S.random_soup(2000, 320, 200, seed=8, sigma_px=15.0, varying_w=True)
    W, H = 320, 200
    v, idx = s["vertices"], s["indices"]
    em = oracle.bin_emit(v, idx, W, H)
    tri_counts, tile_counts = oracle.bin_count(v, idx, W, H)
    K = int(tri_counts.sum())
    assert em["tri"].shape[0] == K
    # triangle ids ascending, tile x outer / tile y inner inside a triangle
    assert (np.diff(em["tri"]) >= 0).all()
    tiles_x = -(-W // 16)
    for t in np.flatnonzero(tri_counts > 1)[:50]:
        sel = em["tile"][em["tri"] == t]
        tx, ty = sel % tiles_x, sel // tiles_x
        order = np.lexsort((ty, tx))
        np.testing.assert_array_equal(order, np.arange(len(sel)))
    # 64-bit keys: tile in the high word, order-preserving float bits in the low word
    bits = em["depth"].view(np.uint32)
    ordb = np.where(bits >> 31 == 1, ~bits, bits | np.uint32(0x80000000)).astype(np.uint64)
    np.testing.assert_array_equal(em["keys64"], (em["tile"].astype(np.uint64) << np.uint64(32)) | ordb)
    # sort = numpy lexsort on (tile, depth as float, triangle id)
    sk, sv = oracle.sort_pairs_u64(em["keys64"], em["tri"])
    order = np.lexsort((em["tri"], em["depth"], em["tile"]))
    np.testing.assert_array_equal(sv, em["tri"][order])
    np.testing.assert_array_equal(sk, em["keys64"][order])
    # ranges = searchsorted, and = cumsum of the per-tile histogram
    T = tile_counts.shape[0]
    off = oracle.tile_ranges(sk, T)
    np.testing.assert_array_equal(off, np.searchsorted((sk >> np.uint64(32)).astype(np.int64), np.arange(T + 1)))
    np.testing.assert_array_equal(off, np.concatenate([[0], np.cumsum(tile_counts)]))
    # the reference-shaped route (histogram, cumsum, slot fill, stable segmented sort) gives the same lists
    ro, rids, rdepths = oracle.per_tile_lists(v, idx, W, H)
    np.testing.assert_array_equal(ro, off)
    np.testing.assert_array_equal(rids, sv)
    np.testing.assert_array_equal(rdepths, em["depth"][order])


def test_orderable_key_handles_negative_depths(oracle):
    """z in NDC may be negative (tests/testcases.py:138-165 gives z = -1): the
    key order must be the numeric order, which raw float bits would invert."""
    xy = [[[-0.5, -0.5], [0.5, -0.5], [0.0, 0.5]]] * 4
    v, idx = _tri_scene(xy, z=(1.0, 1.0, 1.0))
    for t, z in enumerate([-0.25, 0.5, -0.75, 0.0]):
        v[3 * t:3 * t + 3, 2] = z
    off, ids, depths = oracle.per_tile_lists(v, idx, 32, 32)
    for t in range(4):
        seg = ids[off[t]:off[t + 1]]
        if len(seg) == 4:
            assert seg.tolist() == [2, 0, 3, 1]
    assert (np.diff(depths[off[0]:off[1]]) >= 0).all()


def _plane_min_over_clip(P, z, rect, n=400):
    """min of the z-plane over triangle-intersect-rect by dense float64 sampling plus exact candidates."""
    (xmin, xmax, ymin, ymax) = rect
    A = np.array([[P[0, 0], P[0, 1], 1], [P[1, 0], P[1, 1], 1], [P[2, 0], P[2, 1], 1]], dtype=np.float64)
    coef = np.linalg.solve(A, np.asarray(z, dtype=np.float64))
    xs = np.linspace(xmin, xmax, n); ys = np.linspace(ymin, ymax, n)
    X, Y = np.meshgrid(xs, ys)
    pts = np.stack([X.ravel(), Y.ravel()], -1)
    M = np.linalg.inv(np.array([[P[0, 0], P[1, 0], P[2, 0]], [P[0, 1], P[1, 1], P[2, 1]], [1, 1, 1]], dtype=np.float64))
    bary = (M @ np.concatenate([pts, np.ones((len(pts), 1))], 1).T).T
    inside = (bary >= -1e-12).all(1)
    if not inside.any():
        return None
    return float((pts[inside] @ coef[:2] + coef[2]).min())


def test_depth_key_is_plane_min_over_clipped_triangle(oracle):
    rng = np.random.default_rng(3)
    W = H = 64
    checked = 0
    for trial in range(40):
        P = rng.uniform(-0.9, 0.9, size=(3, 2))
        e1, e2 = P[1] - P[0], P[2] - P[0]
        if abs(e1[0] * e2[1] - e1[1] * e2[0]) < 0.05:
            continue
        z = rng.uniform(0.5, 5.0, size=3)
        v = np.concatenate([P, z[:, None], 1 / z[:, None]], 1).astype(F)
        idx = np.array([[0, 1, 2]], np.int32)
        em = oracle.bin_emit(v, idx, W, H)
        for tile, key in zip(em["tile"], em["depth"]):
            tx, ty = tile % 4, tile // 4
            rect = (tx * 16 / W * 2 - 1, (tx + 1) * 16 / W * 2 - 1, ty * 16 / H * 2 - 1, (ty + 1) * 16 / H * 2 - 1)
            want = _plane_min_over_clip(v[:, :2].astype(np.float64), v[:, 2].astype(np.float64), rect)
            if want is None:
                # the sampler found no interior point: either truly empty (far key) or a sliver
                continue
            assert key != F(1e30)
            span = np.ptp(z)
            assert key <= want + 1e-4 * span and key >= want - 0.02 * span, (key, want)
            checked += 1
    assert checked > 100


def test_depth_key_special_cases(oracle):
    # constant-z triangle: the key is z wherever the triangle meets the tile, 1e30 elsewhere
    v, idx = _tri_scene([[[-0.9, -0.9], [0.9, -0.8], [-0.8, 0.9]]], z=(2.5, 2.5, 2.5))
    em = oracle.bin_emit(v, idx, 64, 64)
    real = em["depth"][em["depth"] != F(1e30)]
    assert len(real) > 4 and np.allclose(real, 2.5, rtol=1e-5)
    assert (em["depth"] == F(1e30)).any()  # AABB corner tiles the triangle does not reach
    # triangle inside one tile: the key is the smallest vertex z
    v, idx = _tri_scene([[[0.05, 0.05], [0.2, 0.08], [0.1, 0.2]]], z=(3.0, 1.5, 2.0))
    em = oracle.bin_emit(v, idx, 64, 64)
    assert em["tile"].shape[0] == 1 and abs(em["depth"][0] - 1.5) < 1e-5


def test_bary_matrix_is_inverse_of_vertex_matrix(oracle):
    s = S.random_soup(200, 64, 64, seed=2, sigma_px=10.0)
    v, idx = s["vertices"], s["indices"]
    m = oracle.bary(v.astype(np.float64), idx)
    P = v[idx].astype(np.float64)
    A = np.stack([P[:, :, 0], P[:, :, 1], np.ones((idx.shape[0], 3))], axis=1)  # columns = vertices
    np.testing.assert_allclose(m, np.linalg.inv(A), rtol=1e-9, atol=1e-9)
    m32 = oracle.bary(v, idx)
    scale = np.abs(m).max(axis=(1, 2), keepdims=True)
    assert (np.abs(m32 - m) <= 2e-4 * scale).all()
    # a degenerate triangle divides by 1 instead of 0 (render.cu:325-326)
    vd, idd = _tri_scene([[[0.1, 0.1], [0.1, 0.1], [0.3, 0.2]]])
    assert np.isfinite(oracle.bary(vd, idd)).all()


def test_scene_generators_are_deterministic_and_sized():
    a, b = S.config(0), S.config(0)
    for k in ("vertices", "indices", "colors", "opacities", "target"):
        np.testing.assert_array_equal(a[k], b[k])
    assert a["vertices"].shape == (3000, 4) and a["indices"].shape == (1000, 3) and a["target"].shape == (256, 256, 4)
    assert a["vertices"].dtype == np.float32 and a["indices"].dtype == np.int32
    np.testing.assert_allclose(a["vertices"][:, 3], 1 / a["vertices"][:, 2], rtol=1e-6)
    v, f = S.icosphere(3)
    assert v.shape == (10 * 4 ** 3 + 2, 3) and f.shape == (20 * 4 ** 3, 3)
    np.testing.assert_allclose(np.linalg.norm(v, axis=1), 1.0)
    assert len({tuple(sorted(e)) for t in f for e in ((t[0], t[1]), (t[1], t[2]), (t[2], t[0]))}) == 30 * 4 ** 3  # Euler
    g = S.grid_mesh(500, 500, -0.9, 0.9, -0.9, 0.9)
    assert g["vertices"].shape[0] == 249_750 and g["indices"].shape[0] == 497_503  # notebooks/renderer.ipynb:79 scene
    sq = S.overlapping_squares(10)
    assert sq["vertices"].shape == (40, 4) and sq["indices"].shape == (20, 3)
    assert S.unit_square()["vertices"][0, 2] == -1 and S.unit_square()["vertices"][0, 3] == -1
    assert np.isinf(S.overlap_mesh()["vertices"][:, 3]).all()
