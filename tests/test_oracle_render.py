"""Pins the forward blend and the backward pass of the CPU oracle (no GPU):

  * against an independent float64 dense-tensor renderer (tests/independent_renderer.py)
    whose gradients come from torch autograd;
  * against closed forms (n constant layers, the early-stop layer count of
    reference notebooks/renderer.ipynb:492, a single opaque triangle);
  * against central finite differences of the oracle's own float64 forward --
    the method of the reference's test-suite (tests/test_render_gradients.py,
    torch.autograd.gradcheck on the reference's fixture scenes);
  * component formulas as in reference tests/test_components.py.

It also measures how far the reference's literal backward traversal is from
the derivative in the two regimes where the declared policy departs from it.
"""
import math

import numpy as np
import pytest
import torch

import independent_renderer as IR
import scenes as S

D = np.float64


def _f64(scene):
    return (scene["vertices"].astype(D), scene["indices"], scene["colors"].astype(D), scene["opacities"].astype(D))


def _oracle_grads(oracle, scene64, W, H, tw, th, gi, gd, **mode):
    v, idx, c, o = scene64
    fwd = oracle.render(v, idx, c, o, W, H, tw, th, 1 / 256, mode.get("per_pixel_sort", True), mode.get("max_layers", 32))
    return fwd, oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, tw, th, mode.get("per_pixel_sort", True),
                                       mode.get("max_layers", 32), literal=mode.get("literal", False))


def _autograd(scene64, W, H, gi, gd, **kw):
    v, idx, c, o = (torch.from_numpy(np.ascontiguousarray(a)) for a in scene64)
    v.requires_grad_(); c.requires_grad_(); o.requires_grad_()
    image, depth = IR.render(v, idx, c, o, W, H, **kw)
    fin = torch.isfinite(depth)
    loss = (image * torch.from_numpy(gi)).sum() + (torch.where(fin, depth, torch.zeros_like(depth)) * torch.from_numpy(gd)).sum()
    loss.backward()
    return image.detach().numpy(), depth.detach().numpy(), v.grad.numpy(), c.grad.numpy(), o.grad.numpy()


SOUPS = {
    "equal_w": dict(M=60, W=40, H=32, seed=1, sigma_px=9.0, varying_w=False),
    "varying_w": dict(M=60, W=40, H=32, seed=2, sigma_px=9.0, varying_w=True),
    "shared": dict(M=40, W=32, H=32, seed=3, sigma_px=9.0, shared=True),
}


@pytest.mark.parametrize("name", sorted(SOUPS))
@pytest.mark.parametrize("tile", [(16, 16), (4, 4)])
def test_forward_matches_independent_renderer_per_pixel_order(name, tile, oracle):
    kw = dict(SOUPS[name]); M, W, H = kw.pop("M"), kw.pop("W"), kw.pop("H")
    scene = S.random_soup(M, W, H, **kw)
    s64 = _f64(scene)
    fwd = oracle.render(*s64, W, H, *tile, 1 / 256, True, 1000)
    image, depth = IR.render(*(torch.from_numpy(np.ascontiguousarray(a)) for a in s64), W, H)
    np.testing.assert_allclose(fwd["image"], image.numpy(), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(fwd["depthmap"], depth.numpy(), rtol=1e-9, atol=1e-11)
    assert fwd["ends"].max() > 3  # the scene does stack fragments
    # float32 instantiation agrees at float32 accuracy wherever no fragment sits on an edge
    f32 = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, *tile, 1 / 256, True, 1000)
    same = f32["ends"] == fwd["ends"]
    assert same.mean() > 0.99
    assert np.abs(f32["image"] - fwd["image"])[same].max() < 5e-5


@pytest.mark.parametrize("max_layers,thr", [(1000, 1 / 256), (3, 1 / 256), (1000, 0.3)])
def test_forward_matches_independent_renderer_tile_order(max_layers, thr, oracle):
    W, H, tw, th = 40, 32, 16, 16
    scene = S.random_soup(60, W, H, seed=4, sigma_px=9.0, varying_w=True)
    s64 = _f64(scene)
    fwd = oracle.render(*s64, W, H, tw, th, thr, False, max_layers)
    rank = IR.tile_order_rank(fwd["sorted_ids"], fwd["offsets"], 60, W, H, tw, th)
    image, depth = IR.render(*(torch.from_numpy(np.ascontiguousarray(a)) for a in s64), W, H, order_rank=rank,
                             max_layers=max_layers, threshold=thr)
    np.testing.assert_allclose(fwd["image"], image.numpy(), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(fwd["depthmap"], depth.numpy(), rtol=1e-9, atol=1e-11)
    if max_layers == 3:
        assert fwd["ends"].max() == 3
    if thr == 0.3:
        assert (fwd["image"][..., 3][fwd["ends"] > 0] > 0).all()


def _full_screen_layers(n, opacity, color, depths=None):
    """n triangles that each cover the whole screen, constant attributes."""
    xy = np.array([[-3.0, -3.0], [3.0, -3.0], [0.0, 3.0]])
    v = []
    for k in range(n):
        z = (k + 1.0) if depths is None else depths[k]
        v += [[x, y, z, 1 / z] for x, y in xy]
    v = np.array(v, dtype=np.float32)
    idx = np.arange(3 * n, dtype=np.int32).reshape(n, 3)
    c = np.tile(np.asarray(color, np.float32), (3 * n, 1))
    o = np.full(3 * n, opacity, np.float32)
    return v, idx, c, o


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_closed_form_constant_layers(dtype, oracle):
    """n full-coverage layers of opacity o and colour c: T = (1-o)^n, C = c (1 - (1-o)^n)."""
    n, o, col = 7, 0.3, (0.2, 0.5, 0.9)
    v, idx, c, op = (a.astype(dtype) if a.dtype.kind == "f" else a for a in _full_screen_layers(n, o, col))
    for pps in (True, False):
        out = oracle.render(v, idx, c, op, 24, 24, 16, 16, 1e-9, pps, 1000)
        o = D(op[0])  # the value actually stored (0.3 rounded to float32)
        colr = c[0].astype(D)
        T = (1 - o) ** n
        tol = 1e-5 if dtype == np.float32 else 1e-12
        np.testing.assert_allclose(out["image"][..., 3], T, rtol=tol)
        np.testing.assert_allclose(out["image"][..., :3], np.broadcast_to(colr * (1 - T), (24, 24, 3)), rtol=tol * 10)
        assert (out["ends"] == n).all()
        # depth = sum T_k o z_k / sum T_k o, z_k = k+1 (w = 1/z => view depth z)
        wk = np.array([(1 - o) ** k * o for k in range(n)])
        np.testing.assert_allclose(out["depthmap"], (wk / v[::3, 3].astype(D)).sum() / wk.sum(), rtol=tol * 10)


def test_early_stop_layer_count_tile_order(oracle):
    """per_pixel_sort off: compositing stops after ceil(ln thr / ln(1-o)) layers (notebooks/renderer.ipynb:492)."""
    o, thr = 0.5, 1 / 256
    v, idx, c, op = _full_screen_layers(20, o, (1, 1, 1))
    out = oracle.render(v, idx, c, op, 16, 16, 16, 16, thr, False, 1000)
    n_early = math.ceil(math.log(thr) / math.log(1 - o))
    assert n_early == 8 and (out["ends"] == n_early).all() and (out["last"] == n_early).all()
    np.testing.assert_allclose(out["image"][..., 3], (1 - o) ** n_early)
    # per_pixel_sort on: the threshold is only looked at between selections of 32 (render.cu:588)
    out = oracle.render(v, idx, c, op, 16, 16, 16, 16, thr, True, 1000)
    assert (out["ends"] == 20).all()
    v, idx, c, op = _full_screen_layers(40, o, (1, 1, 1))
    out = oracle.render(v, idx, c, op, 16, 16, 16, 16, thr, True, 1000)
    assert (out["ends"] == 32).all()
    out = oracle.render(v, idx, c, op, 16, 16, 16, 16, thr, True, 5)
    assert (out["ends"] == 5).all()


def test_single_triangle_is_perspective_correct_and_order_invariant(oracle):
    rng = np.random.default_rng(0)
    v = np.array([[-0.8, -0.7, 2.0, 0.5], [0.9, -0.6, 4.0, 0.25], [0.1, 0.8, 8.0, 0.125]], dtype=D)
    idx = np.array([[0, 1, 2]], np.int32)
    c = rng.uniform(0, 1, (3, 3)); o = np.ones(3)
    out = oracle.render(v, idx, c, o, 32, 32)
    iy, ix = 12, 17
    p = np.array([(ix + 0.5) / 32 * 2 - 1, (iy + 0.5) / 32 * 2 - 1, 1.0])
    b = np.linalg.solve(np.array([v[:, 0], v[:, 1], np.ones(3)]), p)
    assert (b > 0).all()
    want = (b * v[:, 3]) @ c / (b * v[:, 3]).sum() * 0.9999
    np.testing.assert_allclose(out["image"][iy, ix, :3], want, rtol=1e-12)
    np.testing.assert_allclose(out["depthmap"][iy, ix], (b / v[:, 3]).sum() / b.sum(), rtol=1e-12)
    # shuffling the triangle list does not change the image (notebook "Depth sorting test")
    scene = S.random_soup(80, 48, 40, seed=6, sigma_px=10.0, varying_w=True)
    s64 = _f64(scene)
    base = oracle.render(*s64, 48, 40, 16, 16, 1 / 256, True, 1000)["image"]
    perm = rng.permutation(80)
    shuffled = oracle.render(s64[0], s64[1][perm], s64[2], s64[3], 48, 40, 16, 16, 1 / 256, True, 1000)["image"]
    np.testing.assert_allclose(base, shuffled, rtol=1e-12, atol=1e-14)


@pytest.mark.parametrize("name", sorted(SOUPS))
def test_backward_matches_autograd_per_pixel_order(name, oracle):
    """Image gradients against autograd through the independent renderer.  The
    depth-map gradient is included only where the three w of every triangle are
    equal: otherwise the reference adds the gradient of the depth interpolation's
    unit weights to the w gradient (render.cu:520-521, :530), which is not part of
    the derivative and is checked separately below."""
    kw = dict(SOUPS[name]); M, W, H = kw.pop("M"), kw.pop("W"), kw.pop("H")
    scene = S.random_soup(M, W, H, **kw)
    s64 = _f64(scene)
    rng = np.random.default_rng(0)
    gi = rng.standard_normal((H, W, 4))
    gd = rng.standard_normal((H, W)) if name == "equal_w" else np.zeros((H, W))
    fwd, (gV, gC, gO) = _oracle_grads(oracle, s64, W, H, 16, 16, gi, gd, per_pixel_sort=True, max_layers=1000)
    _, _, aV, aC, aO = _autograd(s64, W, H, gi, gd)
    np.testing.assert_allclose(gC, aC, rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(gO, aO, rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(gV[:, [0, 1, 3]], aV[:, [0, 1, 3]], rtol=1e-7, atol=1e-8)
    assert np.abs(gV[:, 2]).max() == 0.0  # z only orders fragments (render.cu:531-533)
    # at most 32 fragments were blended, so the literal traversal is the same computation
    assert fwd["ends"].max() <= 32
    lit = oracle.render_backward(gi, gd, *s64, fwd, W, H, 16, 16, True, 1000, literal=True)
    for a, b in zip(lit, (gV, gC, gO)):
        np.testing.assert_array_equal(a, b)


def test_backward_matches_autograd_tile_order(oracle):
    W, H, tw, th = 40, 32, 16, 16
    scene = S.random_soup(60, W, H, seed=4, sigma_px=9.0, varying_w=True)
    s64 = _f64(scene)
    rng = np.random.default_rng(1)
    gi = rng.standard_normal((H, W, 4)); gd = np.zeros((H, W))
    for max_layers, thr in ((1000, 1 / 256), (3, 1 / 256)):
        v, idx, c, o = s64
        fwd = oracle.render(v, idx, c, o, W, H, tw, th, thr, False, max_layers)
        gV, gC, gO = oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, tw, th, False, max_layers)
        rank = IR.tile_order_rank(fwd["sorted_ids"], fwd["offsets"], 60, W, H, tw, th)
        _, _, aV, aC, aO = _autograd(s64, W, H, gi, gd, order_rank=rank, max_layers=max_layers, threshold=thr)
        np.testing.assert_allclose(gC, aC, rtol=1e-8, atol=1e-10)
        np.testing.assert_allclose(gO, aO, rtol=1e-8, atol=1e-10)
        np.testing.assert_allclose(gV[:, [0, 1, 3]], aV[:, [0, 1, 3]], rtol=1e-7, atol=1e-8)
        # the reference's literal traversal (forward order over `ends` list slots,
        # render.cu:659-666) is NOT this derivative
        lV, lC, lO = oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, tw, th, False, max_layers, literal=True)
        assert np.abs(lC - aC).max() > 1e-3


def test_unit_weight_term_of_the_depth_gradient(oracle):
    """With unequal w and a depth-map gradient, the oracle's w gradient equals
    autograd's plus the gradient w.r.t. the unit weights of the 1/w
    interpolation -- the term the reference adds at render.cu:530.  Recomputed
    here by autograd with explicit weight variables."""
    W, H = 24, 24
    v = np.array([[-0.8, -0.7, 2.0, 0.5], [0.9, -0.6, 4.0, 0.25], [0.1, 0.8, 8.0, 0.125]], dtype=D)
    idx = np.array([[0, 1, 2]], np.int32)
    c = np.full((3, 3), 0.5); o = np.full(3, 0.6)
    gi = np.zeros((H, W, 4)); gd = np.random.default_rng(2).standard_normal((H, W))
    fwd, (gV, gC, gO) = _oracle_grads(oracle, (v, idx, c, o), W, H, 16, 16, gi, gd)
    _, _, aV, _, _ = _autograd((v, idx, c, o), W, H, gi, gd)
    tv = torch.from_numpy(v)
    u = torch.ones(3, dtype=torch.float64, requires_grad=True)
    _, bary, inside = IR.fragments(tv, torch.from_numpy(idx), W, H)
    b = bary[:, :, 0, :]
    depth = ((b * u) / tv[:, 3]).sum(-1) / (b * u).sum(-1)   # single fragment: depth map = its view depth
    (torch.where(inside[:, :, 0], depth, torch.zeros_like(depth)) * torch.from_numpy(gd)).sum().backward()
    np.testing.assert_allclose(gV[:, 3], aV[:, 3] + u.grad.numpy(), rtol=1e-8, atol=1e-10)
    assert np.abs(u.grad.numpy()).max() > 1e-3
    np.testing.assert_allclose(gV[:, :2], aV[:, :2], rtol=1e-7, atol=1e-9)


def _finite_difference(fn, x, eps=1e-6):
    g = np.zeros_like(x)
    flat = x.reshape(-1)
    for i in range(flat.size):
        old = flat[i]
        flat[i] = old + eps; hi = fn()
        flat[i] = old - eps; lo = fn()
        flat[i] = old
        g.reshape(-1)[i] = (hi - lo) / (2 * eps)
    return g


@pytest.mark.parametrize("scene_name,output", [("squares", 0), ("large_triangles", 0), ("large_triangles", 1)])
def test_reference_gradcheck_scenes_by_finite_differences(scene_name, output, oracle):
    """The reference's own tests: 50x50 image, 4x4 tiles, threshold 1/256,
    defaults (per_pixel_sort, 32 layers), opacity 0.99, scenes
    overlapping_squares(10) and large_trianlges(3, r=4), image ([0]) and
    depth map ([1]) outputs (tests/test_render_gradients.py:12-173)."""
    scene = S.overlapping_squares(10) if scene_name == "squares" else S.large_triangles(3, r=4)
    W = H = 50
    v, idx, c, o = _f64(scene)
    rng = np.random.default_rng(7)
    gi = rng.standard_normal((H, W, 4)) if output == 0 else np.zeros((H, W, 4))
    gd = rng.standard_normal((H, W)) if output == 1 else np.zeros((H, W))

    def loss():
        f = oracle.render(v, idx, c, o, W, H, 4, 4, 1 / 256, True, 32)
        fin = np.isfinite(f["depthmap"])
        return (f["image"] * gi).sum() + (np.where(fin, f["depthmap"], 0) * gd).sum()

    fwd = oracle.render(v, idx, c, o, W, H, 4, 4, 1 / 256, True, 32)
    gV, gC, gO = oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, 4, 4, True, 32, literal=True)
    np.testing.assert_allclose(gC, _finite_difference(loss, c), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gO, _finite_difference(loss, o), rtol=1e-5, atol=1e-6)
    if scene_name == "large_triangles":  # every edge is off screen: the image is smooth in the vertices
        fd = _finite_difference(loss, v)
        np.testing.assert_allclose(gV[:, :2], fd[:, :2], rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(gV[:, 3], fd[:, 3], rtol=1e-5, atol=1e-6)  # equal w per triangle: no unit-weight term


def test_literal_traversal_beyond_32_layers_is_not_the_derivative(oracle):
    """per_pixel_sort on, 40 blended layers: the reference walks the batches front
    to back (render.cu:673-693); finite differences side with the reverse order."""
    v, idx, c, o = (a.astype(D) if a.dtype.kind == "f" else a for a in _full_screen_layers(40, 0.1, (0.3, 0.6, 0.9)))
    c = np.random.default_rng(3).uniform(0, 1, c.shape)
    W = H = 4
    gi = np.ones((H, W, 4)); gd = np.zeros((H, W))
    fwd = oracle.render(v, idx, c, o, W, H, 4, 4, 1e-9, True, 1000)
    assert (fwd["ends"] == 40).all()
    loss = lambda: (oracle.render(v, idx, c, o, W, H, 4, 4, 1e-9, True, 1000)["image"] * gi).sum()
    fd = _finite_difference(loss, o)
    good = oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, 4, 4, True, 1000, literal=False)[2]
    bad = oracle.render_backward(gi, gd, v, idx, c, o, fwd, W, H, 4, 4, True, 1000, literal=True)[2]
    np.testing.assert_allclose(good, fd, rtol=1e-5, atol=1e-7)
    assert np.abs(bad - fd).max() > 1e-2


def test_component_formulas(oracle):
    """interpolate3 (scalar, vector) and barycentric with their hand-written
    backward formulas against autograd, as in reference tests/test_components.py."""
    rng = np.random.default_rng(11)
    for _ in range(50):
        bc = rng.uniform(0, 1, 3); bc /= bc.sum()
        a, b, c = rng.uniform(-5, 5, 3)
        w = rng.uniform(0.1, 5, 3)
        tb, tw = torch.tensor(bc, requires_grad=True), torch.tensor(w, requires_grad=True)
        tv = torch.tensor([a, b, c], requires_grad=True)
        val = (tb * tw * tv).sum() / (tb * tw).sum()
        val.backward()
        assert abs(oracle.interpolate3_scalar(bc, a, b, c, w) - val.item()) < 1e-12
        gb, gv, gw = oracle.interpolate3_scalar_backward(1.0, bc, a, b, c, w)
        np.testing.assert_allclose(gb, tb.grad.numpy(), rtol=1e-9, atol=1e-12)
        np.testing.assert_allclose(gv, tv.grad.numpy(), rtol=1e-9, atol=1e-12)
        np.testing.assert_allclose(gw, tw.grad.numpy(), rtol=1e-9, atol=1e-12)

        A, B, C3 = rng.uniform(-5, 5, (3, 3))
        g = rng.standard_normal(3)
        tb, tw = torch.tensor(bc, requires_grad=True), torch.tensor(w, requires_grad=True)
        tA, tB, tC = (torch.tensor(x, requires_grad=True) for x in (A, B, C3))
        vec = (tb[0] * tw[0] * tA + tb[1] * tw[1] * tB + tb[2] * tw[2] * tC) / (tb * tw).sum()
        (vec * torch.tensor(g)).sum().backward()
        np.testing.assert_allclose(oracle.interpolate3_vector(bc, A, B, C3, w), vec.detach().numpy(), rtol=1e-12)
        gb, ga, gbv, gc, gw = oracle.interpolate3_vector_backward(g, bc, A, B, C3, w)
        for got, want in ((gb, tb.grad), (ga, tA.grad), (gbv, tB.grad), (gc, tC.grad), (gw, tw.grad)):
            np.testing.assert_allclose(got, want.numpy(), rtol=1e-9, atol=1e-12)

        pts = [torch.tensor(rng.uniform(-5, 5, 2), requires_grad=True) for _ in range(4)]
        p0, p1, p2, q = pts

        def area(u, v_, x):
            return (v_[0] - u[0]) * (x[1] - u[1]) - (v_[1] - u[1]) * (x[0] - u[0])
        lam = torch.stack([area(p1, p2, q), area(p2, p0, q), area(p0, p1, q)]) / area(p0, p1, p2)
        (lam * torch.tensor(g)).sum().backward()
        got = oracle.barycentric(*[p.detach().numpy() for p in pts])
        np.testing.assert_allclose(got, lam.detach().numpy(), rtol=1e-9, atol=1e-12)
        assert abs(got.sum() - 1) < 1e-9
        jac = oracle.barycentric_backward(g, *[p.detach().numpy() for p in pts])
        np.testing.assert_allclose(jac, np.stack([p.grad.numpy() for p in pts]), rtol=1e-8, atol=1e-10)
