"""The double-precision build (libtrigrad_hip_f64.so = the same kernel sources with
-DTG_DOUBLE_PRECISION, the reference's DOUBLE_PRECISION switch, util.h:5-20).

The reference's own tests are torch.autograd.gradcheck runs, which need float64:
tests/test_components.py (CPU component functions) and
tests/test_render_gradients.py (render on 50x50 images with 4x4 tiles on
overlapping_squares(10) and large_trianlges(3, r=4), image and depth outputs,
gradients to colours, opacities and vertices).  They are run here on this
library with the same scenes and arguments; the stages are also compared with
the CPU oracle's float64 instantiation.
"""
import numpy as np
import pytest
import torch
from torch.autograd import gradcheck

from helpers import to_device


@pytest.fixture
def double_precision():
    import trigrad_amd
    from trigrad_amd import _C
    before = _C.precision
    trigrad_amd.set_precision(torch.float64)
    yield torch.float64
    trigrad_amd.set_precision(before)


def _uniform(gen, shape, lo, hi):
    return torch.rand(shape, generator=gen, dtype=torch.float64) * (hi - lo) + lo


@pytest.mark.parametrize("seed", range(8))
def test_component_gradcheck(seed, double_precision):
    """tests/test_components.py of the reference: same value ranges, float64, CPU."""
    import trigrad_amd
    gen = torch.Generator().manual_seed(seed)
    bary = _uniform(gen, 3, 0, 1)
    bary = (bary / bary.sum()).requires_grad_()
    w = _uniform(gen, 3, 0, 5).requires_grad_()
    a, b, c = [_uniform(gen, 1, -5, 5).requires_grad_() for _ in range(3)]
    assert gradcheck(trigrad_amd.interpolate3_scalar, (bary, a, b, c, w))
    va, vb, vc = [_uniform(gen, 3, -5, 5).requires_grad_() for _ in range(3)]
    assert gradcheck(trigrad_amd.interpolate3_vector, (bary, va, vb, vc, w))
    p0, p1, q0, q1 = [_uniform(gen, 2, -5, 5).requires_grad_() for _ in range(4)]
    assert gradcheck(trigrad_amd.barycentric, (p0, p1, q0, q1))


def test_precision_is_checked(double_precision):
    """With the double build selected, float32 tensors are rejected like a reference built with DOUBLE_PRECISION."""
    import trigrad_amd
    with pytest.raises(TypeError, match="must be of type torch.float64"):
        trigrad_amd.barycentric(*[torch.zeros(2, dtype=torch.float32) for _ in range(4)])
    with pytest.raises(TypeError):
        trigrad_amd.set_precision(torch.float16)


def _as_double(scene):
    out = dict(scene)
    for k in ("vertices", "colors", "opacities"):
        out[k] = scene[k].astype(np.float64)
    return out


DOUBLE_SCENES = {
    "soup_varying_w": lambda S: (S.random_soup(1500, 160, 120, seed=1, sigma_px=9.0, varying_w=True), 16, 16),
    "soup_shared_tile8x4": lambda S: (S.random_soup(800, 100, 90, seed=2, shared=True, sigma_px=7.0), 8, 4),
    "squares": lambda S: (S.overlapping_squares(10), 4, 4),
    "large_triangles": lambda S: (S.large_triangles(3, r=4), 4, 4),
    "depth_overlap": lambda S: (S.depth_overlap(), 16, 16),
}
DOUBLE_MODES = {"A": dict(per_pixel_sort=True, max_layers=32), "A_3": dict(per_pixel_sort=True, max_layers=3),
                "A_40": dict(per_pixel_sort=True, max_layers=40), "B": dict(per_pixel_sort=False, max_layers=-1)}


@pytest.mark.gpu
@pytest.mark.parametrize("mode", sorted(DOUBLE_MODES))
@pytest.mark.parametrize("name", sorted(DOUBLE_SCENES))
def test_double_build_matches_oracle(name, mode, cuda, oracle):
    """Lists and bary matrices bit-exact, image bit-identical, gradients to 1e-9 against the oracle's float64 instantiation."""
    from trigrad_amd import _C
    import scenes as S
    scene, tw, th = DOUBLE_SCENES[name](S)
    scene = _as_double(scene)
    m = DOUBLE_MODES[mode]
    W, H = scene["width"], scene["height"]
    M = scene["indices"].shape[0]
    ml = m["max_layers"] if m["max_layers"] > 0 else M + 1
    d = to_device(scene, cuda)
    assert d["vertices"].dtype == torch.float64
    want = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, tw, th, 1 / 256,
                         m["per_pixel_sort"], ml)
    got = _C._forward_full(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, tw, th, 1 / 256, True,
                            m["per_pixel_sort"], ml)
    image, depthmap, weights, sorted_ids, offsets, bary, ends, _, resume = got
    assert image.dtype == torch.float64 and resume[2].verify() is None
    np.testing.assert_array_equal(offsets.cpu().numpy(), want["offsets"])
    np.testing.assert_array_equal(sorted_ids.cpu().numpy(), want["sorted_ids"])
    np.testing.assert_array_equal(bary.cpu().numpy().view(np.uint64), oracle.bary(scene["vertices"], scene["indices"]).view(np.uint64))
    np.testing.assert_array_equal(image.cpu().numpy().view(np.uint64), want["image"].view(np.uint64))
    np.testing.assert_array_equal(ends.cpu().numpy(), want["ends"])
    dm, wd = depthmap.cpu().numpy(), want["depthmap"]
    assert np.array_equal(np.isfinite(dm), np.isfinite(wd))
    np.testing.assert_allclose(np.where(np.isfinite(wd), dm, 0), np.where(np.isfinite(wd), wd, 0), rtol=1e-14, atol=0)

    rng = np.random.default_rng(3)
    gi, gd = rng.standard_normal((H, W, 4)), rng.standard_normal((H, W))
    gV, gC, gO = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], want,
                                        W, H, tw, th, m["per_pixel_sort"], ml, literal=False)
    routes = [resume] + ([resume[:3] + (None, None)] if resume[3] is not None or resume[4] is not None else [])
    for res in routes:
        out = _C.render_backward(torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda), d["vertices"], d["indices"],
                                 d["colors"], d["opacities"], sorted_ids, offsets, bary, image, depthmap, weights, ends, W, H,
                                 tw, th, 1 / 256, m["per_pixel_sort"], ml, resume=res)
        for label, g, w in zip(("grad_vertices", "grad_colors", "grad_opacities"), out, (gV, gC, gO)):
            scale = float(np.abs(w).max()) if w.size else 0.0
            np.testing.assert_allclose(g.cpu().numpy(), w, rtol=1e-9, atol=1e-12 + 1e-12 * scale, err_msg=f"{name}/{mode}: {label}")


def _reference_case(S, which, cuda):
    """Scenes and arguments of the reference's tests/test_render_gradients.py (opacity 0.99 everywhere)."""
    scene = S.overlapping_squares(10) if which == "squares" else S.large_triangles(3, r=4)
    v = torch.from_numpy(scene["vertices"].astype(np.float64)).to(cuda)
    i = torch.from_numpy(scene["indices"]).to(cuda)
    c = torch.from_numpy(scene["colors"].astype(np.float64)).to(cuda)
    o = torch.full_like(v[:, 0], 0.99)
    return v, i, c, o


# (scene, output index, which inputs take gradients): the eight tests of tests/test_render_gradients.py
REFERENCE_GRADCHECKS = [
    ("squares", 0, "c"), ("triangles", 1, "c"), ("squares", 0, "o"), ("triangles", 1, "o"),
    ("triangles", 0, "v"), ("triangles", 1, "v"), ("triangles", 0, "vco"), ("triangles", 1, "vco"),
]


@pytest.mark.gpu
@pytest.mark.parametrize("per_pixel_sort", [True, False])
@pytest.mark.parametrize("scene,output,wrt", REFERENCE_GRADCHECKS)
def test_reference_gradcheck_suite(scene, output, wrt, per_pixel_sort, cuda, double_precision):
    """gradcheck(render) with the reference's scenes, sizes (50x50, 4x4 tiles) and threshold; the reference runs
    the default mode only, the tile-order mode is added."""
    import trigrad_amd
    import scenes as S
    v, i, c, o = _reference_case(S, scene, cuda)
    if "v" in wrt:
        v.requires_grad_()
    if "c" in wrt:
        c.requires_grad_()
    if "o" in wrt:
        o.requires_grad_()
    extra = () if per_pixel_sort else (False, False, -1)  # record_timing, per_pixel_sort, max_layers
    assert gradcheck(lambda *args: trigrad_amd.render(*args)[output], (v, i, c, o, 50, 50, 4, 4, 1 / 256) + extra)
