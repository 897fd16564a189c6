"""GPU parity of the forward blend and the backward pass against the CPU oracle.

Bars (the ones the task states): image within 1e-5 absolute; gradients within
1e-4 relative + 1e-6 absolute.  The forward kernels evaluate the oracle's
float32 expression tree operation for operation, so the image is in fact
expected to be bit-identical; the number of differing values is reported and
bounded.  The oracle accumulates gradients in float64, the GPU sums float32
terms with atomics in arbitrary order, hence the gradient tolerance.

Everything here calls the C ABI of libtrigrad_hip.so through trigrad_amd.
"""
import numpy as np
import pytest

from helpers import GRAD_ATOL, GRAD_RTOL, assert_gradients_close, assert_close, to_device, u64
from test_gpu_stages import SCENES

pytestmark = pytest.mark.gpu

IMAGE_ATOL = 1e-5

MODES = {
    "A_default": dict(per_pixel_sort=True, max_layers=32),
    "A_unlimited": dict(per_pixel_sort=True, max_layers=-1),
    "A_5_layers": dict(per_pixel_sort=True, max_layers=5),
    "A_40_layers": dict(per_pixel_sort=True, max_layers=40),
    "B_unlimited": dict(per_pixel_sort=False, max_layers=-1),
    "B_3_layers": dict(per_pixel_sort=False, max_layers=3),
}


def _nan_equal(a, b):
    return np.array_equal(a, b, equal_nan=True)


def _forward_both(scene, tw, th, mode, cuda, oracle, thr=1 / 256):
    from trigrad_amd import _C
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    M = scene["indices"].shape[0]
    ml = mode["max_layers"] if mode["max_layers"] > 0 else M + 1
    want = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, tw, th, thr,
                         mode["per_pixel_sort"], ml)
    got = _C._forward_full(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, tw, th, thr, True,
                            mode["per_pixel_sort"], ml)
    return d, want, got, ml


def _check_forward(name, want, got, tile_shape):
    from trigrad_amd import _C
    image, depthmap, weights, sorted_ids, offsets, bary, ends, timings, (last, last_depth, status, fragments, hit_masks) = got
    status.verify()
    np.testing.assert_array_equal(offsets.cpu().numpy(), want["offsets"])
    np.testing.assert_array_equal(sorted_ids.cpu().numpy(), want["sorted_ids"])
    img = image.cpu().numpy()
    finite = np.isfinite(want["image"])
    assert _nan_equal(np.isnan(img), np.isnan(want["image"])), f"{name}: NaN pattern differs"
    assert_close(f"{name}: image", np.where(finite, img, 0), np.where(finite, want["image"], 0), 0.0, IMAGE_ATOL)
    dm = depthmap.cpu().numpy()
    fin = np.isfinite(want["depthmap"])
    assert _nan_equal(np.isfinite(dm), fin)
    assert_close(f"{name}: depthmap", np.where(fin, dm, 0), np.where(fin, want["depthmap"], 0), 1e-5, 1e-5)
    np.testing.assert_array_equal(ends.cpu().numpy(), want["ends"])
    np.testing.assert_array_equal(last.cpu().numpy(), want["last"])
    if fragments is not None:
        # saved blend order: `ends` valid layers per pixel, no list position twice, and the last
        # layer is the entry `last` points at (the backward parity tests check the content)
        tile_h, tile_w = tile_shape
        fr = _C.saved_blend_order(fragments, offsets, tile_w, tile_h).cpu().numpy()
        en, la = want["ends"], want["last"]
        layer = np.arange(fr.shape[0])[:, None, None]
        valid = layer < en[None]
        assert (fr[valid] >= 0).all()
        ys, xs = np.nonzero(en > 0)
        np.testing.assert_array_equal(fr[en[ys, xs] - 1, ys, xs], la[ys, xs] - 1)
        srt = np.sort(np.where(valid, fr, -1 - layer), axis=0)
        assert (np.diff(srt, axis=0) != 0).all()
    # (NaN results carry different payload/sign bits on the two machines)
    differing = int(((img.view(np.uint32) != want["image"].view(np.uint32)) & ~np.isnan(img)).sum())
    assert differing == 0, f"{name}: {differing} image values are not bit-identical to the oracle"
    assert _nan_equal(weights.cpu().numpy(), want["weights"])


@pytest.mark.parametrize("mode", sorted(MODES))
@pytest.mark.parametrize("name", sorted(SCENES))
def test_forward_matches_oracle(name, mode, cuda, oracle):
    scene, tw, th = SCENES[name]()
    _, want, got, _ = _forward_both(scene, tw, th, MODES[mode], cuda, oracle)
    _check_forward(f"{name}/{mode}", want, got, (th, tw))


def _long_list_scene():
    """One 16x16 tile whose list is longer than 65535 entries next to tiles with short lists: the per-pixel-order
    forward pass keeps list positions in 16 bits where they fit and hands the other tiles to a second launch."""
    import scenes as S
    crowd = S.random_soup(70000, 32, 32, seed=3, sigma_px=1.5, opacity=(0.02, 0.2))
    v = crowd["vertices"].copy()
    v[:, :2] = v[:, :2] * 0.45 - 0.5  # into the first tile (with a fringe over its neighbours)
    rest = S.random_soup(1500, 32, 32, seed=4, sigma_px=5.0)
    vertices = np.concatenate([v, rest["vertices"]])
    indices = np.concatenate([crowd["indices"], rest["indices"] + v.shape[0]]).astype(np.int32)
    scene = dict(crowd)
    scene.update(vertices=vertices, indices=indices, colors=np.concatenate([crowd["colors"], rest["colors"]]),
                 opacities=np.concatenate([crowd["opacities"], rest["opacities"]]))
    return scene


@pytest.mark.parametrize("mode,tile", [("A_default", 16), ("A_40_layers", 16), ("B_3_layers", 16), ("A_default", 32)])
def test_tile_list_longer_than_16_bit_positions(mode, tile, cuda, oracle):
    import torch
    from trigrad_amd import _C
    scene = _long_list_scene()
    m = MODES[mode]
    d, want, got, ml = _forward_both(scene, tile, tile, m, cuda, oracle)
    lengths = np.diff(want["offsets"])
    # 16x16: one long list next to short ones; 32x32: the one tile is four workgroups on the long list
    assert lengths.max() > 65535 and (tile == 32 or lengths.min() < 65535)
    _check_forward(f"long list/{mode}", want, got, (tile, tile))
    gi, gd = _grad_inputs(scene, 9, True)
    wanted = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], want,
                                    32, 32, tile, tile, m["per_pixel_sort"], ml, literal=False, magnitudes=True)
    image, depthmap, weights, sorted_ids, offsets, bary, ends, _, resume = got
    out = _C.render_backward(torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda), d["vertices"], d["indices"],
                             d["colors"], d["opacities"], sorted_ids, offsets, bary, image, depthmap, weights, ends, 32, 32,
                             tile, tile, 1 / 256, m["per_pixel_sort"], ml, resume=resume)
    for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), out, wanted[:3], wanted[3:]):
        assert_gradients_close(f"long list/{mode}: {label}", g.cpu().numpy(), w, mag)


def _grad_inputs(scene, seed, with_depth):
    rng = np.random.default_rng(seed)
    H, W = scene["height"], scene["width"]
    gi = rng.standard_normal((H, W, 4)).astype(np.float32)
    gd = rng.standard_normal((H, W)).astype(np.float32) if with_depth else np.zeros((H, W), np.float32)
    return gi, gd


BACKWARD_SCENES = ["config0", "soup_varying_w", "soup_shared", "soup_big_tris", "soup_tile4", "soup_tile32", "soup_tile_8x4",
                   "squares", "large_triangles", "depth_overlap", "overlapping_triangles", "unit_square_negative_z", "overlap_mesh_inf_w",
                   "grid_mesh", "degenerate", "center_island", "soup_tile8", "soup_tile_24x16"]


@pytest.mark.parametrize("with_depth", [False, True])
@pytest.mark.parametrize("mode", sorted(MODES))
@pytest.mark.parametrize("name", BACKWARD_SCENES)
def test_backward_matches_oracle(name, mode, with_depth, cuda, oracle):
    import torch
    from trigrad_amd import _C
    scene, tw, th = SCENES[name]()
    m = MODES[mode]
    d, want, got, ml = _forward_both(scene, tw, th, m, cuda, oracle)
    W, H = scene["width"], scene["height"]
    gi, gd = _grad_inputs(scene, 5, with_depth)
    wanted = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], want,
                                    W, H, tw, th, m["per_pixel_sort"], ml, literal=False, magnitudes=True)
    image, depthmap, weights, sorted_ids, offsets, bary, ends, _, resume = got
    # the blend order is saved exactly when per-pixel order meets max_layers <= 32;
    # then the route that selects the fragments again is checked as well
    saved_order = resume[3] is not None
    assert saved_order == (bool(m["per_pixel_sort"]) and ml <= _C.MAX_SAVED_LAYERS)
    assert (resume[4] is not None) == (not m["per_pixel_sort"])  # tile order saves its hit masks
    routes = [("", resume)]
    if saved_order:
        routes.append((" (re-selected)", resume[:3] + (None, None)))
    if resume[4] is not None:
        routes.append((" (inside tests repeated)", resume[:4] + (None,)))
    for route, res in routes:
        out = _C.render_backward(torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda), d["vertices"], d["indices"],
                                 d["colors"], d["opacities"], sorted_ids, offsets, bary, image, depthmap, weights, ends, W, H,
                                 tw, th, 1 / 256, m["per_pixel_sort"], ml, resume=res)
        for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), out, wanted[:3], wanted[3:]):
            assert_gradients_close(f"{name}/{mode}{route}: {label}", g.cpu().numpy(), w, mag)  # NaN where the oracle has NaN
        assert float(out[0][:, 2].abs().max()) == 0.0  # z never receives a gradient (render.cu:531-533)
    if name == "soup_shared" and with_depth:
        # the three layouts of the gradient arrays the kernels know: dense, one (V,8) block, run-time strides
        for strides in ((4, 3, 1), (8, 8, 8), (6, 5, 2)):
            alt = _C.render_backward(torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda), d["vertices"], d["indices"],
                                     d["colors"], d["opacities"], sorted_ids, offsets, bary, image, depthmap, weights, ends, W,
                                     H, tw, th, 1 / 256, m["per_pixel_sort"], ml, resume=resume, grad_strides=strides)
            for a, b in zip(alt, out):
                assert a.is_contiguous() and a.shape == b.shape
                assert float((a - b).abs().max()) <= 1e-5 * float(b.abs().max()) + 1e-6


def test_default_mode_literal_and_policy_agree(oracle):
    """With per_pixel_sort on and at most 32 blended fragments the literal
    reference traversal and the reverse-order policy are the same computation."""
    import scenes as S
    scene = S.random_soup(300, 64, 64, seed=9, sigma_px=14.0, varying_w=True)
    W = H = 64
    fwd = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H)
    gi, gd = _grad_inputs(scene, 1, True)
    a = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], fwd, W, H, literal=True)
    b = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], fwd, W, H, literal=False)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)


def test_render_autograd_end_to_end(cuda, oracle):
    """trigrad_amd.render + loss.backward() on configuration 0 (both modes)."""
    import torch
    import trigrad_amd
    import scenes as S
    scene = S.config(0)
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    for kw in (dict(), dict(per_pixel_sort=False, max_layers=-1)):
        v = d["vertices"].clone().requires_grad_()
        c = d["colors"].clone().requires_grad_()
        o = d["opacities"].clone().requires_grad_()
        image, depthmap = trigrad_amd.render(v, d["indices"], c, o, W, H, **kw)
        loss = ((image - d["target"]) ** 2).sum()
        loss.backward()
        pps = kw.get("per_pixel_sort", True)
        ml = kw.get("max_layers", 32)
        fwd = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, per_pixel_sort=pps,
                            max_layers=ml)
        assert_close("image", image.detach().cpu().numpy(), fwd["image"], 0.0, IMAGE_ATOL)
        gi = 2.0 * (fwd["image"] - scene["target"])
        wanted = oracle.render_backward(gi, np.zeros((H, W), np.float32), scene["vertices"], scene["indices"], scene["colors"],
                                        scene["opacities"], fwd, W, H, per_pixel_sort=pps, max_layers=ml, magnitudes=True)
        for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), (v.grad, c.grad, o.grad), wanted[:3], wanted[3:]):
            assert_gradients_close(label, g.cpu().numpy(), w, mag)


def test_loss_on_depth_only(cuda, oracle):
    """Only the depth map takes part in the loss: the image's gradient arrives as None."""
    import torch
    import trigrad_amd
    import scenes as S
    scene = S.random_soup(400, 96, 80, seed=21, sigma_px=9.0, varying_w=True)
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    v = d["vertices"].clone().requires_grad_()
    c = d["colors"].clone().requires_grad_()
    o = d["opacities"].clone().requires_grad_()
    image, depthmap = trigrad_amd.render(v, d["indices"], c, o, W, H)
    hit = torch.isfinite(depthmap)
    weight = torch.linspace(0.5, 1.5, W * H, device=cuda).reshape(H, W)
    (torch.where(hit, depthmap, torch.zeros_like(depthmap)) * weight).sum().backward()
    fwd = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H)
    gd = np.where(np.isfinite(fwd["depthmap"]), weight.cpu().numpy(), 0.0).astype(np.float32)
    wanted = oracle.render_backward(np.zeros((H, W, 4), np.float32), gd, scene["vertices"], scene["indices"], scene["colors"],
                                    scene["opacities"], fwd, W, H, magnitudes=True)
    for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), (v.grad, c.grad, o.grad), wanted[:3], wanted[3:]):
        assert_gradients_close(label, g.cpu().numpy(), w, mag)
    assert float(v.grad.abs().max()) > 0


@pytest.mark.parametrize("mode", ["A_default", "B_unlimited"])
def test_repeatable_and_stream_ordered(mode, cuda):
    """Two calls give bit-identical images and lists (only the gradient sums depend on the order of atomics), and a
    call on a side stream, ordered after the inputs' producer, gives the same result as on the default stream."""
    import torch
    import trigrad_amd
    import scenes as S
    if mode not in MODES:
        pytest.skip("mode table changed")
    kw = dict(per_pixel_sort=MODES[mode]["per_pixel_sort"], max_layers=MODES[mode]["max_layers"])
    scene = S.random_soup(2500, 200, 160, seed=31, sigma_px=10.0, varying_w=True)
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)

    def run():
        v = d["vertices"].clone().requires_grad_()
        c = d["colors"].clone().requires_grad_()
        o = d["opacities"].clone().requires_grad_()
        image, depthmap = trigrad_amd.render(v, d["indices"], c, o, W, H, **kw)
        (image.square().sum() + torch.where(torch.isfinite(depthmap), depthmap, torch.zeros_like(depthmap)).sum()).backward()
        return image.detach(), depthmap.detach(), v.grad, c.grad, o.grad

    first = run()
    second = run()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        third = run()
    side.synchronize()
    for other in (second, third):
        assert torch.equal(first[0], other[0]) and torch.equal(first[1], other[1])
        for a, b in zip(first[2:], other[2:]):
            scale = float(a.abs().max())
            assert float((a - b).abs().max()) <= 1e-5 * scale + 1e-6


@pytest.mark.parametrize("mode", ["A_default", "A_5_layers", "A_40_layers", "A_unlimited"])
@pytest.mark.parametrize("name", ["soup_big_tris", "squares", "config0", "overlap_mesh_inf_w", "unit_square_negative_z"])
def test_selection_early_stop_changes_nothing(name, mode, cuda, monkeypatch):
    """With depth bounds of the lists the per-pixel selection may leave a list early; every output stays bit-identical."""
    import torch
    from trigrad_amd import _C
    scene, tw, th = SCENES[name]()
    m = MODES[mode]
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    ml = m["max_layers"] if m["max_layers"] > 0 else scene["indices"].shape[0] + 1
    outs = []
    for threshold in (1 << 30, 0):  # never / always
        monkeypatch.setattr(_C, "EARLY_STOP_MIN_AVG_LIST", threshold)
        outs.append(_C._forward_full(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, tw, th, 1 / 256, True, True, ml))
    for a, b in zip(outs[0][:7], outs[1][:7]):
        assert torch.equal(a.view(torch.int32) if a.is_floating_point() else a, b.view(torch.int32) if b.is_floating_point() else b)
    ra, rb = outs[0][8], outs[1][8]
    assert torch.equal(ra[0], rb[0]) and torch.equal(ra[1].view(torch.int32), rb[1].view(torch.int32))
    if ra[3] is not None:
        layer = torch.arange(ra[3].shape[0], device=cuda)[:, None, None]
        valid = layer < outs[0][6][None]
        assert torch.equal(torch.where(valid, ra[3], 0), torch.where(valid, rb[3], 0))


def test_list_bounds_values(cuda):
    """tg_list_bounds: per tile and 256 entries, min over the rest of the list of (min z - 32 ulp max|z|); -inf where a
    weight is not positive and finite."""
    import torch
    from trigrad_amd import _C, _lib
    import scenes as S
    scene = S.random_soup(3000, 64, 48, seed=13, sigma_px=30.0, varying_w=True)
    v = scene["vertices"].copy()
    v[5, 3] = -1.0          # a negative weight
    v[40, 3] = np.inf       # an infinite one
    scene = dict(scene, vertices=v)
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    ids, offsets, keys, status = _C.per_tile_lists(d["vertices"], d["indices"], W, H, 16, 16)
    T = _C.num_tiles(W, H, 16, 16)
    K = ids.numel()
    lib = _lib.load(32)
    bounds = torch.full((int(lib.tg_list_bound_words(K, T)),), float("nan"), dtype=torch.float32, device=cuda)
    far_start = torch.full((T,), -1, dtype=torch.int32, device=cuda)
    low = torch.empty((scene["indices"].shape[0],), dtype=torch.float32, device=cuda)
    _lib.check(lib.tg_list_bounds(_C._ptr(d["vertices"]), v.shape[0], _C._ptr(d["indices"]), scene["indices"].shape[0],
                                  _C._ptr(keys), _C._ptr(ids), _C._ptr(offsets), T, _C._ptr(low), _C._ptr(bounds),
                                  _C._ptr(far_start), _C._stream(ids)), "tg_list_bounds")
    got, far_got = bounds.cpu().numpy(), far_start.cpu().numpy()
    ids_h, off = ids.cpu().numpy(), offsets.cpu().numpy()
    far = (u64(keys) & np.uint64(0xFFFFFFFF)) == np.uint64(np.array([1e30], np.float32).view(np.uint32)[0] ^ 0x80000000)
    tri = v[scene["indices"][ids_h]]                       # (K,3,4)
    z, w = tri[:, :, 2], tri[:, :, 3]
    ok = ((w > 0) & np.isfinite(w) & np.isfinite(z)).all(axis=1)
    lb = np.where(ok, z.min(axis=1) - np.float32(32) * np.finfo(np.float32).eps * np.abs(z).max(axis=1), -np.inf).astype(np.float32)
    lb = np.where(far, np.float32(np.inf), lb)
    assert far.any() and not far.all()
    checked = 0
    for t in range(T):
        seg_far = far[off[t]:off[t + 1]]
        assert far_got[t] == (int(np.argmax(seg_far)) if seg_far.any() else off[t + 1] - off[t])
        for p in range(0, off[t + 1] - off[t], 256):
            want = lb[off[t] + p:off[t + 1]].min()
            assert got[off[t] // 256 + t + p // 256] == want
            checked += 1
    assert checked > T and (lb == -np.inf).any() and max(off[1:] - off[:-1]) > 256


def test_record_timing_and_empty_scene(cuda):
    import torch
    import trigrad_amd
    import scenes as S
    d = to_device(S.config(0), cuda)
    image, depthmap, timings = trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], 256, 256, record_timing=True)
    assert set(timings) == {"init", "per_tile_lists", "sorting", "bary_transforms", "rasterization"}
    assert all(t >= 0 for t in timings.values())
    v = d["vertices"].clone().requires_grad_()
    empty = torch.empty((0, 3), dtype=torch.int32, device=cuda)
    image, depthmap = trigrad_amd.render(v, empty, d["colors"], d["opacities"], 64, 48)
    assert image.shape == (48, 64, 4) and float(image[..., 3].min()) == 1.0 and float(image[..., :3].abs().max()) == 0.0
    assert torch.isinf(depthmap).all()
    image.sum().backward()
    assert float(v.grad.abs().max()) == 0.0
    image, depthmap, timings = trigrad_amd.render(v, empty, d["colors"], d["opacities"], 64, 48, record_timing=True)
    assert timings is None


def test_argument_errors(cuda):
    import torch
    import trigrad_amd
    import scenes as S
    d = to_device(S.config(0), cuda)
    v, i, c, o = d["vertices"], d["indices"], d["colors"], d["opacities"]
    with pytest.raises(ValueError, match="tile_width \\* tile_height must be <= 1024"):
        trigrad_amd.render(v, i, c, o, 64, 64, 64, 32)
    with pytest.raises(TypeError, match="vertices must be on cuda"):
        trigrad_amd.render(v.cpu(), i, c, o)
    with pytest.raises(TypeError, match="indices must be of type torch.int32"):
        trigrad_amd.render(v, i.long(), c, o)
    with pytest.raises(ValueError, match="colors must be of shape"):
        trigrad_amd.render(v, i, c[:-1], o)
    with pytest.raises(TypeError, match="opacities must be of type torch.float32"):
        trigrad_amd.render(v, i, c, o.double())


class _ReferenceShapedRenderer:
    """The call pattern of the reference's autograd Function (src/trigrad/wrapper.py:56-70, 87-98): twelve arguments
    into render_forward, eight results out, exactly eleven tensors saved, twenty arguments into render_backward."""

    @staticmethod
    def make(drop_private_state):
        import torch
        from trigrad_amd import _C

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, vertices, indices, colors, opacities, width, height, tw, th, thr, record_timing, pps, max_layers):
                ctx.args = (width, height, tw, th, thr, pps, max_layers)
                image, depthmap, final_weights, sorted_ids, offsets, bary_transforms, ends, timings = _C.render_forward(
                    vertices, indices, colors, opacities, width, height, tw, th, thr, not record_timing, pps, max_layers)
                if drop_private_state:
                    del ends._tg_resume
                ctx.save_for_backward(vertices, indices, colors, opacities, sorted_ids, offsets, bary_transforms, image, depthmap,
                                      final_weights, ends)
                return image, depthmap

            @staticmethod
            def backward(ctx, grad_image, grad_depthmap):
                saved = ctx.saved_tensors
                # which route render_backward takes: with the private state it walks what the forward pass saved,
                # without it the forward kernel runs once more
                Fn.resume_seen.append(getattr(saved[-1], "_tg_resume", None) is not None)
                gv, gc, go = _C.render_backward(grad_image, grad_depthmap, *saved, *ctx.args)
                return (gv, None, gc, go) + (None,) * 8

        Fn.resume_seen = []
        return Fn


@pytest.mark.parametrize("drop_private_state", [False, True])
@pytest.mark.parametrize("mode", ["A_default", "B_unlimited", "B_3_layers", "A_40_layers"])
def test_native_surface_as_the_reference_wrapper_calls_it(mode, drop_private_state, cuda, oracle):
    """_C.render_forward / _C.render_backward with the reference's argument lists and nothing else carried over:
    with the private state that travels on `ends`, and after a caller lost it (it is then computed again)."""
    import torch
    import scenes as S
    scene = S.random_soup(700, 150, 110, seed=21, sigma_px=11.0, varying_w=True)
    m = MODES[mode]
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    ml = m["max_layers"] if m["max_layers"] > 0 else scene["indices"].shape[0] + 1
    v = d["vertices"].clone().requires_grad_()
    c = d["colors"].clone().requires_grad_()
    o = d["opacities"].clone().requires_grad_()
    Fn = _ReferenceShapedRenderer.make(drop_private_state)
    image, depthmap = Fn.apply(v, d["indices"], c, o, W, H, 16, 16, 1 / 256, False, m["per_pixel_sort"], ml)
    rng = np.random.default_rng(5)
    gi = rng.standard_normal((H, W, 4)).astype(np.float32)
    gd = rng.standard_normal((H, W)).astype(np.float32)
    want = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, 16, 16, 1 / 256,
                         m["per_pixel_sort"], ml)
    assert int((image.detach().cpu().numpy().view(np.uint32) != want["image"].view(np.uint32)).sum()) == 0
    finite = np.isfinite(want["depthmap"])
    gd = np.where(finite, gd, 0).astype(np.float32)
    torch.autograd.backward([image, depthmap], [torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda)])
    wanted = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], want,
                                    W, H, 16, 16, m["per_pixel_sort"], ml, magnitudes=True)
    for label, got, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), (v.grad, c.grad, o.grad), wanted[:3], wanted[3:]):
        assert_gradients_close(f"{mode}: {label}", got.cpu().numpy(), w, mag)
    # the attribute on `ends` must survive save_for_backward, or every backward pass pays for a second forward kernel
    assert Fn.resume_seen == [not drop_private_state]


def test_expired_wait_is_reported_on_every_path(cuda):
    """A non-zero status word of the list kernels (a bounded look-back wait expired: the lists are invalid) raises in
    the backward pass, at the start of the next frame and in verify_frames, not only when timings are recorded, and
    switches the kernels to ticketed tile numbers.  No wait is provoked: the status word is forged."""
    import torch
    import trigrad_amd
    from trigrad_amd import _C
    import scenes as S
    d = to_device(S.config(0), cuda)
    args = (d["vertices"], d["indices"], d["colors"], d["opacities"], 256, 256, 16, 16, 1 / 256)
    *results, resume = _C._forward_full(*args, True, False, 2000)
    image, depthmap, weights, sorted_ids, offsets, bary, ends = results[:7]
    try:
        bad = _C.StatusCheck(torch.ones((1,), dtype=torch.int32, device=cuda), frame=7)
        gi = torch.ones_like(image)
        with pytest.raises(RuntimeError, match="look-back wait timed out.*frame 7"):
            _C.render_backward(gi, None, *args[:4], sorted_ids, offsets, bary, image, depthmap, weights, ends, *args[4:], False, 2000,
                               resume=(resume[0], resume[1], bad, resume[3], resume[4]))
        assert _C._tickets_forced
        # the same through the public entry point: the next frame refuses to start
        _C._pending_checks.append(_C.StatusCheck(torch.ones((1,), dtype=torch.int32, device=cuda)))
        torch.cuda.synchronize()
        with pytest.raises(RuntimeError, match="look-back wait timed out"):
            trigrad_amd.render(*args[:6])
        assert not _C._pending_checks or all(not c.checked for c in _C._pending_checks)
        trigrad_amd.render(*args[:6])  # reported once; later frames run (their tiles numbered by ticket)
        # a caller that only renders forward asks before it trusts its frames
        _C._pending_checks.append(_C.StatusCheck(torch.ones((1,), dtype=torch.int32, device=cuda)))
        with pytest.raises(RuntimeError, match="look-back wait timed out"):
            trigrad_amd.verify_frames()
        trigrad_amd.verify_frames()
        # and a healthy frame's word is zero
        resume[2].verify()
    finally:
        _C.force_tickets(False)


def test_invalid_lists_show_in_the_frame(cuda):
    """The forward kernels look at the status word of the list kernels: with a word that reports an expired wait they
    read no list and fill image and depth map with NaN, in both compositing orders.  The word is forged."""
    import ctypes as C
    import torch
    from trigrad_amd import _C, _lib
    import scenes as S
    d = to_device(S.config(0), cuda)
    W = H = 256
    v, idx, col, op = d["vertices"], d["indices"], d["colors"], d["opacities"]
    *results, resume = _C._forward_full(v, idx, col, op, W, H, 16, 16, 1 / 256, True, False, 2000)
    want_image, _, _, sorted_ids, offsets, bary = results[:6]
    lib = _lib.load(32)
    for word, pps in ((0, False), (1, False), (1, True)):
        status = torch.full((1,), word, dtype=torch.int32, device=cuda)
        image = torch.zeros((H, W, 4), device=cuda)
        planes = [torch.zeros((H, W), device=cuda) for _ in range(3)]
        ends = torch.zeros((H, W), dtype=torch.int32, device=cuda)
        last = torch.zeros((H, W), dtype=torch.int32, device=cuda)
        p = lambda t: C.c_void_p(t.data_ptr())
        _lib.check(lib.tg_render_forward(p(v), p(idx), p(col), p(op), p(sorted_ids), p(offsets), p(bary), W, H, 16, 16, 1 / 256, int(pps),
                                         2000, p(image), p(planes[0]), p(planes[1]), p(ends), p(last), p(planes[2]) if pps else None,
                                         None, None, None, None, p(status), C.c_void_p(torch.cuda.current_stream().cuda_stream)),
                   "tg_render_forward")
        if word == 0:
            assert torch.equal(image, want_image)
        else:
            assert torch.isnan(image).all() and torch.isnan(planes[0]).all() and int(ends.abs().max()) == 0


def test_ticketed_tile_numbers_change_nothing(cuda, oracle):
    """force_tickets: the kernels that wait on other workgroups take their tile numbers from an atomic ticket whatever
    the size of the grid.  Lists and image are, bit for bit, what they are without."""
    import torch
    import trigrad_amd
    from trigrad_amd import _C
    import scenes as S
    scene = S.config(1)
    d = to_device(scene, cuda)
    W, H = scene["width"], scene["height"]

    def frame():
        image, _ = trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, 16, 16, 1 / 256, False, False, -1)
        b = _C.bin_frame(d["vertices"], d["indices"], W, H, 16, 16)
        K = int(b["total_and_status"][0].item())
        keys, ids, status, offsets = _C.build_frame_lists(b, K)
        assert int(status.item()) == 0
        return image, keys.clone(), ids.clone(), offsets.clone()

    plain = frame()
    try:
        _C.force_tickets(True)
        ticketed = frame()
    finally:
        _C.force_tickets(False)
    for a, b in zip(plain, ticketed):
        assert torch.equal(a, b)


def test_frames_on_two_streams_keep_their_own_state(cuda):
    """Two streams render different frames at the same time (tickets on: the device is shared between them).  The
    binning's state between calls -- epoch-stamped look-back words, alternating digit totals -- is kept per stream,
    so every frame is what its stream gives alone."""
    import torch
    import trigrad_amd
    from trigrad_amd import _C
    import scenes as S
    frames = []
    for config in (1, 0):
        scene = S.config(config)
        d = to_device(scene, cuda)
        frames.append((d, scene["width"], scene["height"]))

    def render(k):
        d, W, H = frames[k]
        return trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, 16, 16, 1 / 256, False, False, -1)[0]

    alone = [render(0), render(1)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=cuda), torch.cuda.Stream(device=cuda)]
    got = [[], []]
    try:
        _C.force_tickets(True)
        for _ in range(6):
            for k in (0, 1):
                with torch.cuda.stream(streams[k]):
                    got[k].append(render(k))
        torch.cuda.synchronize()
        trigrad_amd.verify_frames()
    finally:
        _C.force_tickets(False)
    states = {key for key in _C._frame_states if key[0] == cuda.index}
    assert len({key[1] for key in states}) >= 3  # the default stream's and the two streams' own
    for k in (0, 1):
        for image in got[k]:
            assert torch.equal(image, alone[k])


@pytest.mark.parametrize("mode", ["A_default", "B_unlimited"])
def test_scene_without_a_single_key(mode, cuda):
    """M >= 1 but K = 0 (every triangle degenerate): transparent image, infinite depth, zero gradients."""
    import torch
    import trigrad_amd
    m = MODES[mode]
    v = torch.tensor([[0.1, 0.1, 0.5, 2.0]] * 3 + [[float("nan"), 0.0, 0.5, 1.0], [0.2, 0.3, 0.5, 1.0], [0.4, 0.1, 0.5, 1.0]],
                     dtype=torch.float32, device=cuda).requires_grad_()
    idx = torch.tensor([[0, 1, 2], [3, 4, 5], [0, 0, 4]], dtype=torch.int32, device=cuda)
    c = torch.rand((6, 3), device=cuda).requires_grad_()
    o = torch.rand((6,), device=cuda).requires_grad_()
    image, depthmap = trigrad_amd.render(v, idx, c, o, 70, 50, 16, 16, 1 / 256, False, m["per_pixel_sort"], m["max_layers"])
    assert float(image[..., :3].abs().max()) == 0.0 and float(image[..., 3].min()) == 1.0 and torch.isinf(depthmap).all()
    (image.sum() + torch.where(torch.isinf(depthmap), torch.zeros_like(depthmap), depthmap).sum()).backward()
    for g in (v.grad, c.grad, o.grad):
        assert float(g.abs().max()) == 0.0
