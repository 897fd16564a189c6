"""GPU parity at the full size of the five benchmark configurations.

Against the CPU oracle (OpenMP over tiles, so that a 1M-triangle frame takes
seconds): tile counts, emitted keys, sorted keys/payloads and tile ranges
bit-exact; image within 1e-5 absolute (and, since the forward arithmetic is the
oracle's operation for operation, bit-identical); gradients of the L2 loss
against the seeded target within 1e-4 relative + 1e-6 absolute, both for the
loss as the benchmark defines it (mean) and, so that the absolute term does not
make the check vacuous, for the summed loss, where two float32 rounding steps of
the magnitudes of the element's own terms (from the oracle) are allowed on top.

Size-independent properties checked on the GPU results alone: keys sorted,
ranges monotone with offsets[T] = K = sum of counts, payload multiset = emitted
triangle ids, image invariant under a permutation of the triangle list.
"""
import numpy as np
import pytest

from helpers import assert_gradients_close, assert_close, to_device, u64

pytestmark = pytest.mark.gpu

MODES = {"A": dict(per_pixel_sort=True, max_layers=32), "B": dict(per_pixel_sort=False, max_layers=-1)}
_cache = {}


def _scene(cfg):
    import scenes as S
    if cfg not in _cache:
        _cache.clear()
        _cache[cfg] = S.config(cfg)
    return _cache[cfg]


@pytest.fixture(scope="module", autouse=True)
def _threads(oracle):
    import os
    oracle.set_threads(min(16, len(os.sched_getaffinity(0))))
    yield
    oracle.set_threads(1)
    _cache.clear()


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4])
def test_binning_sort_ranges_full_size(cfg, cuda, oracle):
    from trigrad_amd import _C
    scene = _scene(cfg)
    W, H = scene["width"], scene["height"]
    v, idx = scene["vertices"], scene["indices"]
    d = to_device({k: scene[k] for k in ("vertices", "indices")}, cuda)
    T = _C.num_tiles(W, H, 16, 16)
    counts = _C.bin_count(d["vertices"], d["indices"], W, H, 16, 16)
    want_counts, tile_counts = oracle.bin_count(v, idx, W, H)
    np.testing.assert_array_equal(counts.cpu().numpy(), want_counts)
    offs, total, status = _C.scan_exclusive(counts)
    K = int(total.item())
    assert int(status.item()) == 0 and K == int(want_counts.sum())
    em = oracle.bin_emit(v, idx, W, H)
    keys, payload = _C.bin_emit(d["vertices"], d["indices"], offs, K, W, H, 16, 16)
    np.testing.assert_array_equal(u64(keys), em["keys64"])
    np.testing.assert_array_equal(payload.cpu().numpy(), em["tri"])
    skeys, svals, sstatus = _C.sort_pairs(keys, payload, _C.key_bits(T))
    assert int(sstatus.item()) == 0
    sk = u64(skeys)
    sv = svals.cpu().numpy()
    order = np.argsort(em["keys64"], kind="stable")  # library statement of the stable sort
    np.testing.assert_array_equal(sk, em["keys64"][order])
    np.testing.assert_array_equal(sv, em["tri"][order])
    offsets = _C.tile_ranges(skeys, T).cpu().numpy()
    ref_offsets, ref_ids, _ = oracle.per_tile_lists(v, idx, W, H)
    np.testing.assert_array_equal(offsets, ref_offsets)
    np.testing.assert_array_equal(sv, ref_ids)
    # the route the frame takes: count + scan, then the emission without a host wait; tile passes by column and row
    binned = _C.bin_frame(d["vertices"], d["indices"], W, H, 16, 16, capacity=K + 1000)
    assert binned["total_and_status"].tolist() == [K, 0]
    np.testing.assert_array_equal(binned["values"][:K].cpu().numpy(), em["tri"])
    np.testing.assert_array_equal(u64(binned["keys"][:K]) & np.uint64(0xFFFFFFFF), em["keys64"] & np.uint64(0xFFFFFFFF))  # depth words
    fkeys, fids, fstatus, foffsets = _C.build_frame_lists(binned, K)
    assert int(fstatus.item()) == 0
    np.testing.assert_array_equal(u64(fkeys), sk)
    np.testing.assert_array_equal(fids.cpu().numpy(), sv)
    np.testing.assert_array_equal(foffsets.cpu().numpy(), ref_offsets)
    del binned, fkeys, fids, foffsets
    # the two-call route (count + scan in one pass, the host reads K, emission from records, tile-list sort)
    setup = _C.bin_setup(d["vertices"], d["indices"], W, H, 16, 16)
    assert setup["total_and_status"].tolist() == [K, 0]
    np.testing.assert_array_equal(setup["tri_offsets"].cpu().numpy(), offs.cpu().numpy())
    fkeys, fids, fstatus, foffsets = _C.build_tile_lists(setup, K)
    assert int(fstatus.item()) == 0
    np.testing.assert_array_equal(u64(fkeys), sk)
    np.testing.assert_array_equal(fids.cpu().numpy(), sv)
    np.testing.assert_array_equal(foffsets.cpu().numpy(), ref_offsets)
    # properties that need no oracle
    assert (np.diff(sk.astype(np.uint64)) >= 0).all() if K > 1 else True
    assert offsets[0] == 0 and offsets[-1] == K and (np.diff(offsets) >= 0).all()
    np.testing.assert_array_equal(np.diff(offsets), tile_counts)
    np.testing.assert_array_equal(np.bincount(sv, minlength=idx.shape[0]), want_counts)


@pytest.mark.parametrize("mode", ["A", "B"])
@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4])
def test_forward_backward_full_size(cfg, mode, cuda, oracle):
    import torch
    import trigrad_amd
    scene = _scene(cfg)
    W, H = scene["width"], scene["height"]
    m = MODES[mode]
    d = to_device({k: scene[k] for k in ("vertices", "indices", "colors", "opacities", "target")}, cuda)
    fwd = oracle.render(scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], W, H, 16, 16, 1 / 256,
                        m["per_pixel_sort"], m["max_layers"])
    zero_gd = np.zeros((H, W), np.float32)
    for reduction in ("mean", "sum"):
        v = d["vertices"].clone().requires_grad_()
        c = d["colors"].clone().requires_grad_()
        o = d["opacities"].clone().requires_grad_()
        image, depthmap = trigrad_amd.render(v, d["indices"], c, o, W, H, 16, 16, 1 / 256, False, **m)
        diff = (image - d["target"]) ** 2
        loss = diff.mean() if reduction == "mean" else diff.sum()
        loss.backward()
        img = image.detach().cpu().numpy()
        assert_close(f"config{cfg}/{mode}: image", img, fwd["image"], 0.0, 1e-5)
        assert int((img.view(np.uint32) != fwd["image"].view(np.uint32)).sum()) == 0
        dm = depthmap.detach().cpu().numpy()
        fin = np.isfinite(fwd["depthmap"])
        assert np.array_equal(np.isfinite(dm), fin)
        assert_close(f"config{cfg}/{mode}: depthmap", dm[fin], fwd["depthmap"][fin], 1e-5, 1e-5)
        scale = 1.0 / fwd["image"].size if reduction == "mean" else 1.0
        gi = (2.0 * scale * (fwd["image"].astype(np.float64) - scene["target"])).astype(np.float32)
        wanted = oracle.render_backward(gi, zero_gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"],
                                        fwd, W, H, 16, 16, m["per_pixel_sort"], m["max_layers"], magnitudes=True)
        for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), (v.grad, c.grad, o.grad), wanted[:3], wanted[3:]):
            g = g.cpu().numpy()
            if reduction == "mean":  # the benchmark's loss: gradients around 1e-7, the stated bar as it is
                assert_close(f"config{cfg}/{mode}/mean: {label}", g, w, 1e-4, 1e-6)
            # float32 atomics in arbitrary order against the float64 sum of the same terms: the stated bar plus the
            # rounding of a float32 sum of the element's own terms
            assert_gradients_close(f"config{cfg}/{mode}/{reduction}: {label}", g, w, mag)
        del v, c, o, image, depthmap, loss, diff
    torch.cuda.empty_cache()


@pytest.mark.parametrize("cfg", [1, 2])
def test_image_invariant_under_triangle_permutation(cfg, cuda):
    """Shuffling the triangle list changes ids, keys' tie order and every
    intermediate, but not the picture (per-pixel depth order; the generator's
    depths are distinct)."""
    import torch
    import trigrad_amd
    scene = _scene(cfg)
    W, H = scene["width"], scene["height"]
    d = to_device({k: scene[k] for k in ("vertices", "indices", "colors", "opacities")}, cuda)
    a, _ = trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H)
    perm = torch.randperm(d["indices"].shape[0], device=cuda, generator=torch.Generator(device=cuda).manual_seed(0))
    b, _ = trigrad_amd.render(d["vertices"], d["indices"][perm].contiguous(), d["colors"], d["opacities"], W, H)
    assert float((a - b).abs().max()) <= 1e-5


def test_stage_timings_describe_the_frame_that_runs(cuda):
    """record_timing=True times the route an untimed call runs (the same entry points in the same order, with the
    reference's five stage names, render.cu:723-747): on the headline frame the stage times add up to the forward time
    of an untimed call within a tenth."""
    import torch
    import trigrad_amd
    scene = _scene(2)
    W, H = scene["width"], scene["height"]
    d = to_device({k: scene[k] for k in ("vertices", "indices", "colors", "opacities")}, cuda)
    args = (d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, 16, 16, 1 / 256)
    kinds = {}
    for pps, ml in ((False, -1), (True, 32)):
        for _ in range(3):
            trigrad_amd.render(*args, False, pps, ml)
        untimed = []
        for _ in range(7):
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            trigrad_amd.render(*args, False, pps, ml)
            e1.record()
            e1.synchronize()
            untimed.append(e0.elapsed_time(e1) / 1000.0)
        sums = []
        for _ in range(7):
            torch.cuda.synchronize()
            _, _, timings = trigrad_amd.render(*args, True, pps, ml)
            assert set(timings) == {"init", "per_tile_lists", "sorting", "bary_transforms", "rasterization"}
            sums.append(sum(timings.values()))
        a, b = float(np.median(untimed)), float(np.median(sums))
        kinds[pps] = (a, b)
        print(f"per_pixel_sort={pps}: untimed forward {a * 1e3:.3f} ms, stages add up to {b * 1e3:.3f} ms")
        assert abs(b - a) <= 0.1 * a, f"per_pixel_sort={pps}: stages add up to {b * 1e3:.3f} ms, an untimed forward pass takes {a * 1e3:.3f} ms"
