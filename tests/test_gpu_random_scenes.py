"""Randomised parity: image size, tile shape, triangle count and size, vertex sharing, mode, layer limit and
threshold drawn at random; the forward pass is compared bit for bit and the gradients within the tolerance of
test_gpu_render, against the oracle on the same inputs."""
import numpy as np
import pytest

from helpers import assert_gradients_close
from test_gpu_render import _check_forward, _forward_both, _grad_inputs

pytestmark = pytest.mark.gpu

TILES = [(16, 16), (8, 8), (4, 4), (32, 32), (8, 4), (12, 20), (24, 16), (16, 8), (32, 16), (5, 7), (16, 32), (2, 2), (64, 16)]


@pytest.mark.parametrize("block", range(8))
def test_random_scenes_match_oracle(block, cuda, oracle):
    import torch
    from trigrad_amd import _C
    import scenes as S
    for case in range(block * 40, block * 40 + 40):
        rng = np.random.default_rng(1000 + case)
        W, H = int(rng.integers(8, 260)), int(rng.integers(8, 200))
        tw, th = TILES[int(rng.integers(0, len(TILES)))]
        n = int(rng.integers(1, 1500))
        sigma = float(rng.choice([1.5, 4.0, 9.0, 25.0, 80.0]))
        scene = S.random_soup(n, W, H, seed=case, sigma_px=sigma, varying_w=bool(rng.integers(0, 2)),
                              shared=bool(rng.integers(0, 2)) and n >= 60)
        pps = bool(rng.integers(0, 2))
        mode = dict(per_pixel_sort=pps, max_layers=int(rng.choice([-1, 1, 3, 5, 17, 32, 33, 40, 70])))
        thr = float(rng.choice([1 / 256, 0.0, 0.05, 0.5]))
        name = f"case {case}: {W}x{H}, tiles {tw}x{th}, {n} triangles of {sigma} px, {mode}, threshold {thr}"
        d, want, got, ml = _forward_both(scene, tw, th, mode, cuda, oracle, thr=thr)
        _check_forward(name, want, got, (th, tw))
        gi, gd = _grad_inputs(scene, case, bool(rng.integers(0, 2)))
        wanted = oracle.render_backward(gi, gd, scene["vertices"], scene["indices"], scene["colors"], scene["opacities"], want,
                                        W, H, tw, th, pps, ml, literal=False, magnitudes=True)
        image, depthmap, weights, sorted_ids, offsets, bary, ends, _, resume = got
        out = _C.render_backward(torch.from_numpy(gi).to(cuda), torch.from_numpy(gd).to(cuda), d["vertices"], d["indices"],
                                 d["colors"], d["opacities"], sorted_ids, offsets, bary, image, depthmap, weights, ends, W, H,
                                 tw, th, thr, pps, ml, resume=resume)
        for label, g, w, mag in zip(("grad_vertices", "grad_colors", "grad_opacities"), out, wanted[:3], wanted[3:]):
            assert_gradients_close(f"{name}: {label}", g.cpu().numpy(), w, mag)
