"""Shared helpers of the parity tests."""
import numpy as np


def to_device(scene, device):
    import torch
    return {k: (torch.from_numpy(v).to(device) if isinstance(v, np.ndarray) else v) for k, v in scene.items()}


def u64(t):
    """int64 tensor holding uint64 bit patterns -> numpy uint64."""
    return t.cpu().numpy().view(np.uint64)


def assert_close(name, got, want, rtol, atol):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{name}: shape {got.shape} vs {want.shape}"
    both_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    err = np.where(both_inf, 0.0, np.abs(got - want))
    bound = atol + rtol * np.abs(np.where(both_inf, 0.0, want))
    bad = ~(err <= bound)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - bound, -1)), err.shape)
        raise AssertionError(f"{name}: {bad.sum()} of {bad.size} outside rtol={rtol} atol={atol}; worst at {i}: "
                             f"got {got[i]!r} want {want[i]!r}")
    return float(err.max()) if err.size else 0.0


# ---- the gradient bar --------------------------------------------------------------------------------------
# north_star's bar is 1e-4 relative + 1e-6 absolute.  The oracle adds a gradient element's terms into a float64 sum; the
# kernels add the same terms in float32 (run sums, then float atomics, in no fixed order).  Where the terms cancel, that
# alone leaves an error proportional to the sum of their MAGNITUDES, S, whatever the result is: a float32 addition
# chain of n steps is off by at most n * 2^-24 * S and typically by about 2^-24 * S (the largest factor any test of this
# suite needs is 0.9; the allowance is twice 2^-24 * S).  The oracle returns S per element
# (render_backward(..., magnitudes=True)), and the bound used is, element by element,
#     |got - want| <= 1e-4 |want| + 1e-6 + GRAD_SUM_STEPS * 2^-24 * S
# An element whose own terms are small gets no allowance from large gradients elsewhere in the array.
GRAD_RTOL, GRAD_ATOL = 1e-4, 1e-6
GRAD_SUM_STEPS = 2.0
WORST_GRADIENT = {"ratio": 0.0, "where": "", "needed_steps": 0.0, "elements": 0, "beyond_stated_bar": 0}


def assert_gradients_close(name, got, want, magnitude, rtol=GRAD_RTOL, atol=GRAD_ATOL, steps=GRAD_SUM_STEPS):
    """got: float32 gradients of the kernels; want, magnitude: the oracle's float64 sums and sums of magnitudes.
    NaN must sit where the oracle has NaN.  Keeps the worst error/bound ratio seen (conftest prints it)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    magnitude = np.asarray(magnitude, dtype=np.float64)
    assert got.shape == want.shape == magnitude.shape, f"{name}: shapes {got.shape}, {want.shape}, {magnitude.shape}"
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{name}: NaN pattern differs"
    ok = ~np.isnan(want)
    err = np.abs(np.where(ok, got - want, 0.0))
    stated = atol + rtol * np.abs(np.where(ok, want, 0.0))
    rounding = 2.0 ** -24 * np.where(ok & np.isfinite(magnitude), magnitude, 0.0)
    bound = stated + steps * rounding
    bad = ~(err <= bound)
    if err.size:
        ratio = err / bound
        i = np.unravel_index(np.argmax(ratio), ratio.shape)
        w = WORST_GRADIENT
        w["elements"] += int(err.size)
        w["beyond_stated_bar"] += int((err > stated).sum())
        beyond = err > stated
        if beyond.any():
            w["needed_steps"] = max(w["needed_steps"], float(((err - stated)[beyond] / np.maximum(rounding[beyond], 1e-300)).max()))
        if ratio[i] > w["ratio"]:
            w["ratio"], w["where"] = float(ratio[i]), f"{name} at {i}"
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - bound, -1)), err.shape)
        raise AssertionError(f"{name}: {bad.sum()} of {bad.size} outside {rtol} |want| + {atol} + {steps} * 2^-24 * S; worst at {i}: "
                             f"got {got[i]!r} want {want[i]!r} S {magnitude[i]!r}")


SCENE_PARAMS = {}
