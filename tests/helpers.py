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


SCENE_PARAMS = {}
