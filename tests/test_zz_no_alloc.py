"""The scan entry point that allocates nothing (its look-back state is a device array inside the library)
against the entry point that takes a workspace: same results, bit for bit, on two calls in a row, the second
on a smaller input (the shared state keeps the first call's contents and must not leak into the second).
Both are called through the C ABI."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _both(lib, x, cuda, with_heads):
    import torch
    n = x.numel()
    stream = C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)
    results = []
    for noalloc in (False, True):
        out = torch.full((n,), -7, dtype=torch.int32, device=cuda)
        pair = torch.full((2,), -7, dtype=torch.int32, device=cuda)  # total, status
        heads = torch.full((max(1, n // 8),), -7, dtype=torch.int32, device=cuda) if with_heads else None
        cap = 0 if heads is None else heads.numel()
        if noalloc:
            code = lib.tg_scan_exclusive_u32_noalloc(_p(x), _p(out), n, _p(pair[:1]), _p(pair[1:]), 256, cap, _p(heads), stream)
        else:
            nbytes = int(lib.tg_scan_workspace_bytes(n))
            ws = torch.empty((nbytes,), dtype=torch.uint8, device=cuda)
            code = lib.tg_scan_exclusive_u32(_p(x), _p(out), n, _p(pair[:1]), _p(ws), nbytes, _p(pair[1:]), 256, cap, _p(heads), stream)
        assert code == 0, lib.tg_last_error()
        torch.cuda.synchronize()
        results.append((out.cpu().numpy(), pair.cpu().numpy(), None if heads is None else heads.cpu().numpy()))
    return results


@pytest.mark.parametrize("with_heads", [False, True])
def test_scan_without_allocation_matches_scan_with_workspace(with_heads, cuda):
    import torch
    from trigrad_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(5)
    # the first call spans thousands of state words, the second (smaller) one reuses the first few of them
    for n in (3_000_017, 70_001, 2048, 1):
        x_np = rng.integers(0, 9, size=n).astype(np.int32)
        x = torch.from_numpy(x_np).to(cuda)
        (out_a, pair_a, heads_a), (out_b, pair_b, heads_b) = _both(lib, x, cuda, with_heads)
        np.testing.assert_array_equal(out_b, out_a)
        np.testing.assert_array_equal(pair_b, pair_a)
        np.testing.assert_array_equal(out_b, np.cumsum(x_np) - x_np)
        assert pair_b[0] == x_np.sum() and pair_b[1] == 0
        if with_heads:
            np.testing.assert_array_equal(heads_b, heads_a)


def test_scan_without_allocation_rejects_oversize_and_allocates_nothing(cuda):
    import torch
    from trigrad_amd import _lib
    lib = _lib.load()
    limit = int(lib.tg_scan_noalloc_max_n())
    assert limit == 1 << 24
    one = torch.zeros((4,), dtype=torch.int32, device=cuda)
    assert lib.tg_scan_exclusive_u32_noalloc(_p(one), _p(one), limit + 1, _p(one), None, 256, 0, None, None) == -1
    assert b"exceeds" in lib.tg_last_error()
    # the largest size it takes, and no growth of the device's memory in use across calls
    x = torch.ones((limit,), dtype=torch.int32, device=cuda)
    out = torch.empty_like(x)
    pair = torch.empty((2,), dtype=torch.int32, device=cuda)
    stream = C.c_void_p(torch.cuda.current_stream(cuda).cuda_stream)
    assert lib.tg_scan_exclusive_u32_noalloc(_p(x), _p(out), limit, _p(pair[:1]), _p(pair[1:]), 256, 0, None, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(cuda)
    for _ in range(3):
        assert lib.tg_scan_exclusive_u32_noalloc(_p(x), _p(out), limit, _p(pair[:1]), _p(pair[1:]), 256, 0, None, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(cuda)
    assert free_after == free_before
    assert pair.tolist() == [limit, 0]
    assert out[-1].item() == limit - 1 and out[12345].item() == 12345
