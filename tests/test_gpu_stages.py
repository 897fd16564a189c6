"""GPU parity of the integer stages (binning, scan, key emission, radix sort, tile
ranges) and of the bary matrices against the CPU oracle: bit-exact.

Everything here calls the C ABI of libtrigrad_hip.so through trigrad_amd._C.
"""
import numpy as np
import pytest

from helpers import to_device, u64

pytestmark = pytest.mark.gpu


def _scenes():
    import scenes as S
    out = {
        "config0": lambda: (S.config(0, with_target=False), 16, 16),
        "soup_varying_w": lambda: (S.random_soup(3000, 300, 200, seed=1, sigma_px=9.0, varying_w=True), 16, 16),
        "soup_shared": lambda: (S.random_soup(2000, 257, 131, seed=2, shared=True), 16, 16),
        "soup_big_tris": lambda: (S.random_soup(400, 128, 128, seed=3, sigma_px=80.0, varying_w=True), 16, 16),
        "soup_tile4": lambda: (S.random_soup(500, 50, 50, seed=4, sigma_px=5.0), 4, 4),
        "soup_tile32": lambda: (S.random_soup(800, 200, 150, seed=5, sigma_px=12.0), 32, 32),
        "soup_tile_8x4": lambda: (S.random_soup(800, 100, 90, seed=6, sigma_px=7.0), 8, 4),
        "soup_tile_12x20": lambda: (S.random_soup(800, 130, 170, seed=7, sigma_px=7.0), 12, 20),
        "soup_tile8": lambda: (S.random_soup(600, 90, 70, seed=8, sigma_px=6.0), 8, 8),            # one wave per tile
        "soup_tile_24x16": lambda: (S.random_soup(800, 150, 110, seed=9, sigma_px=9.0), 24, 16),   # six 8x8 squares over two workgroups
        "squares": lambda: (S.overlapping_squares(10), 4, 4),
        "large_triangles": lambda: (S.large_triangles(3, r=4), 4, 4),
        "depth_overlap": lambda: (S.depth_overlap(), 16, 16),
        "overlapping_triangles": lambda: (S.overlapping_triangles(), 16, 16),
        "unit_square_negative_z": lambda: (S.unit_square(), 16, 16),
        "overlap_mesh_inf_w": lambda: (S.overlap_mesh(), 16, 16),
        "grid_mesh": lambda: (S.grid_mesh(40, 40, -0.9, 0.9, -0.9, 0.9, width=96, height=96), 16, 16),
        # every border tile, the first one included, has an empty list and nothing to walk back
        "center_island": lambda: (S.grid_mesh(12, 12, -0.3, 0.3, -0.3, 0.3, width=128, height=96), 16, 16),
    }
    return out


def _degenerate_scene():
    """Zero-area, NaN, infinite, huge and far off-screen triangles mixed with ordinary ones."""
    import scenes as S
    s = S.random_soup(64, 96, 80, seed=11, sigma_px=10.0, varying_w=True)
    v = s["vertices"].copy()
    v[0:3, :2] = v[0, :2]                       # zero area
    v[3:6, 0] = np.float32("nan")               # NaN
    v[6, 0] = np.float32("inf")                 # infinite
    v[9:12, :2] *= np.float32(1e20)             # area overflows to inf
    v[12:15, 0] += np.float32(5.0)              # entirely right of the screen: clamped into the border tiles
    v[15:18, :2] = np.array([[-1, -1], [1, -1], [0, 1]], np.float32) * np.float32(3)  # covers everything
    v[18, :2] = (-1.0, -1.0); v[19, :2] = (-0.75, -1.0); v[20, :2] = (-1.0, -0.5)    # on tile boundaries
    s["vertices"] = v
    return s, 16, 16


SCENES = _scenes()
SCENES["degenerate"] = _degenerate_scene


@pytest.mark.parametrize("name", sorted(SCENES))
def test_binning_sort_ranges_bit_exact(name, cuda, oracle):
    from trigrad_amd import _C
    scene, tw, th = SCENES[name]()
    W, H = scene["width"], scene["height"]
    v, idx = scene["vertices"], scene["indices"]
    d = to_device(scene, cuda)
    T = _C.num_tiles(W, H, tw, th)

    tri_counts, tile_counts = oracle.bin_count(v, idx, W, H, tw, th)
    got_counts = _C.bin_count(d["vertices"], d["indices"], W, H, tw, th)
    np.testing.assert_array_equal(got_counts.cpu().numpy(), tri_counts)

    offs, total, status = _C.scan_exclusive(got_counts)
    assert int(status.item()) == 0
    K = int(total.item())
    assert K == int(tri_counts.sum())
    np.testing.assert_array_equal(offs.cpu().numpy(), np.cumsum(tri_counts) - tri_counts)

    em = oracle.bin_emit(v, idx, W, H, tw, th)
    keys, payload = _C.bin_emit(d["vertices"], d["indices"], offs, K, W, H, tw, th)
    np.testing.assert_array_equal(u64(keys), em["keys64"])
    np.testing.assert_array_equal(payload.cpu().numpy(), em["tri"])
    # same emission with the owners noted by the scan instead of searched, also with a table too short for all keys
    for capacity in (_C.owner_heads_for(idx.shape[0], cuda).numel(), 3):
        import torch
        heads = torch.full((capacity,), -1, dtype=torch.int32, device=cuda)
        offs2, total2, _ = _C.scan_exclusive(got_counts, heads=heads)
        n_heads = min(capacity, -(-K // _C.OWNER_STRIDE))
        want_heads = np.searchsorted(np.cumsum(tri_counts), np.arange(n_heads) * _C.OWNER_STRIDE, side="right")
        np.testing.assert_array_equal(heads.cpu().numpy()[:n_heads], want_heads)
        keys2, payload2 = _C.bin_emit(d["vertices"], d["indices"], offs2, K, W, H, tw, th, heads)
        np.testing.assert_array_equal(u64(keys2), em["keys64"])
        np.testing.assert_array_equal(payload2.cpu().numpy(), em["tri"])

    want_keys, want_vals = oracle.sort_pairs_u64(em["keys64"], em["tri"])
    skeys, svals, sstatus = _C.sort_pairs(keys, payload, _C.key_bits(T))
    assert int(sstatus.item()) == 0
    np.testing.assert_array_equal(u64(skeys), want_keys)
    np.testing.assert_array_equal(svals.cpu().numpy(), want_vals)

    offsets = _C.tile_ranges(skeys, T)
    np.testing.assert_array_equal(offsets.cpu().numpy(), oracle.tile_ranges(want_keys, T))

    # the same observable through the reference-shaped route: per-tile histogram,
    # cumsum, slot fill in triangle order, stable segmented sort on float keys
    ref_offsets, ref_ids, _ = oracle.per_tile_lists(v, idx, W, H, tw, th)
    np.testing.assert_array_equal(offsets.cpu().numpy(), ref_offsets)
    np.testing.assert_array_equal(svals.cpu().numpy(), ref_ids)
    np.testing.assert_array_equal(np.diff(ref_offsets), tile_counts)

    # the frame's route: count + scan in one pass, emission from the triangles' records, tile bits sorted
    # through memory and depth bits per tile in LDS
    for with_heads in (True, False):
        setup = _C.bin_setup(d["vertices"], d["indices"], W, H, tw, th, with_heads=with_heads)
        assert setup["total_and_status"].tolist() == [K, 0]
        np.testing.assert_array_equal(setup["tri_offsets"].cpu().numpy(), np.cumsum(tri_counts) - tri_counts)
        ekeys, epayload, estatus, _ = _C.build_tile_lists(setup, K, emit_only=True)
        np.testing.assert_array_equal(u64(ekeys), em["keys64"])
        np.testing.assert_array_equal(epayload.cpu().numpy(), em["tri"])
        fkeys, fids, fstatus, foffsets = _C.build_tile_lists(setup, K)
        assert int(fstatus.item()) == 0
        np.testing.assert_array_equal(u64(fkeys), want_keys)
        np.testing.assert_array_equal(fids.cpu().numpy(), want_vals)
        np.testing.assert_array_equal(foffsets.cpu().numpy(), ref_offsets)

    got_bary = _C.cartesian_to_bary(d["vertices"], d["indices"]).cpu().numpy()
    want_bary = oracle.bary(v, idx)
    np.testing.assert_array_equal(got_bary.view(np.uint32), want_bary.view(np.uint32))


# the largest size has more tiles than workgroups fit the device at once (ticketed tile numbers)
@pytest.mark.parametrize("n", [1, 5, 63, 64, 65, 2047, 2048, 2049, 100_003, (1 << 20) + 7, 6_000_011])
def test_scan_matches_cumsum(n, cuda):
    import torch
    from trigrad_amd import _C
    rng = np.random.default_rng(n)
    x = rng.integers(0, 50, size=n).astype(np.int32)
    x[rng.integers(0, n, size=max(1, n // 10))] = 0
    t = torch.from_numpy(x).to(cuda)
    out, total, status = _C.scan_exclusive(t)
    assert int(status.item()) == 0
    np.testing.assert_array_equal(out.cpu().numpy(), np.cumsum(x) - x)
    assert int(total.item()) == int(x.sum())
    out2, total2, _ = _C.scan_exclusive(t, out=t)  # in place
    np.testing.assert_array_equal(out2.cpu().numpy(), np.cumsum(x) - x)
    assert int(total2.item()) == int(x.sum())


def test_scan_empty(cuda):
    import torch
    from trigrad_amd import _C
    out, total, status = _C.scan_exclusive(torch.empty((0,), dtype=torch.int32, device=cuda))
    assert out.numel() == 0 and int(total.item()) == 0 and int(status.item()) == 0


@pytest.mark.parametrize("n,end_bit,distinct", [
    (1, 64, None), (2, 64, None), (100, 64, None), (4095, 64, None), (4096, 64, None), (4097, 64, None),
    (100_000, 64, None), (100_000, 45, None), (50_000, 64, 7), (300_000, 40, 1000), ((1 << 20) + 13, 45, None),
    (5_000_017, 45, None), (5_000_017, 24, 50_000),  # more tiles than fit the device at once: ticketed tile numbers
])
def test_sort_pairs_stable(n, end_bit, distinct, cuda, oracle):
    """Random keys, optionally drawn from few distinct values so that stability
    (equal keys keep input order) decides the result; numpy's stable argsort is
    the library statement of the expected permutation."""
    import torch
    from trigrad_amd import _C
    rng = np.random.default_rng(n + end_bit)
    if distinct:
        pool = rng.integers(0, 1 << min(end_bit, 63), size=distinct, dtype=np.uint64)
        keys = pool[rng.integers(0, distinct, size=n)]
    else:
        keys = rng.integers(0, 1 << min(end_bit, 63), size=n, dtype=np.uint64)
        if end_bit == 64:
            keys |= rng.integers(0, 2, size=n, dtype=np.uint64) << np.uint64(63)
    vals = np.arange(n, dtype=np.int32)
    order = np.argsort(keys, kind="stable")
    k = torch.from_numpy(keys.view(np.int64).copy()).to(cuda)
    v = torch.from_numpy(vals.copy()).to(cuda)
    sk, sv, status = _C.sort_pairs(k, v, end_bit)
    assert int(status.item()) == 0
    np.testing.assert_array_equal(u64(sk), keys[order])
    np.testing.assert_array_equal(sv.cpu().numpy(), vals[order])
    if n <= 100_000:
        ok, ov = oracle.sort_pairs_u64(keys, vals)
        np.testing.assert_array_equal(ok, keys[order])
        np.testing.assert_array_equal(ov, vals[order])


def test_sort_empty_and_zero_bits(cuda):
    import torch
    from trigrad_amd import _C
    k = torch.empty((0,), dtype=torch.int64, device=cuda)
    v = torch.empty((0,), dtype=torch.int32, device=cuda)
    sk, sv, status = _C.sort_pairs(k, v, 64)
    assert sk.numel() == 0 and sv.numel() == 0
    k = torch.tensor([5, 3, 9], dtype=torch.int64, device=cuda)
    v = torch.tensor([0, 1, 2], dtype=torch.int32, device=cuda)
    sk, sv, _ = _C.sort_pairs(k, v, 0)  # no key bits: the identity
    assert sk.tolist() == [5, 3, 9] and sv.tolist() == [0, 1, 2]


def test_tile_ranges_with_empty_tiles(cuda, oracle):
    import torch
    from trigrad_amd import _C
    tiles = np.array([2, 2, 2, 5, 9, 9], dtype=np.uint64)
    keys = (tiles << np.uint64(32)) | np.arange(6, dtype=np.uint64)
    t = torch.from_numpy(keys.view(np.int64)).to(cuda)
    got = _C.tile_ranges(t, 12).cpu().numpy()
    np.testing.assert_array_equal(got, np.searchsorted(tiles, np.arange(13)))
    np.testing.assert_array_equal(got, oracle.tile_ranges(keys, 12))
    empty = _C.tile_ranges(torch.empty((0,), dtype=torch.int64, device=cuda), 7).cpu().numpy()
    np.testing.assert_array_equal(empty, np.zeros(8, np.int32))


def test_out_of_range_indices_are_skipped(cuda):
    """A triangle naming a vertex outside [0, V) counts no tiles instead of being read."""
    import torch
    from trigrad_amd import _C
    import scenes as S
    s = S.random_soup(10, 64, 64, seed=3)
    idx = s["indices"].copy()
    idx[4, 1] = 10_000
    idx[7, 0] = -1
    d = to_device(s, cuda)
    counts = _C.bin_count(d["vertices"], torch.from_numpy(idx).to(cuda), 64, 64, 16, 16).cpu().numpy()
    assert counts[4] == 0 and counts[7] == 0 and (np.delete(counts, [4, 7]) > 0).all()


def _tile_list_case(n, n_tiles, rng, depth_pool=None, skew=None):
    """Random (tile << 32 | depth bits) keys; skew: a share of the keys goes to one tile (a long list)."""
    tiles = rng.integers(0, n_tiles, size=n, dtype=np.uint64)
    if skew:
        tiles[rng.random(n) < skew] = np.uint64(n_tiles // 2)
    if depth_pool:
        depth = rng.integers(0, 1 << 32, size=depth_pool, dtype=np.uint64)[rng.integers(0, depth_pool, size=n)]
    else:
        depth = rng.integers(0, 1 << 32, size=n, dtype=np.uint64)
    return (tiles << np.uint64(32)) | depth


@pytest.mark.parametrize("n,n_tiles,depth_pool,skew", [
    (1, 1, None, None), (2, 7, None, None), (300, 1, None, None), (5000, 256, None, None), (70_000, 300, 3, None),
    (200_000, 8160, None, None), (200_000, 8160, 50, 0.02),       # one list of about 4000 entries among short ones
    (300_000, 97, None, None),                                    # every list between 2048 and 4096 entries
    (400_000, 64, None, None), (700_000, 128, 1000, None),        # 6250 and 5500 entries a list
    (60_000, 3, None, None), (50_000, 5, 2, 0.9),                 # lists longer than the LDS holds; few distinct depths
    (3_000_000, 8160, None, None), (5_000_017, 1024, None, 0.001),  # more sort tiles than fit the device at once
])
def test_sort_tile_lists_matches_stable_sort(n, n_tiles, depth_pool, skew, cuda):
    """The tile-list sort (tile bits through memory, depth bits per tile in LDS) against numpy's stable argsort
    of the whole key, and its ranges against searchsorted."""
    import torch
    from trigrad_amd import _C
    rng = np.random.default_rng(n + n_tiles)
    keys = _tile_list_case(n, n_tiles, rng, depth_pool, skew)
    vals = np.arange(n, dtype=np.int32)
    order = np.argsort(keys, kind="stable")
    k = torch.from_numpy(keys.view(np.int64).copy()).to(cuda)
    v = torch.from_numpy(vals.copy()).to(cuda)
    sk, sv, status, offsets = _C.sort_tile_lists(k, v, n_tiles)
    assert int(status.item()) == 0
    np.testing.assert_array_equal(u64(sk), keys[order])
    np.testing.assert_array_equal(sv.cpu().numpy(), vals[order])
    np.testing.assert_array_equal(offsets.cpu().numpy(), np.searchsorted(keys[order] >> np.uint64(32), np.arange(n_tiles + 1)))


def test_sort_tile_lists_uniform_digits_and_empty(cuda):
    """Depth words that differ in one byte only (three of the four passes are left out), equal keys, no keys."""
    import torch
    from trigrad_amd import _C
    rng = np.random.default_rng(3)
    for byte in range(4):
        n, T = 40_000, 50
        depth = np.uint64(0x3A5C77E1) & ~np.uint64(0xFF << (8 * byte)) | (rng.integers(0, 256, size=n, dtype=np.uint64) << np.uint64(8 * byte))
        keys = (rng.integers(0, T, size=n, dtype=np.uint64) << np.uint64(32)) | depth
        order = np.argsort(keys, kind="stable")
        sk, sv, status, offsets = _C.sort_tile_lists(torch.from_numpy(keys.view(np.int64).copy()).to(cuda),
                                                     torch.arange(n, dtype=torch.int32, device=cuda), T)
        np.testing.assert_array_equal(u64(sk), keys[order])
        np.testing.assert_array_equal(sv.cpu().numpy(), order.astype(np.int32))
    keys = np.full(9000, (np.uint64(3) << np.uint64(32)) | np.uint64(77), dtype=np.uint64)
    sk, sv, status, offsets = _C.sort_tile_lists(torch.from_numpy(keys.view(np.int64).copy()).to(cuda),
                                                 torch.arange(9000, dtype=torch.int32, device=cuda), 6)
    np.testing.assert_array_equal(sv.cpu().numpy(), np.arange(9000, dtype=np.int32))
    assert offsets.tolist() == [0, 0, 0, 0, 9000, 9000, 9000]
    sk, sv, status, offsets = _C.sort_tile_lists(torch.empty((0,), dtype=torch.int64, device=cuda),
                                                 torch.empty((0,), dtype=torch.int32, device=cuda), 300)
    assert sk.numel() == 0 and int(status.item()) == 0 and offsets.tolist() == [0] * 301


def test_frame_route_with_more_than_65536_tiles(cuda, oracle):
    """Three tile passes (2x2 tiles of a 600x500 image: 75 000 tiles): the emission counts no digits, the sort
    makes its own histogram; results as the stage-by-stage route gives them."""
    from trigrad_amd import _C
    import scenes as S
    scene = S.random_soup(300, 600, 500, seed=12, sigma_px=14.0, varying_w=True)
    W, H, tw, th = 600, 500, 2, 2
    d = to_device(scene, cuda)
    T = _C.num_tiles(W, H, tw, th)
    assert T > 65536
    em = oracle.bin_emit(scene["vertices"], scene["indices"], W, H, tw, th)
    want_keys, want_vals = oracle.sort_pairs_u64(em["keys64"], em["tri"])
    setup = _C.bin_setup(d["vertices"], d["indices"], W, H, tw, th)
    K = int(setup["total_and_status"][0].item())
    assert K == em["keys64"].shape[0]
    fkeys, fids, fstatus, foffsets = _C.build_tile_lists(setup, K)
    np.testing.assert_array_equal(u64(fkeys), want_keys)
    np.testing.assert_array_equal(fids.cpu().numpy(), want_vals)
    np.testing.assert_array_equal(foffsets.cpu().numpy(), oracle.tile_ranges(want_keys, T))
    # the one-call binning with more than 256 tile columns: plain tile ids in the keys, the sort counts its own digits
    assert _C.bin_frame_supported(d["vertices"], W, H, tw, th)
    binned = _C.bin_frame(d["vertices"], d["indices"], W, H, tw, th)
    assert int(binned["total_and_status"][0].item()) == K and int(binned["total_and_status"][1].item()) == 0
    np.testing.assert_array_equal(np.sort(u64(binned["keys"][:K])), np.sort(em["keys64"]))
    fkeys, fids, fstatus, foffsets = _C.build_frame_lists(binned, K)
    assert int(fstatus.item()) == 0
    np.testing.assert_array_equal(u64(fkeys), want_keys)
    np.testing.assert_array_equal(fids.cpu().numpy(), want_vals)
    np.testing.assert_array_equal(foffsets.cpu().numpy(), oracle.tile_ranges(want_keys, T))


def test_one_frame_state_serves_two_sorting_calls(cuda):
    """tg_build_tile_lists twice on the state of one tg_bin_setup, with more sort tiles than fit the device at once
    (ticketed tile numbers): the second call finds its tickets at zero again and gives the same lists."""
    import torch
    from trigrad_amd import _C
    import scenes as S
    scene = S.config(3, with_target=False)
    W, H = scene["width"], scene["height"]
    d = to_device(scene, cuda)
    setup = _C.bin_setup(d["vertices"], d["indices"], W, H, 16, 16)
    K = int(setup["total_and_status"][0].item())
    assert K > 3_200_000
    first = [t.clone() for t in _C.build_tile_lists(setup, K)]
    second = _C.build_tile_lists(setup, K)
    assert int(first[2].item()) == 0 and int(second[2].item()) == 0
    for a, b in zip(first, second):
        assert torch.equal(a, b)
    skeys = u64(first[0])
    assert (np.diff(skeys.astype(np.uint64).view(np.int64)) >= 0).all()


def test_key_buffers_smaller_than_the_frame_needs(cuda, oracle):
    """tg_bin_frame with a key capacity below K: K comes back exact, the keys that fit are the first ones of the emission
    order, nothing is written behind the capacity; and a frame whose guess of K was too small is binned again."""
    import torch
    import trigrad_amd
    from trigrad_amd import _C
    import scenes as S
    scene = S.random_soup(900, 200, 150, seed=21, sigma_px=9.0, varying_w=True)
    W, H, tw, th = 200, 150, 16, 16
    d = to_device(scene, cuda)
    em = oracle.bin_emit(scene["vertices"], scene["indices"], W, H, tw, th)
    K = em["keys64"].shape[0]
    full = _C.bin_frame(d["vertices"], d["indices"], W, H, tw, th, capacity=K + 100)
    assert int(full["total_and_status"][0].item()) == K
    capacity = K // 3
    small = _C.bin_frame(d["vertices"], d["indices"], W, H, tw, th, capacity=capacity)
    assert small["keys"].numel() == capacity
    assert int(small["total_and_status"][0].item()) == K and int(small["total_and_status"][1].item()) == 0
    assert torch.equal(small["keys"], full["keys"][:capacity]) and torch.equal(small["values"], full["values"][:capacity])
    np.testing.assert_array_equal(full["values"][:K].cpu().numpy(), em["tri"])
    with pytest.raises(ValueError):
        _C.build_frame_lists(small, K)
    # the whole frame with a guess of K that is far too small: the same image as with a good one
    good = trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, tw, th, 1 / 256, False, False, -1)[0]
    _C._key_count_hint[cuda.index] = 7
    again = trigrad_amd.render(d["vertices"], d["indices"], d["colors"], d["opacities"], W, H, tw, th, 1 / 256, False, False, -1)[0]
    assert torch.equal(good, again)
    assert _C._key_count_hint[cuda.index] == K
