"""CPU-only checks of the boundary: the shared library loads and exports every
entry point declared in include/trigrad_hip.h, rejects bad arguments before
touching a device, and the Python layer raises the reference's exceptions."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_entry_points():
    text = open(os.path.join(ROOT, "include", "trigrad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tg_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("bits", [32, 64])
def test_library_exports_every_declared_entry_point(bits):
    """Both builds of the library (float, and double = the reference's DOUBLE_PRECISION)."""
    from trigrad_amd import _lib
    lib = _lib.load(bits)
    names = _declared_entry_points()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/trigrad_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "trigrad_amd/_lib.py must declare exactly the header's entry points"
    assert lib.tg_version() == 1
    assert lib.tg_precision_bits() == bits


@pytest.mark.parametrize("bits", [32, 64])
def test_host_side_helpers_and_argument_rejection(bits):
    from trigrad_amd import _lib
    lib = _lib.load(bits)
    assert lib.tg_num_tiles(1920, 1080, 16, 16) == 120 * 68
    assert lib.tg_num_tiles(50, 50, 4, 4) == 13 * 13
    assert lib.tg_num_tiles(0, 10, 16, 16) == 0
    assert lib.tg_scan_workspace_bytes(0) > 0 and lib.tg_scan_workspace_bytes(10 ** 6) < 10 ** 5
    assert lib.tg_sort_workspace_bytes(1 << 30) == 0  # more pairs than the 30-bit look-back counters hold
    assert lib.tg_sort_workspace_bytes(10 ** 6) > 0
    # rejected before any device work: negative sizes, null pointers, oversized tiles
    assert lib.tg_bin_count(None, 0, None, -1, 64, 64, 16, 16, None, None) == -1
    assert b"tg_bin_count" in lib.tg_last_error()
    assert lib.tg_bin_count(None, 3, None, 5, 64, 64, 16, 16, None, None) == -1
    assert lib.tg_bin_count(None, 0, None, 0, 64, 64, 16, 16, None, None) == 0  # nothing to do
    assert lib.tg_scan_exclusive_u32(None, None, 8, None, None, 0, None, 256, 0, None, None) == -1
    res = C.c_int(7)
    assert lib.tg_sort_pairs_u64_u32(None, None, None, None, 1 << 31, 64, None, 0, None, C.byref(res), None) == -1
    assert lib.tg_tile_ranges(None, 5, 10, None, None) == -1
    assert lib.tg_render_forward(*([None] * 7), 64, 64, 64, 32, 0.0, 0, 1, *([None] * 12)) == -1
    assert b"tile_w*tile_h" in lib.tg_last_error()
    assert lib.tg_render_forward(*([None] * 7), 64, 64, 16, 16, 0.0, 0, 0, *([None] * 12)) == -1
    assert b"max_layers" in lib.tg_last_error()
    assert lib.tg_render_backward(*([None] * 17), 64, 64, 16, 16, 0.0, 0, 1, None, None, None, 4, 3, 1, None) == -1
    assert lib.tg_split_gradient_block(None, 5, None, None, None, None) == -1 and b"null pointer" in lib.tg_last_error()
    assert lib.tg_split_gradient_block(None, -1, None, None, None, None) == -1
    assert lib.tg_split_gradient_block(None, 0, None, None, None, None) == 0
    assert lib.tg_hit_mask_words(6400, 64, 64, 16, 16) == 16 + (100 + 16 + 1) * 256  # a word per workgroup, then the chunks
    assert lib.tg_list_bound_words(6400, 16) == 25 + 16 + 1
    assert lib.tg_list_bounds(None, 0, None, 0, None, None, None, 0, None, None, None, None) == -1
    # the frame's two calls and the tile-list sort
    assert lib.tg_bin_setup_workspace_bytes(10 ** 6, 1920, 1080, 16, 16) % 256 == 0
    assert 0 < lib.tg_bin_setup_workspace_bytes(0, 64, 64, 16, 16) < 10 ** 4
    assert lib.tg_bin_setup_workspace_bytes(-1, 64, 64, 16, 16) == 0
    assert lib.tg_bin_setup(None, 0, None, 5, 64, 64, 16, 16, None, None, None, 0, None, None, 0, None) == -1
    assert b"tg_bin_setup" in lib.tg_last_error()
    assert lib.tg_build_tile_lists_workspace_bytes(10 ** 6, 8160) > 0 and lib.tg_build_tile_lists_workspace_bytes(1 << 30, 8160) == 0
    assert lib.tg_tile_list_sort_workspace_bytes(10 ** 6, 0) == 0
    res = C.c_int(7)
    assert lib.tg_build_tile_lists(None, None, 5, 10, 0, None, None, 64, 64, 16, 16, None, None, None, None, None, None, 0, None, 0,
                                   C.byref(res), None) == -1
    assert lib.tg_sort_tile_lists(None, None, None, None, 10, 0, None, None, 0, None, C.byref(res), None) == -1
    # the frame's binning without a wait for the host (float build) and the sort of its keys
    assert lib.tg_bin_frame_supported(1920, 1080, 16, 16) == (1 if bits == 32 else 0)
    assert lib.tg_bin_frame_supported(1 << 14, 1 << 14, 2, 2) == 0  # more than 2^21 tiles
    assert lib.tg_bin_frame_workspace_bytes(10 ** 6, 3 * 10 ** 6, 1920, 1080, 16, 16) % 256 == 0
    assert lib.tg_bin_frame_workspace_bytes(10 ** 6, 3 * 10 ** 6, 1920, 1080, 16, 16) > 52 * 10 ** 6  # records and offsets of the triangles
    assert lib.tg_bin_frame_workspace_bytes(-1, 0, 64, 64, 16, 16) == 0
    assert lib.tg_bin_frame(None, 0, None, 5, 64, 64, 16, 16, None, None, 0, None, None, 0, 1, None, 0, None, None) == -1
    assert b"tg_bin_frame" in lib.tg_last_error()
    assert lib.tg_build_frame_lists_workspace_bytes(10 ** 6, 120, 68) > 0 and lib.tg_build_frame_lists_workspace_bytes(1 << 30, 120, 68) == 0
    assert lib.tg_build_frame_lists(None, 1, 10, 120, 68, None, None, None, None, None, None, 0, None, C.byref(res), None) == -1
    lib.tg_force_tickets(1)
    lib.tg_force_tickets(0)
    assert lib.tg_scan_noalloc_max_n() == 1 << 24
    assert lib.tg_scan_exclusive_u32_noalloc(None, None, (1 << 24) + 1, None, None, 256, 0, None, None) == -1
    with pytest.raises(RuntimeError, match="tg_bin_count failed with code -1"):
        _lib.check(lib.tg_bin_count(None, 0, None, -1, 64, 64, 16, 16, None, None), "tg_bin_count", bits)


def test_python_entry_point_errors_without_gpu():
    """Error behaviour of reference src/trigrad/util.py:7-14 and wrapper.py:143-144."""
    import torch
    import trigrad_amd
    assert trigrad_amd.precision == torch.float32
    v = torch.zeros((3, 4)); i = torch.zeros((1, 3), dtype=torch.int32); c = torch.zeros((3, 3)); o = torch.zeros(3)
    with pytest.raises(TypeError, match="vertices must be on cuda, but got cpu"):
        trigrad_amd.render(v, i, c, o)
    with pytest.raises(ValueError, match="tile_width \\* tile_height must be <= 1024"):
        trigrad_amd.render(v, i, c, o, 64, 64, 33, 32)
    from trigrad_amd.util import create_check
    chk = create_check("cpu", torch.float32)
    chk(v, "v", (3, 4))
    with pytest.raises(ValueError, match="v must be of shape \\(3, 3\\)"):
        chk(v, "v", (3, 3))
    with pytest.raises(TypeError, match="v must be of type torch.float64"):
        chk(v, "v", (3, 4), torch.float64)
    chk(o, "o", 3)  # a bare int is promoted to a 1-tuple


def test_product_does_not_reach_into_the_oracle():
    """Nothing under trigrad_amd/ may import, include or load the oracle."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "trigrad_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_key_bits():
    from trigrad_amd import _C
    assert _C.key_bits(8160) == 45 and _C.key_bits(4096) == 44 and _C.key_bits(256) == 40 and _C.key_bits(1) == 33


def test_status_word_check_raises_without_a_gpu():
    """The check the frame makes of the list kernels' status word, on a host tensor."""
    import torch
    from trigrad_amd import _C
    _C.StatusCheck(torch.zeros((1,), dtype=torch.int32)).verify()
    bad = _C.StatusCheck(torch.tensor([1], dtype=torch.int32), what="tg_build_tile_lists")
    with pytest.raises(RuntimeError, match="tg_build_tile_lists: look-back wait timed out"):
        bad.verify()
    bad.verify()  # reported once
    _C._pending_checks.append(_C.StatusCheck(torch.tensor([1], dtype=torch.int32)))
    with pytest.raises(RuntimeError, match="look-back wait timed out"):
        _C.verify_finished_frames()
    _C.verify_finished_frames()
    assert _C._pending_checks == []
