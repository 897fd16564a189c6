"""Native surface of the renderer: the functions the reference exports from its
pybind module (src/trigrad/module.cu:8-21, render.h) with the same names and
argument order, implemented by calling the C ABI of libtrigrad_hip.so on the
current torch stream.  torch is used for device memory and streams only.

`render_forward` runs the frame's route:
    bin_frame (count + scan, then key emission that reads K on the device) -> (K to the host, bary matrices meanwhile)
    -> build_frame_lists (two passes over the tile bits through memory, depth bits and tile ranges per tile)
    -> forward kernel
The double build and frames with more than 2^21 tiles go through bin_setup + build_tile_lists, and the single stages
(bin_count, scan_exclusive, bin_emit, sort_pairs, tile_ranges) are exposed as functions for tests and benchmarks.
"""
import ctypes as C
import threading

import torch

import os

from . import _lib

# The reference fixes its scalar type when the extension is compiled (util.h:5-20, module.cu:17-21).
# Here both builds of the library are present; TRIGRAD_PRECISION=float64 (or set_precision) selects the
# double one, which the entry points then expect, like a reference built with DOUBLE_PRECISION.
precision = torch.float64 if os.environ.get("TRIGRAD_PRECISION", "float32").lower() in ("float64", "double", "64") else torch.float32


def _bits(t):
    """Which library serves tensor t: the double build for float64 data, the float build otherwise."""
    return 64 if t.dtype == torch.float64 else 32

STAGE_KEYS = ("init", "per_tile_lists", "sorting", "bary_transforms", "rasterization")  # render.cu:723-747


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _raw_stream(dev):
    """The hipStream_t of the device's current torch stream, as an int (no Stream object is made)."""
    return torch._C._cuda_getCurrentRawStream(dev.index)


def _stream(t):
    return C.c_void_p(_raw_stream(t.device))


class _on_device:
    """`with _on_device(dev)` that costs nothing when dev is already current (the stages of a frame nest)."""

    def __init__(self, device):
        self.guard = None if torch.cuda.current_device() == device.index else torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _need_cuda(*tensors):
    for t in tensors:
        if t.device.type != "cuda":
            raise TypeError(f"expected a cuda tensor, got {t.device.type}")


def num_tiles(width, height, tile_width, tile_height):
    return int(_lib.load().tg_num_tiles(width, height, tile_width, tile_height))


def key_bits(n_tiles):
    """Significant bits of a (tile << 32 | depth) key."""
    return 32 + max(1, int(n_tiles - 1).bit_length())


# ---- stages ------------------------------------------------------------------------

def bin_count(vertices, indices, width, height, tile_width, tile_height):
    """Per-triangle tile-overlap counts, (M,) int32."""
    _need_cuda(vertices, indices)
    lib = _lib.load(_bits(vertices))
    M = indices.shape[0]
    counts = torch.empty((M,), dtype=torch.int32, device=vertices.device)
    with _on_device(vertices.device):
        _lib.check(lib.tg_bin_count(_ptr(vertices), vertices.shape[0], _ptr(indices), M, width, height, tile_width, tile_height,
                                    _ptr(counts), _stream(vertices)), "tg_bin_count", _bits(vertices))
    return counts


OWNER_STRIDE = 256  # keys per workgroup of the emission kernel
MAX_SAVED_LAYERS = 32  # TG_MAX_SAVED_LAYERS of the C header
# With per_pixel_sort and max_layers <= MAX_SAVED_LAYERS the forward pass saves every pixel's
# blend order (16-bit planes, see saved_blend_order) and the backward pass walks it in reverse instead of
# selecting the fragments again.  False trades the memory for the re-selection.
SAVE_BLEND_ORDER = True
# Without per_pixel_sort the forward pass saves which list entries cover which pixel (one bit per pair it
# looked at) and the backward pass reads that back instead of repeating the inside tests.
SAVE_HIT_MASKS = True
# With per_pixel_sort and tile lists of at least this many entries on average, depth bounds of the lists are
# computed (one more pass over the keys) so that the selection can stop before the end of a list.
EARLY_STOP_MIN_AVG_LIST = 512
# Binning (count, scan, key emission) in one launch where the library takes the frame (tg_bin_frame_supported);
# False: tg_bin_setup + tg_build_tile_lists, the route of the double build and of frames with more than 2^21 tiles.
FUSED_BINNING = True


def _as_int32(v):
    """A uint32 as the int32 it reads back as."""
    return v - (1 << 32) if v >= (1 << 31) else v


def scan_exclusive(counts, out=None, heads=None):
    """Exclusive prefix sum of an int32 tensor -> (offsets, total (1,) int32, status (1,) int32).

    total and status are the two halves of one (2,) tensor (`total._base`).

    heads (optional int32 tensor): receives, for every multiple of OWNER_STRIDE
    below the total, the index of the element that owns that output position.
    """
    _need_cuda(counts)
    lib = _lib.load()
    n = counts.numel()
    dev = counts.device
    out = torch.empty_like(counts) if out is None else out
    pair = torch.empty((2,), dtype=torch.int32, device=dev)  # one allocation, so that one copy brings both to the host
    total, status = pair[:1], pair[1:]
    ws_bytes = int(lib.tg_scan_workspace_bytes(n))
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    with _on_device(dev):
        _lib.check(lib.tg_scan_exclusive_u32(_ptr(counts), _ptr(out), n, _ptr(total), _ptr(ws), ws_bytes, _ptr(status), OWNER_STRIDE,
                                             0 if heads is None else heads.numel(), _ptr(heads), _stream(counts)),
                   "tg_scan_exclusive_u32")
    return out, total, status


def owner_heads_for(n_triangles, device):
    """Buffer for the scan's `heads` output; covers up to 8 keys per triangle (beyond that the emission searches)."""
    return torch.empty(((8 * n_triangles + 65536) // OWNER_STRIDE,), dtype=torch.int32, device=device)


def bin_emit(vertices, indices, tri_offsets, n_keys, width, height, tile_width, tile_height, heads=None):
    """-> (keys (K,) int64 holding uint64 bit patterns, payload (K,) int32) in emission order.

    float64 vertices: keys has 2K entries, the depth keys (all 64 bits) followed by the tile ids."""
    _need_cuda(vertices, indices, tri_offsets)
    lib = _lib.load(_bits(vertices))
    dev = vertices.device
    keys = torch.empty((n_keys * (2 if _bits(vertices) == 64 else 1),), dtype=torch.int64, device=dev)
    payload = torch.empty((n_keys,), dtype=torch.int32, device=dev)
    with _on_device(dev):
        _lib.check(lib.tg_bin_emit(_ptr(vertices), vertices.shape[0], _ptr(indices), indices.shape[0], width, height, tile_width,
                                   tile_height, _ptr(tri_offsets), n_keys, _ptr(heads), 0 if heads is None else heads.numel(),
                                   _ptr(keys), _ptr(payload), _stream(vertices)), "tg_bin_emit", _bits(vertices))
    return keys, payload


def sort_pairs(keys, values, end_bit=64):
    """Stable sort of (uint64 key, 32-bit value) pairs on key bits [0, end_bit).

    The inputs are used as scratch (their contents are undefined afterwards).
    -> (sorted_keys, sorted_values, status (1,) int32)
    """
    _need_cuda(keys, values)
    lib = _lib.load()
    n = keys.numel()
    dev = keys.device
    keys_alt = torch.empty_like(keys)
    values_alt = torch.empty_like(values)
    status = torch.empty((1,), dtype=torch.int32, device=dev)  # the library writes it in every path
    ws_bytes = int(lib.tg_sort_workspace_bytes(n))
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    in_alt = C.c_int(0)
    with _on_device(dev):
        _lib.check(lib.tg_sort_pairs_u64_u32(_ptr(keys), _ptr(values), _ptr(keys_alt), _ptr(values_alt), n, end_bit, _ptr(ws),
                                             ws_bytes, _ptr(status), C.byref(in_alt), _stream(keys)), "tg_sort_pairs_u64_u32")
    if in_alt.value:
        return keys_alt, values_alt, status
    return keys, values, status


def tile_ranges(sorted_keys, n_tiles):
    """offsets (T+1,) int32 of the tile segments of a sorted key array."""
    _need_cuda(sorted_keys)
    lib = _lib.load()
    offsets = torch.empty((n_tiles + 1,), dtype=torch.int32, device=sorted_keys.device)
    with _on_device(sorted_keys.device):
        _lib.check(lib.tg_tile_ranges(_ptr(sorted_keys), sorted_keys.numel(), n_tiles, _ptr(offsets), _stream(sorted_keys)),
                   "tg_tile_ranges")
    return offsets


def sort_tile_lists(keys, values, n_tiles):
    """(tile << 32 | depth bits, triangle) pairs -> (sorted_keys, sorted_values, status (1,) int32, offsets (T+1,) int32).

    Same result as sort_pairs on key_bits(n_tiles) followed by tile_ranges; the passes over the depth bits run
    per tile inside a workgroup.  The inputs are used as scratch."""
    _need_cuda(keys, values)
    lib = _lib.load()
    n = keys.numel()
    dev = keys.device
    keys_alt = torch.empty_like(keys)
    values_alt = torch.empty_like(values)
    status = torch.empty((1,), dtype=torch.int32, device=dev)
    offsets = torch.empty((n_tiles + 1,), dtype=torch.int32, device=dev)
    ws_bytes = int(lib.tg_tile_list_sort_workspace_bytes(n, n_tiles))
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    in_alt = C.c_int(0)
    with _on_device(dev):
        _lib.check(lib.tg_sort_tile_lists(_ptr(keys), _ptr(values), _ptr(keys_alt), _ptr(values_alt), n, n_tiles, _ptr(offsets),
                                          _ptr(ws), ws_bytes, _ptr(status), C.byref(in_alt), _stream(keys)), "tg_sort_tile_lists")
    if in_alt.value:
        return keys_alt, values_alt, status, offsets
    return keys, values, status, offsets


RECORD_SCALARS = 12  # TG_RECORD_SCALARS of the C header


def bin_setup(vertices, indices, width, height, tile_width, tile_height, with_heads=True):
    """Counts, scans and prepares the emission in one pass over the triangles.

    -> dict(tri_offsets (M,) int32, records (M, 12), total_and_status (2,) int32, heads, frame, geometry)"""
    _need_cuda(vertices, indices)
    bits = _bits(vertices)
    lib = _lib.load(bits)
    dev = vertices.device
    M = indices.shape[0]
    tri_offsets = torch.empty((M,), dtype=torch.int32, device=dev)
    records = torch.empty((M, RECORD_SCALARS), dtype=vertices.dtype, device=dev)
    pair = torch.empty((2,), dtype=torch.int32, device=dev)
    heads = owner_heads_for(M, dev) if with_heads else None
    frame_bytes = int(lib.tg_bin_setup_workspace_bytes(M, width, height, tile_width, tile_height))
    frame = torch.empty((frame_bytes,), dtype=torch.uint8, device=dev)
    with _on_device(dev):
        _lib.check(lib.tg_bin_setup(_ptr(vertices), vertices.shape[0], _ptr(indices), M, width, height, tile_width, tile_height,
                                    _ptr(tri_offsets), _ptr(records), _ptr(pair), 0 if heads is None else heads.numel(), _ptr(heads),
                                    _ptr(frame), frame_bytes, _stream(vertices)), "tg_bin_setup", bits)
    return dict(tri_offsets=tri_offsets, records=records, total_and_status=pair, heads=heads, frame=frame,
                geometry=(width, height, tile_width, tile_height), bits=bits)


_key_count_hint = {}  # device index -> K of the device's last frame


def prepare_tile_lists(setup):
    """Buffers for build_tile_lists, allocated before K is known: for as many keys as the device's last frame had
    plus an eighth.  The host has nothing to do while it waits for K, and every allocation made after K has
    arrived is time the device idles.  None without a last frame (or for the double build)."""
    hint = _key_count_hint.get(setup["records"].device.index)
    if hint is None or setup["bits"] != 32:
        return None
    capacity = hint + hint // 8 + 1024
    if int(_lib.load(32).tg_build_tile_lists_workspace_bytes(capacity, num_tiles(*setup["geometry"]))) == 0:
        return None  # more keys than the sort takes: leave it to the call that knows K
    return _tile_list_buffers(setup, capacity)


def _tile_list_buffers(setup, capacity):
    lib = _lib.load(setup["bits"])
    dev = setup["records"].device
    T = num_tiles(*setup["geometry"])
    ws_bytes = int(lib.tg_build_tile_lists_workspace_bytes(capacity, T))
    return dict(capacity=capacity, ws_bytes=ws_bytes,
                keys=torch.empty((capacity,), dtype=torch.int64, device=dev),
                values=torch.empty((capacity,), dtype=torch.int32, device=dev),
                keys_alt=torch.empty((capacity,), dtype=torch.int64, device=dev),
                values_alt=torch.empty((capacity,), dtype=torch.int32, device=dev),
                offsets=torch.empty((T + 1,), dtype=torch.int32, device=dev),
                status=torch.empty((1,), dtype=torch.int32, device=dev),
                ws=torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev))


def build_tile_lists(setup, n_keys, emit_only=False, prepared=None):
    """bin_setup's result + K -> (sorted_keys, sorted_ids, status (1,) int32, offsets (T+1,) int32);
    emit_only: (keys, ids, status, None) in emission order (float64: 2K keys, depth keys then tile ids).
    prepared: prepare_tile_lists' buffers, used if they hold n_keys keys."""
    bits = setup["bits"]
    lib = _lib.load(bits)
    records, tri_offsets, heads, frame = setup["records"], setup["tri_offsets"], setup["heads"], setup["frame"]
    width, height, tile_width, tile_height = setup["geometry"]
    dev = records.device
    _key_count_hint[dev.index] = n_keys
    if emit_only or bits != 32:
        keys = torch.empty((n_keys * (2 if bits == 64 else 1),), dtype=torch.int64, device=dev)
        values = torch.empty((n_keys,), dtype=torch.int32, device=dev)
        status = torch.empty((1,), dtype=torch.int32, device=dev)
        keys_alt = values_alt = offsets = ws = None
        ws_bytes = 0
        if not emit_only:
            T = num_tiles(width, height, tile_width, tile_height)
            keys_alt, values_alt = torch.empty_like(keys), torch.empty_like(values)
            offsets = torch.empty((T + 1,), dtype=torch.int32, device=dev)
            ws_bytes = int(lib.tg_build_tile_lists_workspace_bytes(n_keys, T))
            ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    else:
        b = prepared if prepared is not None and n_keys <= prepared["capacity"] else _tile_list_buffers(setup, n_keys)
        keys, values, keys_alt, values_alt = b["keys"], b["values"], b["keys_alt"], b["values_alt"]
        offsets, status, ws, ws_bytes = b["offsets"], b["status"], b["ws"], b["ws_bytes"]
    in_alt = C.c_int(0)
    with _on_device(dev):
        _lib.check(lib.tg_build_tile_lists(_ptr(records), _ptr(tri_offsets), tri_offsets.numel(), n_keys,
                                           0 if heads is None else heads.numel(), _ptr(heads), _ptr(frame), width, height,
                                           tile_width, tile_height, _ptr(keys), _ptr(values), _ptr(keys_alt), _ptr(values_alt),
                                           _ptr(offsets), _ptr(ws), ws_bytes, _ptr(status), int(bool(emit_only)), C.byref(in_alt),
                                           _stream(records)), "tg_build_tile_lists", bits)
    if in_alt.value:
        keys, values = keys_alt, values_alt
    if keys.numel() != n_keys * (2 if bits == 64 else 1):
        keys, values = keys[:n_keys], values[:n_keys]  # buffers made for more keys
    return keys, values, status, offsets


# ---- the frame's route: binning in one launch -------------------------------------------------------------

_frame_states = {}  # (device index, stream) -> dict(frame, epoch): the state tg_bin_frame keeps between calls
_frame_lock = threading.Lock()
_FRAME_TAIL = 256  # bytes behind the library's frame state: K and the status word of the binning


def saved_blend_order(fragments, offsets, tile_width, tile_height):
    """(max_layers, H, W) int32 list positions, relative to the tile's start, out of the planes the forward pass
    saved: the low halves in the first max_layers planes, the high halves (written only in tiles whose list holds
    more than 65535 entries) in the rest.  Layer k of a pixel means something for k < ends only."""
    layers, height, width = fragments.shape[0] // 2, fragments.shape[1], fragments.shape[2]
    tiles_x, tiles_y = -(-width // tile_width), -(-height // tile_height)
    lengths = (offsets[1:] - offsets[:-1]).reshape(tiles_y, tiles_x)
    is_long = (lengths > 0xFFFF).repeat_interleave(tile_height, 0).repeat_interleave(tile_width, 1)[:height, :width]
    low = fragments[:layers].to(torch.int32) & 0xFFFF
    high = fragments[layers:].to(torch.int32) & 0xFFFF
    return torch.where(is_long[None], low | (high << 16), low)


def bin_frame_supported(vertices, width, height, tile_width, tile_height):
    """Whether tg_bin_frame takes this frame (float build, at most 2^21 tiles)."""
    return _bits(vertices) == 32 and bool(_lib.load(32).tg_bin_frame_supported(width, height, tile_width, tile_height))


def _next_frame_state(dev, need):
    """The frame state of at least `need` bytes of the device's current stream, zeroed when it is made, and the epoch of
    the call about to use it (they count up by one; a state whose epochs run out is replaced by a fresh one).  A state
    per stream: frames on one stream follow each other, frames on two streams may run at the same time."""
    key = (dev.index, _raw_stream(dev))
    with _frame_lock:
        st = _frame_states.get(key)
        if st is None or st["bytes"] < need or st["epoch"] >= 0x3FFFFFF0:
            size = need + need // 4
            st = dict(frame=torch.zeros((size + _FRAME_TAIL,), dtype=torch.uint8, device=dev), epoch=0, bytes=size)
            _frame_states[key] = st
        st["epoch"] += 1
        return st["frame"], st["bytes"], st["epoch"]


def bin_frame(vertices, indices, width, height, tile_width, tile_height, capacity=None):
    """Counts, scans and emits without a wait for the host (tg_bin_frame) into buffers for `capacity` keys (default:
    what the device's last frame needed plus an eighth, or three keys per triangle).

    -> dict(keys, values (emission order, the first min(K, capacity) valid), total_and_status (2,) int32:
    K and, if a wait expired, `epoch`; capacity, epoch, and the buffers the sort needs)"""
    _need_cuda(vertices, indices)
    lib = _lib.load(32)
    dev = vertices.device
    M = indices.shape[0]
    T = num_tiles(width, height, tile_width, tile_height)
    if capacity is None:
        hint = _key_count_hint.get(dev.index)
        capacity = hint + hint // 8 + 1024 if hint is not None else 3 * M + 65536
    capacity = max(1, min(int(capacity), (1 << 30) - 1))
    need = int(lib.tg_bin_frame_workspace_bytes(M, capacity, width, height, tile_width, tile_height))
    frame, frame_bytes, epoch = _next_frame_state(dev, need)
    pair = frame[frame_bytes:frame_bytes + 8].view(torch.int32)
    tiles = (-(-width // tile_width), -(-height // tile_height))
    ws_bytes = int(lib.tg_build_frame_lists_workspace_bytes(capacity, *tiles))
    b = dict(capacity=capacity, epoch=epoch, frame=frame, total_and_status=pair, tiles=tiles, ws_bytes=ws_bytes,
             keys=torch.empty((capacity,), dtype=torch.int64, device=dev),
             values=torch.empty((capacity,), dtype=torch.int32, device=dev),
             keys_alt=torch.empty((capacity,), dtype=torch.int64, device=dev),
             values_alt=torch.empty((capacity,), dtype=torch.int32, device=dev),
             offsets=torch.empty((T + 1,), dtype=torch.int32, device=dev),
             status=torch.empty((1,), dtype=torch.int32, device=dev),
             ws=torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=dev))
    # the sort's own histogram route (more than 256 tile columns or rows) clears its workspace itself
    zero_bytes = ws_bytes if max(tiles) <= 256 else 0
    with _on_device(dev):
        _lib.check(lib.tg_bin_frame(_ptr(vertices), vertices.shape[0], _ptr(indices), M, width, height, tile_width, tile_height,
                                    _ptr(b["keys"]), _ptr(b["values"]), capacity, _ptr(pair), _ptr(frame),
                                    frame_bytes, epoch, _ptr(b["ws"]), zero_bytes, _ptr(b["status"]), _stream(vertices)),
                   "tg_bin_frame")
    return b


def build_frame_lists(binned, n_keys):
    """bin_frame's result + K (at most its capacity) -> (sorted_keys, sorted_ids, status (1,) int32, offsets (T+1,) int32)."""
    lib = _lib.load(32)
    b = binned
    if n_keys > b["capacity"]:
        raise ValueError(f"{n_keys} keys, buffers for {b['capacity']}")
    dev = b["keys"].device
    _key_count_hint[dev.index] = n_keys
    in_alt = C.c_int(0)
    with _on_device(dev):
        _lib.check(lib.tg_build_frame_lists(_ptr(b["frame"]), b["epoch"], n_keys, *b["tiles"], _ptr(b["keys"]), _ptr(b["values"]),
                                            _ptr(b["keys_alt"]), _ptr(b["values_alt"]), _ptr(b["offsets"]), _ptr(b["ws"]),
                                            b["ws_bytes"], _ptr(b["status"]), C.byref(in_alt), _stream(b["keys"])),
                   "tg_build_frame_lists")
    keys, values = (b["keys_alt"], b["values_alt"]) if in_alt.value else (b["keys"], b["values"])
    return keys[:n_keys], values[:n_keys], b["status"], b["offsets"]


def cartesian_to_bary(vertices, indices):
    """(M,3,3) cartesian-to-barycentric matrices (reference _C.cartesian_to_bary, render.cu:697-711)."""
    _need_cuda(vertices, indices)
    lib = _lib.load(_bits(vertices))
    vertices = vertices.contiguous()
    indices = indices.contiguous()
    M = indices.shape[0]
    out = torch.empty((M, 3, 3), dtype=vertices.dtype, device=vertices.device)
    with _on_device(vertices.device):
        _lib.check(lib.tg_bary(_ptr(vertices), vertices.shape[0], _ptr(indices), M, _ptr(out), _stream(vertices)), "tg_bary", _bits(vertices))
    return out


def per_tile_lists(vertices, indices, width, height, tile_width, tile_height):
    """Binning + sort + ranges -> (sorted_ids (K,) int32, offsets (T+1,) int32, sorted_keys (K,) int64).

    Observable of the reference's per_tile_lists + sort_depth_ranges
    (render.cu:272-308).  Reads K back from the device once, like the
    reference's sum().item() (render.cu:290).
    """
    T = num_tiles(width, height, tile_width, tile_height)
    counts = bin_count(vertices, indices, width, height, tile_width, tile_height)
    heads = owner_heads_for(indices.shape[0], vertices.device)
    tri_offsets, total, status = scan_exclusive(counts, out=counts, heads=heads)
    host = total._base.cpu()  # the one device->host read of the forward pass
    K, st = int(host[0]), int(host[1])
    if st != 0:
        raise RuntimeError("tg_scan_exclusive_u32: look-back wait timed out")
    keys, payload, sort_status, offsets = emit_and_sort(vertices, indices, tri_offsets, K, T, width, height, tile_width,
                                                        tile_height, heads)
    return payload, offsets, keys, sort_status


def emit_and_sort(vertices, indices, tri_offsets, K, T, width, height, tile_width, tile_height, heads):
    """Key emission, sort and tile ranges -> (sorted_keys, sorted_ids, sort_status, offsets)."""
    keys, payload = bin_emit(vertices, indices, tri_offsets, K, width, height, tile_width, tile_height, heads)
    return sort_lists(keys, payload, K, T)


def sort_lists(keys, payload, K, T):
    """bin_emit's output -> (sorted_keys, sorted_ids, sort_status, offsets).

    float32 (K keys): one sort of (tile << 32 | depth bits).  float64 (2K keys: depth keys, then tile ids): the
    depth takes all 64 key bits, so the pairs are sorted by depth first and then, stably, by tile id;
    sorted_keys are then (tile << 32) only.
    """
    if keys.numel() == K:
        keys, payload, sort_status = sort_pairs(keys, payload, key_bits(T))
        return keys, payload, sort_status, tile_ranges(keys, T)
    depth_keys, tile_ids = keys[:K], keys[K:]
    order = torch.arange(K, dtype=torch.int32, device=keys.device)
    _, order, status1 = sort_pairs(depth_keys, order, 64)
    tile_keys, order, status2 = sort_pairs(tile_ids[order.long()], order, key_bits(T) - 32)
    sorted_keys = tile_keys << 32
    return sorted_keys, payload[order.long()], torch.maximum(status1, status2), tile_ranges(sorted_keys, T)


class _StageTimer:
    """Seconds per stage from events on the current stream (render.cu:11-49)."""

    def __init__(self, disable):
        self.disable = disable
        self.marks = []

    def start(self, name):
        if self.disable:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self.marks.append((name, ev))

    def stop(self):
        if self.disable:
            return {}
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        end.synchronize()
        evs = [e for _, e in self.marks] + [end]
        return {name: evs[k].elapsed_time(evs[k + 1]) / 1000.0 for k, (name, _) in enumerate(self.marks)}


_frame_counter = 0  # frames rendered by this process, for the messages of StatusCheck


def force_tickets(on=True):
    """Makes every kernel that waits on other workgroups number its tiles by an atomic ticket (tg_force_tickets):
    slower, and safe when other work shares the device.  Switched on by the first wait that expires."""
    for bits, lib in list(_lib._libs.items()) or [(32, _lib.load(32))]:
        lib.tg_force_tickets(1 if on else 0)
    global _tickets_forced
    _tickets_forced = bool(on)


_tickets_forced = False


class StatusCheck:
    """The status word of the kernels that wait on other workgroups (TG_STATUS_*), on its way to the host.

    The word is copied to pinned host memory behind the kernels that write it, without a wait; `verify`
    waits for that copy (long done when the backward pass or the next frame asks) and raises RuntimeError
    if a bounded wait expired, because the lists and everything rendered from them are then invalid (the
    forward kernels have filled such a frame's image with NaN).  From then on the kernels take tickets."""

    def __init__(self, status, what="tg_build_frame_lists", frame=None):
        self.what = what
        self.frame = frame
        self.checked = False
        if status.device.type == "cuda":
            self.host = torch.empty((status.numel(),), dtype=torch.int32, pin_memory=True)
            self.host.copy_(status, non_blocking=True)
            self.event = torch.cuda.Event()
            self.event.record(torch.cuda.current_stream(status.device))
        else:
            self.host = status.clone()
            self.event = None

    def ready(self):
        return self.event is None or self.event.query()

    def failed(self):
        """Waits for the word; True if a wait expired."""
        if self.event is not None:
            self.event.synchronize()
        self.checked = True
        return int(self.host.max()) != 0

    def verify(self):
        if self.checked:
            return
        if self.failed():
            force_tickets(True)
            which = "" if self.frame is None else f" of frame {self.frame}"
            raise RuntimeError(f"{self.what}: look-back wait timed out (status {self.host.tolist()}); the lists{which} are "
                               "invalid and its image is NaN.  Later frames number their tiles by ticket.")


_pending_checks = []  # status words of earlier frames that nobody has looked at yet
_pending_lock = threading.Lock()


def verify_frames(wait=True):
    """Raises RuntimeError if the lists of a frame rendered earlier are invalid because a bounded wait between
    workgroups expired (its image is then NaN).  wait=True also waits for the status words still on their way, so
    after it returns every frame rendered so far on this process is known to be good: what a caller who only
    renders forward (no backward pass, whose first step is this check) calls before it trusts a frame.
    wait=False looks only at the words that have arrived."""
    with _pending_lock:
        checks = list(_pending_checks)
        del _pending_checks[:]
    still = []
    try:
        while checks:
            check = checks.pop(0)
            if check.checked:
                continue
            if wait or check.ready():
                check.verify()
            else:
                still.append(check)
    finally:
        with _pending_lock:
            _pending_checks[:0] = still + [c for c in checks if not c.checked]


def verify_finished_frames():
    """verify_frames(wait=False): never waits."""
    verify_frames(wait=False)


def _forward_full(vertices, indices, colors, opacities, width, height, tile_width, tile_height,
                  early_stopping_threshold, disable_timing, per_pixel_sort, max_layers):
    """render_forward's eight results plus `resume` = (last, last_depth, status_check, fragments, hit_masks):
    what the backward pass needs for its reverse traversal (fragments / hit_masks are None unless the blend
    order / the hit masks were saved) and the status word of the list kernels on its way to the host."""
    _need_cuda(vertices, indices, colors, opacities)
    verify_finished_frames()
    bits = _bits(vertices)
    lib = _lib.load(bits)
    real = vertices.dtype
    timer = _StageTimer(disable_timing)
    dev = vertices.device
    with _on_device(dev):
        timer.start("init")
        vertices = vertices.contiguous()
        indices = indices.contiguous()
        colors = colors.contiguous()
        opacities = opacities.contiguous()
        image = torch.empty((height, width, 4), dtype=real, device=dev)
        depthmap = torch.empty((height, width), dtype=real, device=dev)
        final_weights = torch.empty((height, width), dtype=real, device=dev)
        ends = torch.empty((height, width), dtype=torch.int32, device=dev)
        last = torch.empty((height, width), dtype=torch.int32, device=dev)
        last_depth = torch.empty((height, width), dtype=real, device=dev) if per_pixel_sort else None
        save_order = bool(per_pixel_sort) and SAVE_BLEND_ORDER and 0 < int(max_layers) <= MAX_SAVED_LAYERS
        fragments = torch.empty((2 * int(max_layers), height, width), dtype=torch.int16, device=dev) if save_order else None

        timer.start("per_tile_lists")
        T = num_tiles(width, height, tile_width, tile_height)
        bary_transforms = None
        if FUSED_BINNING and bin_frame_supported(vertices, width, height, tile_width, tile_height):
            # count, scan and emission in one launch into buffers sized by the last frame's K; K and the status word
            # travel to pinned host memory while the device computes the bary matrices, which do not depend on K
            binned = bin_frame(vertices, indices, width, height, tile_width, tile_height)
            while True:
                host = torch.empty((2,), dtype=torch.int32, pin_memory=True)
                host.copy_(binned["total_and_status"], non_blocking=True)
                arrived = torch.cuda.Event()
                arrived.record()
                if bary_transforms is None and disable_timing:
                    bary_transforms = cartesian_to_bary(vertices, indices)
                arrived.synchronize()
                K, st = host.tolist()
                if st == _as_int32(binned["epoch"]):
                    # a workgroup gave up waiting for another (other work on the device): once more, with tickets
                    if _tickets_forced:
                        raise RuntimeError("tg_bin_frame: wait for another workgroup timed out")
                    force_tickets(True)
                    K = binned["capacity"] + 1
                if K <= binned["capacity"]:
                    break
                binned = bin_frame(vertices, indices, width, height, tile_width, tile_height,
                                   capacity=None if st == _as_int32(binned["epoch"]) else K + K // 8)
            timer.start("sorting")
            keys, sorted_ids, sort_status, offsets = build_frame_lists(binned, K)
        else:
            setup = bin_setup(vertices, indices, width, height, tile_width, tile_height)
            K, st = setup["total_and_status"].cpu().tolist()
            if st != 0:
                raise RuntimeError("tg_bin_setup: look-back wait timed out")
            keys, payload, _, _ = build_tile_lists(setup, K, emit_only=True)
            timer.start("sorting")
            if bits == 32:
                keys, sorted_ids, sort_status, offsets = sort_tile_lists(keys, payload, T)
            else:  # the double build's depth keys take 64 bits and are sorted in two rounds
                keys, sorted_ids, sort_status, offsets = sort_lists(keys, payload, K, T)
        global _frame_counter
        _frame_counter += 1
        status_check = StatusCheck(sort_status, frame=_frame_counter)
        with _pending_lock:
            _pending_checks.append(status_check)

        timer.start("bary_transforms")
        if bary_transforms is None:
            bary_transforms = cartesian_to_bary(vertices, indices)

        timer.start("rasterization")
        batch_bounds = far_start = None
        if per_pixel_sort and K >= EARLY_STOP_MIN_AVG_LIST * T:
            # long lists: depth bounds let the selection leave a list before its end
            batch_bounds = torch.empty((int(lib.tg_list_bound_words(K, T)),), dtype=real, device=dev)
            far_start = torch.empty((T,), dtype=torch.int32, device=dev)
            triangle_low = torch.empty((indices.shape[0],), dtype=real, device=dev)
            _lib.check(lib.tg_list_bounds(_ptr(vertices), vertices.shape[0], _ptr(indices), indices.shape[0], _ptr(keys),
                                          _ptr(sorted_ids), _ptr(offsets), T, _ptr(triangle_low), _ptr(batch_bounds),
                                          _ptr(far_start), _stream(vertices)), "tg_list_bounds", bits)
        hit_masks = None
        if not per_pixel_sort and SAVE_HIT_MASKS:
            words = int(lib.tg_hit_mask_words(K, width, height, tile_width, tile_height))
            hit_masks = torch.empty((words,), dtype=torch.int64, device=dev)
        _lib.check(lib.tg_render_forward(
            _ptr(vertices), _ptr(indices), _ptr(colors), _ptr(opacities), _ptr(sorted_ids), _ptr(offsets), _ptr(bary_transforms),
            width, height, tile_width, tile_height, float(early_stopping_threshold), int(bool(per_pixel_sort)), int(max_layers),
            _ptr(image), _ptr(depthmap), _ptr(final_weights), _ptr(ends), _ptr(last), _ptr(last_depth), _ptr(fragments),
            _ptr(hit_masks), _ptr(batch_bounds), _ptr(far_start), _ptr(sort_status), _stream(vertices)), "tg_render_forward", bits)
        timings = timer.stop()
        if not disable_timing:  # the timer has waited for the stream anyway
            if status_check.failed() and not _tickets_forced:
                # the lists are invalid (and the image NaN): the whole frame once more, its tiles numbered by ticket
                force_tickets(True)
                return _forward_full(vertices, indices, colors, opacities, width, height, tile_width, tile_height,
                                     early_stopping_threshold, disable_timing, per_pixel_sort, max_layers)
            status_check.checked = False
            status_check.verify()
    return (image, depthmap, final_weights, sorted_ids, offsets, bary_transforms, ends, timings,
            (last, last_depth, status_check, fragments, hit_masks))


def render_forward(vertices, indices, colors, opacities, width, height, tile_width, tile_height,
                   early_stopping_threshold, disable_timing, per_pixel_sort, max_layers):
    """Reference _C.render_forward (render.h:22-36, render.cu:713-763), same arguments, same eight results:

    -> (image, depthmap, final_weights, sorted_ids, offsets, bary_transforms, ends, timings)

    What this build's backward pass wants beyond them travels as an attribute of `ends` (render_backward
    looks for it there and does without if it is gone)."""
    *results, resume = _forward_full(vertices, indices, colors, opacities, width, height, tile_width, tile_height,
                                     early_stopping_threshold, disable_timing, per_pixel_sort, max_layers)
    results[6]._tg_resume = resume
    return tuple(results)


def _resume_by_forward(vertices, indices, colors, opacities, sorted_ids, offsets, bary_transforms, width, height, tile_width,
                       tile_height, early_stopping_threshold, per_pixel_sort, max_layers):
    """What the forward kernel hands to the backward pass, computed again from the saved lists: the forward
    kernel runs once more into scratch outputs (a caller that kept only the reference's saved tensors)."""
    bits = _bits(vertices)
    lib = _lib.load(bits)
    real, dev = vertices.dtype, vertices.device
    image = torch.empty((height, width, 4), dtype=real, device=dev)
    plane = [torch.empty((height, width), dtype=real, device=dev) for _ in range(2)]
    ends = torch.empty((height, width), dtype=torch.int32, device=dev)
    last = torch.empty((height, width), dtype=torch.int32, device=dev)
    last_depth = torch.empty((height, width), dtype=real, device=dev) if per_pixel_sort else None
    save_order = bool(per_pixel_sort) and SAVE_BLEND_ORDER and 0 < int(max_layers) <= MAX_SAVED_LAYERS
    fragments = torch.empty((2 * int(max_layers), height, width), dtype=torch.int16, device=dev) if save_order else None
    hit_masks = None
    if not per_pixel_sort and SAVE_HIT_MASKS:
        words = int(lib.tg_hit_mask_words(sorted_ids.numel(), width, height, tile_width, tile_height))
        hit_masks = torch.empty((words,), dtype=torch.int64, device=dev)
    _lib.check(lib.tg_render_forward(
        _ptr(vertices), _ptr(indices), _ptr(colors), _ptr(opacities), _ptr(sorted_ids), _ptr(offsets), _ptr(bary_transforms),
        width, height, tile_width, tile_height, float(early_stopping_threshold), int(bool(per_pixel_sort)), int(max_layers),
        _ptr(image), _ptr(plane[0]), _ptr(plane[1]), _ptr(ends), _ptr(last), _ptr(last_depth), _ptr(fragments),
        _ptr(hit_masks), None, None, None, _stream(vertices)), "tg_render_forward", bits)
    return last, last_depth, None, fragments, hit_masks


def render_backward(grad_output, grad_depthmap, vertices, indices, colors, opacities, sorted_ids, offsets, bary_transforms,
                    image, depthmap, final_weights, ends, width, height, tile_width, tile_height, early_stopping_threshold,
                    per_pixel_sort, max_layers, resume=None, grad_strides=None):
    """Reference _C.render_backward (render.h:6-20, render.cu:765-804), same twenty arguments
    -> (grad_vertices, grad_colors, grad_opacities).

    resume: what _forward_full returned next to the reference's results; without it (the reference's wrapper
    saves eleven tensors and nothing else) it is taken from `ends` if render_forward's attribute is still
    there, else computed again.  grad_depthmap may be None (no gradient reached the depth map).  grad_strides
    (scalars per vertex in the three arrays the kernel accumulates into) defaults to dense arrays in tile order
    and to one (V,8) block with per_pixel_sort; the returned tensors are dense either way."""
    _need_cuda(grad_output, vertices)
    if max_layers <= 0:
        max_layers = indices.shape[0] + 1
    bits = _bits(vertices)
    lib = _lib.load(bits)
    dev = vertices.device
    with _on_device(dev):
        tensors = [None if t is None else t.contiguous()
                   for t in (grad_output, grad_depthmap, vertices, indices, colors, opacities, sorted_ids, offsets,
                             bary_transforms, image, depthmap, final_weights, ends)]
        if resume is None:
            resume = getattr(ends, "_tg_resume", None)
        if resume is None:
            resume = _resume_by_forward(*tensors[2:9], width, height, tile_width, tile_height, early_stopping_threshold,
                                        per_pixel_sort, max_layers)
        last, last_depth, status_check, fragments, hit_masks = resume
        if status_check is not None:
            status_check.verify()
        tensors.append(last.contiguous())
        # one zero fill for the three gradients.  Tile order: (V,4) | (V,3) | (V,) views of one block.  Per-pixel
        # order issues five times as many atomics; there the eight gradients of a vertex share a 32-byte
        # sector of a (V,8) block while the kernel runs, and the three arrays are copied out afterwards.
        V = vertices.shape[0]
        strides = tuple(grad_strides) if grad_strides is not None else ((8, 8, 8) if per_pixel_sort else (4, 3, 1))
        if strides == (4, 3, 1):
            block = torch.zeros((8 * V,), dtype=vertices.dtype, device=dev)
            grad_vertices = block[:4 * V].view(V, 4)
            grad_colors = block[4 * V:7 * V].view(V, 3)
            grad_opacities = block[7 * V:]
        elif strides == (8, 8, 8):
            b8 = torch.zeros((V, 8), dtype=vertices.dtype, device=dev)
            grad_vertices, grad_colors, grad_opacities = b8[:, 0:4], b8[:, 4:7], b8[:, 7]
        else:
            sv, sc, so = strides
            grad_vertices = torch.zeros((V, sv), dtype=vertices.dtype, device=dev)[:, :4]
            grad_colors = torch.zeros((V, sc), dtype=vertices.dtype, device=dev)[:, :3]
            grad_opacities = torch.zeros((V, so), dtype=vertices.dtype, device=dev)[:, 0]
        _lib.check(lib.tg_render_backward(
            *[_ptr(t) for t in tensors], _ptr(last_depth), _ptr(fragments), _ptr(hit_masks), width, height, tile_width, tile_height,
            float(early_stopping_threshold), int(bool(per_pixel_sort)), int(max_layers), _ptr(grad_vertices), _ptr(grad_colors),
            _ptr(grad_opacities), *strides, _stream(vertices)), "tg_render_backward", bits)
        if strides == (8, 8, 8):
            grad_vertices = torch.empty((V, 4), dtype=vertices.dtype, device=dev)
            grad_colors = torch.empty((V, 3), dtype=vertices.dtype, device=dev)
            grad_opacities = torch.empty((V,), dtype=vertices.dtype, device=dev)
            _lib.check(lib.tg_split_gradient_block(_ptr(b8), V, _ptr(grad_vertices), _ptr(grad_colors), _ptr(grad_opacities),
                                                   _stream(vertices)), "tg_split_gradient_block", bits)
        elif strides != (4, 3, 1):
            grad_vertices, grad_colors, grad_opacities = (grad_vertices.contiguous(), grad_colors.contiguous(),
                                                          grad_opacities.contiguous())
    return grad_vertices, grad_colors, grad_opacities


# ---- per-kernel timing (the library's counterpart of the reference's CudaTimer) ----

def profile_enable(on=True):
    _lib.load().tg_profile_enable(1 if on else 0)


def profile_report():
    """-> {kernel_name: (launches, total_milliseconds)} since the last report; waits for the recorded events."""
    lib = _lib.load()
    buf = C.create_string_buffer(1 << 16)
    lib.tg_profile_report(buf, len(buf))
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, ms = line.split()
        out[name] = (int(count), float(ms))
    return out


def set_precision(dtype):
    """Selects the scalar type the public entry points expect (torch.float32 or torch.float64)."""
    global precision
    if dtype not in (torch.float32, torch.float64):
        raise TypeError(f"precision must be torch.float32 or torch.float64, got {dtype}")
    _lib.load(64 if dtype == torch.float64 else 32)
    precision = dtype
