"""ctypes binding of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module.  It loads oracle/libtrigrad_oracle.so (built by oracle/Makefile from
oracle/trigrad_oracle.cpp) and wraps each entry point with numpy arrays.

All functions take/return numpy arrays; dtype float32 selects the shipped
precision, float64 the reference's DOUBLE_PRECISION build
(reference src/trigrad/util.h:6-20).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtrigrad_oracle.so")


def build(force=False):
    """Compile the oracle with g++ (strict IEEE flags live in oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "libtrigrad_oracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        for suf in ("f32", "f64"):
            getattr(_lib, f"tgo_bin_emit_{suf}").restype = C.c_long
            getattr(_lib, f"tgo_per_tile_lists_{suf}").restype = C.c_long
        _lib.tgo_interpolate3_scalar_f32.restype = C.c_float
        _lib.tgo_interpolate3_scalar_f64.restype = C.c_double
        _lib.tgo_max_threads.restype = C.c_int
    return _lib


def set_threads(n):
    lib().tgo_set_threads(int(n))


def max_threads():
    return int(lib().tgo_max_threads())


def _suf(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError(f"oracle supports float32/float64, got {dtype}")


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def n_tiles(W, H, tw, th):
    return ((W + tw - 1) // tw) * ((H + th - 1) // th)


def bin_count(verts, idx, W, H, tw=16, th=16):
    """-> (per-triangle overlap counts (M,), per-tile counts (T,)); render.cu:51-139."""
    suf, _ = _suf(verts.dtype)
    verts = _c(verts, verts.dtype)
    idx = _c(idx, np.int32)
    M = idx.shape[0]
    tri = np.zeros(M, np.int32)
    tile = np.zeros(n_tiles(W, H, tw, th), np.int32)
    getattr(lib(), f"tgo_bin_count_{suf}")(_p(verts), _p(idx), M, W, H, tw, th, _p(tri), _p(tile))
    return tri, tile


def bin_emit(verts, idx, W, H, tw=16, th=16):
    """-> dict(tile, depth, tri, keys64) in emission order (triangle id, tile x outer, tile y inner)."""
    suf, _ = _suf(verts.dtype)
    verts = _c(verts, verts.dtype)
    idx = _c(idx, np.int32)
    M = idx.shape[0]
    fn = getattr(lib(), f"tgo_bin_emit_{suf}")
    K = fn(_p(verts), _p(idx), M, W, H, tw, th, None, None, None, None)
    tile = np.zeros(K, np.int32)
    depth = np.zeros(K, verts.dtype)
    tri = np.zeros(K, np.int32)
    keys = np.zeros(K, np.uint64)
    fn(_p(verts), _p(idx), M, W, H, tw, th, _p(tile), _p(depth), _p(tri), _p(keys))
    return dict(tile=tile, depth=depth, tri=tri, keys64=keys)


def per_tile_lists(verts, idx, W, H, tw=16, th=16):
    """-> (offsets (T+1,), sorted_ids (K,), sorted_depths (K,)); render.cu:272-308."""
    suf, _ = _suf(verts.dtype)
    verts = _c(verts, verts.dtype)
    idx = _c(idx, np.int32)
    M = idx.shape[0]
    T = n_tiles(W, H, tw, th)
    offsets = np.zeros(T + 1, np.int32)
    fn = getattr(lib(), f"tgo_per_tile_lists_{suf}")
    K = fn(_p(verts), _p(idx), M, W, H, tw, th, _p(offsets), None, None, C.c_long(0))
    ids = np.zeros(K, np.int32)
    depths = np.zeros(K, verts.dtype)
    fn(_p(verts), _p(idx), M, W, H, tw, th, _p(offsets), _p(ids), _p(depths), C.c_long(K))
    return offsets, ids, depths


def sort_pairs_u64(keys, vals):
    keys = _c(keys, np.uint64)
    vals = _c(vals, np.int32)
    ko = np.zeros_like(keys)
    vo = np.zeros_like(vals)
    lib().tgo_sort_pairs_u64(_p(keys), _p(vals), C.c_long(keys.shape[0]), _p(ko), _p(vo))
    return ko, vo


def tile_ranges(sorted_keys, T):
    sorted_keys = _c(sorted_keys, np.uint64)
    off = np.zeros(T + 1, np.int32)
    lib().tgo_tile_ranges(_p(sorted_keys), C.c_long(sorted_keys.shape[0]), T, _p(off))
    return off


def bary(verts, idx):
    """-> (M,3,3) cartesian-to-barycentric matrices; render.cu:310-337."""
    suf, _ = _suf(verts.dtype)
    verts = _c(verts, verts.dtype)
    idx = _c(idx, np.int32)
    out = np.zeros((idx.shape[0], 3, 3), verts.dtype)
    getattr(lib(), f"tgo_bary_{suf}")(_p(verts), _p(idx), idx.shape[0], _p(out))
    return out


def forward(verts, idx, colors, opac, ids, offsets, bary_m, W, H, tw=16, th=16, thr=1 / 256,
            per_pixel_sort=True, max_layers=32):
    """-> dict(image, depthmap, weights, ends, last); render.cu:540-619.

    `last` is not a reference output: per pixel, one past the list position
    (relative to the tile's start) of the last blended entry.
    """
    suf, ct = _suf(verts.dtype)
    dt = verts.dtype
    verts, colors, opac, bary_m = (_c(a, dt) for a in (verts, colors, opac, bary_m))
    idx, ids, offsets = (_c(a, np.int32) for a in (idx, ids, offsets))
    if max_layers <= 0:
        max_layers = idx.shape[0] + 1  # wrapper.py:35-36
    image = np.zeros((H, W, 4), dt)
    depthmap = np.zeros((H, W), dt)
    weights = np.zeros((H, W), dt)
    ends = np.zeros((H, W), np.int32)
    last = np.zeros((H, W), np.int32)
    getattr(lib(), f"tgo_forward_{suf}")(
        _p(verts), _p(idx), _p(colors), _p(opac), _p(ids), _p(offsets), _p(bary_m), W, H, tw, th, ct(thr),
        int(bool(per_pixel_sort)), int(max_layers), _p(image), _p(depthmap), _p(weights), _p(ends), _p(last))
    return dict(image=image, depthmap=depthmap, weights=weights, ends=ends, last=last)


def backward(grad_image, grad_depthmap, verts, idx, colors, opac, ids, offsets, bary_m, fwd, W, H, tw=16, th=16,
             per_pixel_sort=True, max_layers=32, literal=False, magnitudes=False):
    """-> (grad_vertices (V,4), grad_colors (V,3), grad_opacities (V,)) as float64; render.cu:621-695.

    magnitudes: also three arrays of the same shapes with, per element, the sum of the magnitudes of everything that
    was added into it (for a position gradient: of the products its terms are made of).  The rounding error of a
    float32 accumulation of the same terms, in any order, is proportional to that sum, element by element."""
    suf, _ = _suf(verts.dtype)
    dt = verts.dtype
    verts, colors, opac, bary_m, grad_image, grad_depthmap = (
        _c(a, dt) for a in (verts, colors, opac, bary_m, grad_image, grad_depthmap))
    idx, ids, offsets = (_c(a, np.int32) for a in (idx, ids, offsets))
    if max_layers <= 0:
        max_layers = idx.shape[0] + 1
    V = verts.shape[0]
    copies = 2 if magnitudes else 1
    gV = np.zeros((copies, V, 4), np.float64)
    gC = np.zeros((copies, V, 3), np.float64)
    gO = np.zeros((copies, V), np.float64)
    getattr(lib(), f"tgo_backward_{suf}")(
        _p(grad_image), _p(grad_depthmap), _p(verts), _p(idx), _p(colors), _p(opac), _p(ids), _p(offsets), _p(bary_m),
        _p(_c(fwd["image"], dt)), _p(_c(fwd["depthmap"], dt)), _p(_c(fwd["weights"], dt)), _p(_c(fwd["ends"], np.int32)),
        W, H, tw, th, int(bool(per_pixel_sort)), int(max_layers), int(bool(literal)), V, _p(gV), _p(gC), _p(gO),
        int(bool(magnitudes)))
    if magnitudes:
        return gV[0], gC[0], gO[0], gV[1], gC[1], gO[1]
    return gV[0], gC[0], gO[0]


def render(verts, idx, colors, opac, W, H, tw=16, th=16, thr=1 / 256, per_pixel_sort=True, max_layers=32):
    """Whole forward pipeline (render.cu:713-763); returns the forward dict plus the saved intermediates."""
    offsets, ids, depths = per_tile_lists(verts, idx, W, H, tw, th)
    bm = bary(verts, idx)
    out = forward(verts, idx, colors, opac, ids, offsets, bm, W, H, tw, th, thr, per_pixel_sort, max_layers)
    out.update(offsets=offsets, sorted_ids=ids, sorted_depths=depths, bary=bm)
    return out


def render_backward(grad_image, grad_depthmap, verts, idx, colors, opac, fwd, W, H, tw=16, th=16,
                    per_pixel_sort=True, max_layers=32, literal=False, magnitudes=False):
    return backward(grad_image, grad_depthmap, verts, idx, colors, opac, fwd["sorted_ids"], fwd["offsets"], fwd["bary"],
                    fwd, W, H, tw, th, per_pixel_sort, max_layers, literal, magnitudes)


# ---- component hooks (reference src/trigrad/tests.cu:43-76) ---------------------

def barycentric(p0, p1, q0, q1):
    suf, _ = _suf(p0.dtype)
    out = np.zeros(3, p0.dtype)
    getattr(lib(), f"tgo_barycentric_{suf}")(_p(_c(p0, p0.dtype)), _p(_c(p1, p0.dtype)), _p(_c(q0, p0.dtype)),
                                             _p(_c(q1, p0.dtype)), _p(out))
    return out


def barycentric_backward(g, a, b, c, p):
    suf, _ = _suf(a.dtype)
    dt = a.dtype
    out = np.zeros((4, 2), dt)
    getattr(lib(), f"tgo_barycentric_backward_{suf}")(_p(_c(g, dt)), _p(_c(a, dt)), _p(_c(b, dt)), _p(_c(c, dt)),
                                                      _p(_c(p, dt)), _p(out))
    return out


def interpolate3_scalar(bc, a, b, c, w):
    suf, ct = _suf(bc.dtype)
    dt = bc.dtype
    return getattr(lib(), f"tgo_interpolate3_scalar_{suf}")(_p(_c(bc, dt)), ct(a), ct(b), ct(c), _p(_c(w, dt)))


def interpolate3_scalar_backward(g, bc, a, b, c, w):
    suf, ct = _suf(bc.dtype)
    dt = bc.dtype
    gb, gv, gw = np.zeros(3, dt), np.zeros(3, dt), np.zeros(3, dt)
    getattr(lib(), f"tgo_interpolate3_scalar_backward_{suf}")(ct(g), _p(_c(bc, dt)), ct(a), ct(b), ct(c), _p(_c(w, dt)),
                                                              _p(gb), _p(gv), _p(gw))
    return gb, gv, gw


def interpolate3_vector(bc, a, b, c, w):
    suf, _ = _suf(bc.dtype)
    dt = bc.dtype
    out = np.zeros(3, dt)
    getattr(lib(), f"tgo_interpolate3_vector_{suf}")(_p(_c(bc, dt)), _p(_c(a, dt)), _p(_c(b, dt)), _p(_c(c, dt)),
                                                     _p(_c(w, dt)), _p(out))
    return out


def interpolate3_vector_backward(g, bc, a, b, c, w):
    suf, _ = _suf(bc.dtype)
    dt = bc.dtype
    outs = [np.zeros(3, dt) for _ in range(5)]
    getattr(lib(), f"tgo_interpolate3_vector_backward_{suf}")(
        _p(_c(g, dt)), _p(_c(bc, dt)), _p(_c(a, dt)), _p(_c(b, dt)), _p(_c(c, dt)), _p(_c(w, dt)), *[_p(o) for o in outs])
    return tuple(outs)  # grad_bary, grad_a, grad_b, grad_c, grad_w
