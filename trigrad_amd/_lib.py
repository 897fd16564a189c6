"""ctypes loader of libtrigrad_hip.so: declares every entry point of include/trigrad_hip.h.

There is no fallback: if the library is missing or an entry point fails, an
exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TRIGRAD_HIP_LIB names another build of the same library (same ABI), e.g. one made with different tuning constants
LIB_PATH = os.environ.get("TRIGRAD_HIP_LIB") or os.path.join(_HERE, "lib", "libtrigrad_hip.so")

_p = C.c_void_p
_i = C.c_int
_i32 = C.c_int32
_i64 = C.c_int64
_f = C.c_float
_sz = C.c_size_t

# name -> (restype, argtypes); the order is that of include/trigrad_hip.h
SIGNATURES = {
    "tg_version": (_i, []),
    "tg_last_error": (C.c_char_p, []),
    "tg_num_tiles": (_i, [_i, _i, _i, _i]),
    "tg_profile_enable": (None, [_i]),
    "tg_profile_report": (_i, [C.c_char_p, _sz]),
    "tg_bin_count": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _p]),
    "tg_scan_workspace_bytes": (_sz, [_i64]),
    "tg_scan_exclusive_u32": (_i, [_p, _p, _i64, _p, _p, _sz, _p, C.c_uint32, C.c_uint32, _p, _p]),
    "tg_bin_emit": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _i64, _p, C.c_uint32, _p, _p, _p]),
    "tg_sort_workspace_bytes": (_sz, [_i64]),
    "tg_sort_pairs_u64_u32": (_i, [_p, _p, _p, _p, _i64, _i, _p, _sz, _p, C.POINTER(_i), _p]),
    "tg_tile_ranges": (_i, [_p, _i64, _i, _p, _p]),
    "tg_bary": (_i, [_p, _i32, _p, _i32, _p, _p]),
    "tg_render_forward": (_i, [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _f, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p]),
    "tg_render_backward": (_i, [_p] * 16 + [_i, _i, _i, _i, _f, _i, _i, _p, _p, _p, _p]),
    "tg_barycentric": (None, [_p] * 5),
    "tg_barycentric_backward": (None, [_p] * 6),
    "tg_interpolate3_scalar": (_f, [_p, _f, _f, _f, _p]),
    "tg_interpolate3_scalar_backward": (None, [_f, _p, _f, _f, _f, _p, _p, _p, _p]),
    "tg_interpolate3_vector": (None, [_p] * 6),
    "tg_interpolate3_vector_backward": (None, [_p] * 11),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m trigrad_amd.build` "
                "(hipcc --offload-arch=gfx950); trigrad_amd has no other backend")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(code, what):
    """Raise RuntimeError for a non-zero return code of an entry point."""
    if code != 0:
        msg = load().tg_last_error()
        raise RuntimeError(f"{what} failed with code {code}: {msg.decode() if msg else ''}")
