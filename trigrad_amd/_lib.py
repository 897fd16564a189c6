"""ctypes loader of libtrigrad_hip.so: declares every entry point of include/trigrad_hip.h.

There is no fallback: if the library is missing or an entry point fails, an
exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# One library per scalar type, like the reference's compile-time DOUBLE_PRECISION switch (util.h:5-20).
# TRIGRAD_HIP_LIB names another build of the float library (same ABI), e.g. one made with different tuning constants.
LIB_PATHS = {
    32: os.environ.get("TRIGRAD_HIP_LIB") or os.path.join(_HERE, "lib", "libtrigrad_hip.so"),
    64: os.path.join(_HERE, "lib", "libtrigrad_hip_f64.so"),
}
LIB_PATH = LIB_PATHS[32]

_p = C.c_void_p
_i = C.c_int
_i32 = C.c_int32
_i64 = C.c_int64
_sz = C.c_size_t
_f = "tg_real"  # placeholder: c_float in the float library, c_double in the double one


# name -> (restype, argtypes); the order is that of include/trigrad_hip.h
SIGNATURES = {
    "tg_version": (_i, []),
    "tg_precision_bits": (_i, []),
    "tg_last_error": (C.c_char_p, []),
    "tg_num_tiles": (_i, [_i, _i, _i, _i]),
    "tg_force_tickets": (None, [_i]),
    "tg_profile_enable": (None, [_i]),
    "tg_profile_report": (_i, [C.c_char_p, _sz]),
    "tg_bin_count": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _p]),
    "tg_scan_workspace_bytes": (_sz, [_i64]),
    "tg_scan_exclusive_u32": (_i, [_p, _p, _i64, _p, _p, _sz, _p, C.c_uint32, C.c_uint32, _p, _p]),
    "tg_scan_noalloc_max_n": (_i64, []),
    "tg_scan_exclusive_u32_noalloc": (_i, [_p, _p, _i64, _p, _p, C.c_uint32, C.c_uint32, _p, _p]),
    "tg_bin_emit": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _i64, _p, C.c_uint32, _p, _p, _p]),
    "tg_sort_workspace_bytes": (_sz, [_i64]),
    "tg_sort_pairs_u64_u32": (_i, [_p, _p, _p, _p, _i64, _i, _p, _sz, _p, C.POINTER(_i), _p]),
    "tg_tile_ranges": (_i, [_p, _i64, _i, _p, _p]),
    "tg_tile_list_sort_workspace_bytes": (_sz, [_i64, _i]),
    "tg_sort_tile_lists": (_i, [_p, _p, _p, _p, _i64, _i, _p, _p, _sz, _p, C.POINTER(_i), _p]),
    "tg_bin_setup_workspace_bytes": (_sz, [_i32, _i, _i, _i, _i]),
    "tg_bin_setup": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _p, _p, C.c_uint32, _p, _p, _sz, _p]),
    "tg_build_tile_lists_workspace_bytes": (_sz, [_i64, _i]),
    "tg_build_tile_lists": (_i, [_p, _p, _i32, _i64, C.c_uint32, _p, _p, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p, _i,
                                C.POINTER(_i), _p]),
    "tg_bin_frame_supported": (_i, [_i, _i, _i, _i]),
    "tg_bin_frame_workspace_bytes": (_sz, [_i32, _i64, _i, _i, _i, _i]),
    "tg_bin_frame": (_i, [_p, _i32, _p, _i32, _i, _i, _i, _i, _p, _p, _i64, _p, _p, _sz, C.c_uint32, _p, _sz, _p, _p]),
    "tg_build_frame_lists_workspace_bytes": (_sz, [_i64, _i, _i]),
    "tg_build_frame_lists": (_i, [_p, C.c_uint32, _i64, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p, C.POINTER(_i), _p]),
    "tg_bary": (_i, [_p, _i32, _p, _i32, _p, _p]),
    "tg_list_bound_words": (_sz, [_i64, _i]),
    "tg_list_bounds": (_i, [_p, _i32, _p, _i32, _p, _p, _p, _i, _p, _p, _p, _p]),
    "tg_hit_mask_words": (_sz, [_i64, _i, _i, _i, _i]),
    "tg_render_forward": (_i, [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _f, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "tg_render_backward": (_i, [_p] * 17 + [_i, _i, _i, _i, _f, _i, _i, _p, _p, _p, _i, _i, _i, _p]),
    "tg_split_gradient_block": (_i, [_p, _i64, _p, _p, _p, _p]),
    "tg_barycentric": (None, [_p] * 5),
    "tg_barycentric_backward": (None, [_p] * 6),
    "tg_interpolate3_scalar": (_f, [_p, _f, _f, _f, _p]),
    "tg_interpolate3_scalar_backward": (None, [_f, _p, _f, _f, _f, _p, _p, _p, _p]),
    "tg_interpolate3_vector": (None, [_p] * 6),
    "tg_interpolate3_vector_backward": (None, [_p] * 11),
}

_libs = {}


def load(bits=32):
    """The library whose scalar type has `bits` bits (32: float, 64: double)."""
    lib = _libs.get(bits)
    if lib is None:
        path = LIB_PATHS[bits]
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: build it with `python -m trigrad_amd.build` "
                "(hipcc --offload-arch=gfx950); trigrad_amd has no other backend")
        lib = C.CDLL(path)
        real = C.c_float if bits == 32 else C.c_double
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = real if res is _f else res
            fn.argtypes = [real if a is _f else a for a in args]
        if lib.tg_precision_bits() != bits:
            raise RuntimeError(f"{path} is built for {lib.tg_precision_bits()}-bit scalars, expected {bits}")
        _libs[bits] = lib
    return lib


def check(code, what, bits=32):
    """Raise RuntimeError for a non-zero return code of an entry point."""
    if code != 0:
        msg = load(bits).tg_last_error()
        raise RuntimeError(f"{what} failed with code {code}: {msg.decode() if msg else ''}")
