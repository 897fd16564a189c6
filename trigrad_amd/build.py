"""Builds libtrigrad_hip.so (gfx950) from trigrad_amd/csrc/*.hip with hipcc.

    python -m trigrad_amd.build

The flags are part of the arithmetic contract of the kernels:
  -ffp-contract=off   no fused multiply-add may be formed from a*b+c: tile
                      bounds, depth keys, inside tests and transmittance must
                      round exactly like the source expressions;
  no -ffast-math      float division stays correctly rounded (hipcc default).
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtrigrad_hip.so")
LIB_PATH_F64 = os.path.join(LIB_DIR, "libtrigrad_hip_f64.so")  # the same sources with -DTG_DOUBLE_PRECISION

SOURCES = ["tg_api.hip", "tg_binning.hip", "tg_scan.hip", "tg_sort.hip", "tg_forward.hip", "tg_backward.hip",
           "tg_components.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-munsafe-fp-atomics",  # float atomic adds use the hardware instruction (coarse-grained memory)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(out, flags, verbose):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, *flags, *[os.path.join(CSRC, s) for s in SOURCES], "-o", out]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return out


def build(verbose=False, extra_flags=(), double_too=True):
    """Builds the float library and (double_too) the double one; returns the float library's path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    _compile(LIB_PATH, list(extra_flags), verbose)
    if double_too:
        _compile(LIB_PATH_F64, [*extra_flags, "-DTG_DOUBLE_PRECISION"], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
