"""megcc_amd: MI355X (gfx950) implementation of MegCC's generated-kernel hot path.

The product is the C-ABI shared library `libmegcc_gfx950.so` (include/megcc_gfx950.h), built from
megcc_amd/csrc by `build()`. This package is the thin Python harness around it that the tests and
bench.py use: ctypes mirrors of the ABI structs (abi.py) and device-buffer helpers (runtime.py).
There is no CPU fallback: loading fails loudly when the library has not been built.
"""
import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# (MEGCC_GFX950_LIB: another build of the same library, e.g. one made with EXTRA_FLAGS for an experiment)
LIB_PATH = os.environ.get("MEGCC_GFX950_LIB") or os.path.join(PKG_DIR, "libmegcc_gfx950.so")


def build(jobs=8):
    """Compile every HIP source for gfx950 into libmegcc_gfx950.so (works without a GPU)."""
    subprocess.check_call(["make", "-s", "-C", os.path.join(PKG_DIR, "csrc"), "-j%d" % jobs, "-B"])
    return LIB_PATH
