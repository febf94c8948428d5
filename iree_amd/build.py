"""Builds the C-ABI library (iree_amd/csrc/libiree_amd_uk.so) and the code
object of the mmt4d kernels for a HAL executable
(iree_amd/hal/mi355x_kernels_gfx950.co) for gfx950.

    python -m iree_amd.build            # incremental
    python -m iree_amd.build --force    # recompile everything

hipcc cross-compiles, so this works on a machine without a GPU.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")


def build(force=False, jobs=8, quiet=False):
    cmd = ["make", "-C", CSRC, f"-j{jobs}"]
    if force:
        cmd.append("-B")
    out = subprocess.DEVNULL if quiet else None
    subprocess.check_call(cmd, stdout=out)
    lib = os.path.join(CSRC, "libiree_amd_uk.so")
    if not os.path.exists(lib):
        raise RuntimeError("build finished but libiree_amd_uk.so is missing")
    if not os.path.exists(os.path.join(HERE, "hal", "mi355x_kernels_gfx950.co")):
        raise RuntimeError("build finished but hal/mi355x_kernels_gfx950.co is missing")
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
