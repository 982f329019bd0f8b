"""Builds the HIP library in-tree (``permutohedral_encoding_amd/libpenc_hip.so``) with hipcc for gfx950."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libpenc_hip.so")


def build_library(force=True, verbose=False):
    """Runs ``make`` in ``csrc/``; with ``force`` the library is rebuilt even if it is up to date."""
    cmd = ["make", "-C", CSRC]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError("building libpenc_hip.so failed (see the compiler output above)")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, verbose=True))
