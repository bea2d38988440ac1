"""Compiles ``libfwdmi.so`` for gfx950 in-tree (``python -m forward_amd.build``)."""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfwdmi.so")


def build(force=True, jobs=8):
    cmd = ["make", "-C", CSRC, "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd, stdout=subprocess.DEVNULL if not force else None)
    return LIB


if __name__ == "__main__":
    print(build(force="--no-force" not in sys.argv))
