"""Compiles csrc/ for gfx950 with hipcc (make); cross-compiles without a GPU."""
import os
import subprocess

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build_library(clean=False, jobs=8, drivers=True):
    if clean:
        subprocess.run(["make", "-C", _CSRC, "clean"], check=True, capture_output=True)
    target = ["all"] if drivers else ["libmpspmm.so"]
    proc = subprocess.run(["make", "-C", _CSRC, "-j%d" % jobs] + target, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libmpspmm failed:\n" + proc.stdout[-4000:] + proc.stderr[-4000:])
    return os.path.join(_CSRC, "libmpspmm.so")
