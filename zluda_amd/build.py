"""Compiles the gfx950 library in-tree: zluda_amd/lib/libcublaslt.so (+ the soname links)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib", "libcublaslt.so")


def build(force=False, jobs=8, verbose=False):
    """Runs make in csrc/.  force=True rebuilds every object even if it is up to date."""
    cmd = ["make", "-C", CSRC, "-j%d" % jobs] + (["-B"] if force else [])
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode:
        print(res.stdout)
    if res.returncode:
        raise RuntimeError("building libcublaslt.so failed (exit %d)" % res.returncode)
    return LIB


if __name__ == "__main__":
    import sys
    print(build(force="-B" in sys.argv, verbose=True))
