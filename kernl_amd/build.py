"""Build libkernl_hip.so in-tree:  python -m kernl_amd.build  (drives kernl_amd/csrc/Makefile)."""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build(force: bool = True, jobs: int = 4) -> str:
    """Compile every HIP source for gfx950 and link the shared library; returns its path."""
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", CSRC, f"-j{jobs}"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError("building libkernl_hip.so failed")
    return os.path.join(os.path.dirname(CSRC), "libkernl_hip.so")


if __name__ == "__main__":
    print(build())
