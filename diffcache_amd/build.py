"""Builds libdiffcache_hip.so in-tree with hipcc for gfx950.

`python diffcache_amd/build.py` (or `make -C diffcache_amd/csrc`) — cross-compiles without a
GPU.  Run it as a script, not with `-m`: importing the package needs the library this builds.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = True, jobs: int = 8) -> str:
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("building libdiffcache_hip.so failed")
    return os.path.join(HERE, "libdiffcache_hip.so")


if __name__ == "__main__":
    print(build())
