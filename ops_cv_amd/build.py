"""Builds libopscv_amd.so in-tree with hipcc for gfx950 (python -m ops_cv_amd.build)."""
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force=True, jobs=8):
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j%d" % jobs]
    if force:
        cmd.append("-B")
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError("building libopscv_amd.so failed")
    return os.path.join(_HERE, "libopscv_amd.so")


if __name__ == "__main__":
    print(build())
