"""Build the host-side native helpers of the tests.

    python -m tests.native.build

libm_sweep.so is the device math header (shadow_amd/csrc/libm_exact.h) compiled
for the host, with the loops that compare it against the host's libm.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))


def build():
    out = os.path.join(HERE, "libm_sweep.so")
    _run(["g++", "-std=c++17", "-O2", "-ffp-contract=off", "-fPIC", "-shared", "-pthread",
          os.path.join(HERE, "libm_sweep.cpp"), "-o", out])
    return [out]


if __name__ == "__main__":
    for path in build():
        print("built", os.path.relpath(path, os.path.dirname(os.path.dirname(HERE))))
