"""Build the host-side native helpers of the tests.

    python -m tests.native.build

libm_sweep.so is the device math header (shadow_amd/csrc/libm_exact.h) compiled
for the host, with the loops that compare it against the host's libm.
launch_shapes is a gfx950 program that times the launch shapes the kernels were
given against their alternatives (tests/test_gpu_launch_shapes.py runs it).
"""
import os
import shutil
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
    shapes = os.path.join(HERE, "launch_shapes")
    hipcc = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
    _run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
          os.path.join(HERE, "launch_shapes.hip"), "-o", shapes])
    return [out, shapes]


if __name__ == "__main__":
    for path in build():
        print("built", os.path.relpath(path, os.path.dirname(os.path.dirname(HERE))))
