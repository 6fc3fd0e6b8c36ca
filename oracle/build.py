"""Build oracle/liboracle.so, the CPU restatement of the reference's kernels.

    python -m oracle.build

Flags: the reference's Release flags (CMakeLists.txt:30-37) plus contraction off,
so that no host can fuse what baseline x86-64 does not.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
FLAGS = ["-O3", "-DNDEBUG", "-fPIC", "-ffp-contract=off", "-fno-fast-math"]


def build():
    src, out = os.path.join(HERE, "shadow_cpu.c"), os.path.join(HERE, "liboracle.so")
    cmd = ["gcc", "-std=c11"] + FLAGS + ["-shared", src, "-lm", "-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return out


if __name__ == "__main__":
    print("built", os.path.relpath(build(), os.path.dirname(HERE)))
