"""Build the two product libraries in-tree.

    python -m shadow_amd.build            # both
    python -m shadow_amd.build hip        # selected targets

Targets
    hip     shadow_amd/lib/libshadow_hip.so   gfx950 kernels + C ABI (hipcc)
    host    shadow_amd/lib/libshadow_host.so  C++ operator layer over the C ABI (g++)

The test-side libraries have their own recipes: `python -m oracle.build` (the
CPU restatement of the reference) and `python -m tests.native.build` (the host
build of the device math code).

hipcc cross-compiles for gfx950 without a GPU.  The device code must keep
multiply and add separate (the reference never fuses), hence -ffp-contract=off;
packed fp32 instructions are disabled for every HIP translation unit.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "shadow_amd", "csrc")
HOST = os.path.join(ROOT, "shadow_amd", "host")
LIB = os.path.join(ROOT, "shadow_amd", "lib")
OBJ = os.path.join(LIB, "obj")

HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HIP_SOURCES = ["elementwise.hip", "broadcast.hip", "reduce.hip", "fused.hip", "vision.hip", "softmax.hip", "norm.hip", "movers.hip",
               "lrn.hip", "grid_sample.hip", "runtime.hip"]

def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip():
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    jobs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as pool:
        for src in HIP_SOURCES:
            obj = os.path.join(OBJ, src.replace(".hip", ".o"))
            objs.append(obj)
            jobs.append(pool.submit(_run, [HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]))
        plan_obj = os.path.join(OBJ, "plan.o")
        objs.append(plan_obj)
        jobs.append(pool.submit(_run, ["g++", "-O2", "-std=c++17", "-fPIC", "-c",
                                       os.path.join(CSRC, "plan.cpp"), "-o", plan_obj]))
        for j in jobs:
            j.result()
    out = os.path.join(LIB, "libshadow_hip.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", out])
    return out


def build_host():
    srcs = sorted(
        os.path.join(dp, f) for dp, _, fs in os.walk(HOST) for f in fs if f.endswith(".cpp"))
    if not srcs:
        return None
    out = os.path.join(LIB, "libshadow_host.so")
    _run(["g++", "-O2", "-std=c++14", "-fPIC", "-shared", "-I", HOST, "-I", os.path.join(ROOT, "include")]
         + srcs + ["-L", LIB, "-lshadow_hip", "-Wl,-rpath,$ORIGIN", "-o", out])
    return out


TARGETS = {"hip": build_hip, "host": build_host}


def build_all(names=None):
    built = []
    for name in (names or ["hip", "host"]):
        path = TARGETS[name]()
        if path:
            built.append(path)
    return built


if __name__ == "__main__":
    for p in build_all(sys.argv[1:] or None):
        print("built", os.path.relpath(p, ROOT))
