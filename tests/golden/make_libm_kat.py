"""Writes tests/golden/libm_glibc235.npz: known-answer vectors for every
libm-backed function on the path, produced by the CPU oracle in the build
container (glibc 2.35, x86-64 with FMA: expf/logf/powf/sinf/cosf resolve to their
FMA variants).  The reference ships no vectors for this path; these let a run on
another machine tell "the host libm differs" apart from "the kernel is wrong".

    python tests/golden/make_libm_kat.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from tests.helpers import SPECIALS  # noqa: E402


def inputs():
    r = np.random.default_rng(20240521)
    parts = [SPECIALS,
             np.linspace(-12, 12, 4001, dtype=np.float32),
             (r.standard_normal(6000, dtype=np.float32) * np.float32(2.0)),
             (r.standard_normal(2000, dtype=np.float32) * np.float32(30.0)),
             np.float32(2.0) ** r.integers(-60, 8, 2000).astype(np.float32) * r.choice(np.float32([-1, 1]), 2000)]
    return np.concatenate(parts).astype(np.float32)


def main():
    x = inputs()
    out = {"x": x}
    for op, name in [(3, "log"), (4, "exp"), (5, "sin"), (6, "cos"), (7, "tan"), (8, "asin"),
                     (9, "acos"), (10, "atan")]:
        out["unary_" + name] = oracle.unary(op, x)
    for act, name in [(3, "sigmoid"), (4, "softplus"), (5, "tanh"), (8, "gelu")]:
        out["act_" + name] = oracle.activate(x, act)
    r = np.random.default_rng(7)
    pa = (r.random(4000, dtype=np.float32) * np.float32(6.0)).astype(np.float32)
    pb = (r.standard_normal(4000, dtype=np.float32) * np.float32(2.0)).astype(np.float32)
    out["pow_a"], out["pow_b"], out["pow"] = pa, pb, oracle.binary(4, pa, pb)
    np.savez_compressed(os.path.join(HERE, "libm_glibc235.npz"), **out)
    print("wrote %d inputs, %d arrays" % (x.size, len(out)))


if __name__ == "__main__":
    main()
