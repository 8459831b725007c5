"""Writes tests/golden/workloads_small.npz: seeded small inputs of the five
workloads and the outputs the CPU oracle gives for them.

    python tests/golden/make_golden.py

The reference ships no binary fixtures for this path and none of its Python was
imported to make these: the vectors come from oracle/closed_forms.py (the
whole-array NumPy expressions the reference's tests check against) and were
cross-checked against the plain-C statement in oracle/c/oracle.c when written.
They pin the oracle itself: a change of NumPy version, of a seed, or of a
formula shows up as a difference against this file (tests/test_golden.py), and
the GPU results are compared with the same file.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import c_oracle as co          # noqa: E402
from oracle import closed_forms as cf      # noqa: E402

SHAPES = {"c1": 1003, "c2": (37, 131), "c3": (9, 517), "c4": (11, 1000), "c5": (128, 128, 128)}


def build():
    out = {}
    a, b = cf.inputs_c1(SHAPES["c1"])
    out.update(c1_a=a, c1_b=b, c1_out=cf.np_add(a, b))
    assert np.array_equal(out["c1_out"].view(np.uint32), co.add_f32(a, b).view(np.uint32))
    a, b, c = cf.inputs_c2(SHAPES["c2"])
    out.update(c2_a=a, c2_b=b, c2_c=c, c2_out=cf.np_fma_f16(a, b, c))
    assert np.array_equal(out["c2_out"].view(np.uint16), co.fma_f16(a, b, c).view(np.uint16))
    (x,) = cf.inputs_c3(SHAPES["c3"])
    out.update(c3_x=x, c3_out=cf.np_softmax(x))
    (x,) = cf.inputs_c4(SHAPES["c4"])
    q, s = cf.np_quantize(x)
    out.update(c4_x=x, c4_q=q, c4_scale=s)
    qc, sc = co.quantize(x)
    assert np.array_equal(q, qc) and np.array_equal(s.view(np.uint32), sc.view(np.uint32))
    ab, bb = cf.inputs_c5(SHAPES["c5"])
    out.update(c5_a=ab, c5_bt=bb, c5_out_f32acc=cf.np_gemm_bf16(ab, bb, np.float32))
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "workloads_small.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
