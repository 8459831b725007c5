"""Whole-array NumPy statements of the five workloads, their seeded inputs and
the launch-geometry rules.  Test infrastructure only (see oracle/__init__.py).

Each expression is the check the reference's tests apply to a tile-wise kernel:
compute the same thing on the whole array with NumPy and compare
(python/hckernel/tests/test_examples.py:121,165 `np.dot`; :330-335 `np_softmax`).
"""

from __future__ import annotations

import numpy as np

# Shapes, seeded inputs and the bf16 bit-pattern helpers are shared with the
# benchmark and live in the package; re-exported here for the tests.
from hc_amd.workloads import (C1_N, C2_SHAPE, C3_SHAPE, C4_SHAPE, C5_MNK,  # noqa: F401
                              bf16_bits_to_f32, f32_to_bf16_bits, inputs_c1,
                              inputs_c2, inputs_c3, inputs_c4, inputs_c5)


# ---------------------------------------------------------------------------
# W0..W5
# ---------------------------------------------------------------------------
def np_copy_window(src: np.ndarray, dst: np.ndarray) -> np.ndarray:
    """Masked tile copy over the whole array: the common window is copied, the
    rest of dst is untouched (python/hckernel/kernel_api.py:297-342)."""
    out = dst.copy()
    win = tuple(slice(0, min(a, b)) for a, b in zip(src.shape, dst.shape))
    out[win] = src[win]
    return out


def np_add(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    return a + b


def np_fma_f16(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    f = np.float32
    return (a.astype(f) * b.astype(f) + c.astype(f)).astype(np.float16)


def np_softmax(x: np.ndarray) -> np.ndarray:
    # python/hckernel/tests/test_examples.py:330-335
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def np_quantize(x: np.ndarray):
    """Returns (q int8, scale fp32 per row).  A zero row is defined as scale 0,
    q 0; a NaN quotient as q 0."""
    xf = x.astype(np.float32)
    amax = np.abs(xf).max(axis=1, keepdims=True)
    scale = amax / np.float32(127)
    div = np.where(amax == 0, np.float32(1), scale)
    with np.errstate(invalid="ignore", divide="ignore"):
        qf = np.clip(np.rint(xf / div), -127, 127)
    q = np.where(np.isnan(qf), np.float32(0), qf).astype(np.int8)
    return q, scale[:, 0].astype(np.float32)


def np_gemm_bf16(a_bits: np.ndarray, bt_bits: np.ndarray, acc=np.float32):
    """fp32 (or fp64) matmul of the bf16 inputs; returns the unrounded product
    in `acc` precision.  B is column-major: C = A @ Bt.T."""
    a = bf16_bits_to_f32(a_bits).astype(acc)
    bt = bf16_bits_to_f32(bt_bits).astype(acc)
    return a @ bt.T


# ---------------------------------------------------------------------------
# Launch geometry
# ---------------------------------------------------------------------------
def suggest_block_size(global_sizes):
    """gpu-runtime/hip-runtime/src/Runtime.cpp:161-191 (x-first sizes)."""
    if not 1 <= len(global_sizes) <= 3:
        raise ValueError("nDims must be 1..3")
    budget = 1024
    out = []
    for g in global_sizes:
        if g > 1:
            l = min(g, budget)
            out.append(l)
            budget //= 1 << (l - 1).bit_length()
        else:
            out.append(1)
    return tuple(out)


def default_group_shape(work_shape):
    """Group shape the GPU path picks when none is given: the suggestion for
    the reversed work shape, reversed back
    (mlir/lib/Transforms/LowerHKernel.cpp:293-312)."""
    return tuple(reversed(suggest_block_size(tuple(reversed(work_shape)))))


def launch_geometry(work_shape, group_shape):
    """Grid and block (x, y, z) for Python-order shapes
    (mlir/lib/Transforms/LowerHKernel.cpp:314-354)."""
    counts = [-(-w // g) for w, g in zip(work_shape, group_shape)]
    grid = list(reversed(counts)) + [1] * (3 - len(counts))
    block = list(reversed(group_shape)) + [1] * (3 - len(group_shape))
    return tuple(grid), tuple(block)
