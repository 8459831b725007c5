"""Whole-array NumPy statements of the five workloads, their seeded inputs and
the launch-geometry rules.  Test infrastructure only (see oracle/__init__.py).

Each expression is the check the reference's tests apply to a tile-wise kernel:
compute the same thing on the whole array with NumPy and compare
(python/hckernel/tests/test_examples.py:121,165 `np.dot`; :330-335 `np_softmax`).
"""

from __future__ import annotations

import numpy as np

# Shapes, seeded inputs and bf16 bit patterns are stated here on their own: the
# package under test has the same figures in hc_amd/workloads.py for its
# benchmark, and tests/test_oracle_closed_forms.py holds the two against each
# other, so that a slip in either shows up instead of being shared.
C1_N = 16_777_259
C2_SHAPE = (8191, 8193)
C3_SHAPE = (4096, 8192)
C4_SHAPE = (16384, 4096)
C5_MNK = (4096, 4096, 4096)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round to nearest, ties to even; NaN stays a
    quiet NaN.  Written as a comparison of the discarded half word with one half
    unit in the last place, not as the carry trick the package uses."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    keep, rest = u >> 16, u & 0xFFFF
    up = (rest > 0x8000) | ((rest == 0x8000) & ((keep & 1) == 1))
    out = keep + up                       # a carry out of the mantissa is the next exponent (or inf)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, keep | 0x40, out).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    wide = np.zeros(np.shape(b) + (2,), np.uint16)
    wide[..., 1 if np.little_endian else 0] = b
    return wide.view(np.float32)[..., 0]


def inputs_c1(n: int = C1_N, seed: int = 1):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    b = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    return a, b


def inputs_c2(shape=C2_SHAPE, seed: int = 2):
    rng = np.random.default_rng(seed)
    return tuple(rng.standard_normal(shape, dtype=np.float32).astype(np.float16) for _ in range(3))


def inputs_c3(shape=C3_SHAPE, seed: int = 3):
    rng = np.random.default_rng(seed)
    return (np.float32(3.0) * rng.standard_normal(shape, dtype=np.float32),)


def inputs_c4(shape=C4_SHAPE, seed: int = 4):
    rng = np.random.default_rng(seed)
    n = rng.standard_normal(shape, dtype=np.float32)
    outlier = rng.random(shape, dtype=np.float32) < np.float32(0.01)
    return ((n * np.where(outlier, np.float32(50.0), np.float32(1.0))).astype(np.float16),)


def inputs_c5(mnk=C5_MNK, seed: int = 5):
    """A[M,K] and Bt[N,K] as bf16 bit patterns (B is column-major)."""
    m, n, k = mnk
    rng = np.random.default_rng(seed)
    a = np.float32(0.02) * rng.standard_normal((m, k), dtype=np.float32)
    bt = np.float32(0.02) * rng.standard_normal((n, k), dtype=np.float32)
    return f32_to_bf16_bits(a), f32_to_bf16_bits(bt)


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
