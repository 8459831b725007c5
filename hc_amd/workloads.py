"""The five benchmark workloads: shapes, seeded synthetic inputs, algorithmic
work, and bf16 <-> fp32 bit-pattern helpers (NumPy has no bfloat16).

Inputs come from numpy.random.default_rng(seed), generated in fp32 and then cast,
so that the same arrays can be rebuilt anywhere from the seed alone.
"""

from __future__ import annotations

import numpy as np

# Sizes of the five benchmark configurations.
C1_N = 16_777_259
C2_SHAPE = (8191, 8193)
C3_SHAPE = (4096, 8192)
C4_SHAPE = (16384, 4096)
C5_MNK = (4096, 4096, 4096)


# ---------------------------------------------------------------------------
# bf16 as uint16 bit patterns (NumPy has no bfloat16)
# ---------------------------------------------------------------------------
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round to nearest even on the upper 16 bits; NaN stays a quiet NaN."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    rounded = ((u + (np.uint32(0x7FFF) + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), rounded)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------------------
# Seeded inputs: numpy.random.default_rng(seed), generated in fp32 then cast.
# ---------------------------------------------------------------------------
def inputs_c1(n: int = C1_N, seed: int = 1):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    b = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    return a, b


def inputs_c2(shape=C2_SHAPE, seed: int = 2):
    rng = np.random.default_rng(seed)
    return tuple(rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
                 for _ in range(3))


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



# Algorithmic work per launch: bytes that must cross HBM once (memory-bound
# kernels) or floating-point operations (GEMM).
def work_c1(n: int = C1_N) -> int:
    return 3 * 4 * n


def work_c2(shape=C2_SHAPE) -> int:
    return 4 * 2 * shape[0] * shape[1]


def work_c3(shape=C3_SHAPE) -> int:
    return 2 * 4 * shape[0] * shape[1]


def work_c4(shape=C4_SHAPE) -> int:
    return (2 + 1) * shape[0] * shape[1] + 4 * shape[0]


def work_c5(mnk=C5_MNK) -> int:
    return 2 * mnk[0] * mnk[1] * mnk[2]
