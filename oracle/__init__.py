"""CPU oracle for the hc_amd kernels.  TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import anything from this package; hc_amd/ never does, and has no CPU
fallback of any kind.

Contents
--------
closed_forms   whole-array NumPy expressions for each workload (the checks the
               reference's tests perform, python/hckernel/tests/test_examples.py:
               121,165,330-335), seeded input generators, launch-geometry rules.
c_oracle       ctypes binding of oracle/c/oracle.c, an independent plain-C
               statement of the same results (hand-written fp16/bf16
               conversions, IEEE division, rint).
hcsim          host executor restating the reference's tile/mask simulator
               (python/hckernel/kernel_api.py, kernel_sim.py): runs a kernel
               body group by group on NumPy arrays.

Pinning status (what each part is checked against, see tests/test_oracle_*.py):
  * hcsim geometry, masked load/store, allocators, scopes, barrier order,
    symbol binding, tunables: the reference's own known answers
    (python/hckernel/tests/test_kernel_sim.py, all 25 functions) and example
    kernels (test_examples.py: reductions, dot, softmax, pairwise distance,
    implicit GEMM).
  * closed forms W1/W2/W4 (add, fma, quantize): the plain-C statement,
    exhaustive fp16 conversion round trips, constructed rounding ties.
  * W3 softmax: the reference's np_softmax on its own 30x25 input, an fp64
    statement, rows-sum-to-one and shift invariance.
  * W5 GEMM: exact small-integer matrices, the reference's 16x32x64 dot
    input recipe (test_examples.py:113-121), fp64 accumulation.
  * parity unpinned: behaviour that follows only from numpy.ma internals
    (in-place operators on partially active tiles, loads from already masked
    tiles, domain masking of divide/sqrt/log, np.dot on masked tiles,
    compressed()/repr).  hcsim follows the documented numpy.ma rules for
    these, but no reference test or fixture fixes them.
  * parity unpinned: a bare Python scalar next to a tile (`tile * 0.5`).
    numpy.ma turns the scalar into a 0-d float64 array, so under NumPy >= 2
    the simulator computes such an expression in float64, under NumPy 1.x in
    the tile's type; the reference pins no NumPy version and no test covers
    it.  The GPU front-end gives the scalar the tile's type (what a plain
    ndarray does); tests that compare the two write scalars as np.float32(..)
    / np.float16(..), which both sides treat alike.
"""
