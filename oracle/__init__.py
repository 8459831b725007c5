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
  * hcsim behaviour that follows from numpy.ma internals (in-place operators
    on partially active tiles, loads from already masked tiles, domain
    masking of / // % **, NumPy functions and reductions on tiles,
    compressed()/repr, every installed operator on int32 / float32 / bool
    tiles, stores of numpy.ma results, Python and NumPy scalars next to a
    tile): tests/golden/sim_golden.json, written by
    tests/golden/make_sim_golden.py from the reference's own simulator running
    the bodies of tests/golden/sim_cases.py; tests/test_oracle_sim_golden.py
    demands equal bytes wherever the reference returns a value.  The vectors
    are numpy.ma's behaviour at the NumPy version recorded in the file (the
    reference pins none): under NumPy >= 2 a bare Python scalar promotes a
    float32 tile to float64 (`tile * 0.5`), a NumPy scalar of the tile's type
    does not.
  * W0 copy (np_copy_window, oracle_copy2d): the reference's arange(12) / -1
    known answer (python/hckernel/tests/test_kernel_sim.py:91-104), a ragged
    2-D window written out by hand, strided poison-filled views.
"""
