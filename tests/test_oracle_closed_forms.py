"""Pins the two statements of the workloads (NumPy whole-array expressions in
oracle/closed_forms.py, plain C in oracle/c/oracle.c) against each other and
against what the mathematics fixes: exact rational arithmetic, constructed
rounding ties, textbook special cases, exhaustive sweeps over fp16."""

from concurrent.futures import ThreadPoolExecutor
from fractions import Fraction

import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_array_equal

from oracle import c_oracle as co
from oracle import closed_forms as cf


# ---------------------------------------------------------------------------
# number formats
# ---------------------------------------------------------------------------
def test_half_to_float_all_65536_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = co.half_to_float(bits)
    nan = np.isnan(want)
    assert_array_equal(np.isnan(got), nan)
    assert_array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_round_trip_ties_and_random():
    bits = np.arange(65536, dtype=np.uint16)
    finite = bits[np.isfinite(bits.view(np.float16))]
    f = finite.view(np.float16).astype(np.float32)
    assert_array_equal(co.float_to_half(f), finite)          # exact values
    # midpoints between neighbouring halves are exactly representable in fp32
    # and must go to the even neighbour
    pos = np.sort(f[~np.signbit(f)])
    mid = ((pos[:-1].astype(np.float64) + pos[1:]) / 2).astype(np.float32)
    assert_array_equal(co.float_to_half(mid), mid.astype(np.float16).view(np.uint16))
    lo = pos[:-1].astype(np.float16).view(np.uint16)
    want_even = np.where(lo & 1, lo + 1, lo)
    assert_array_equal(co.float_to_half(mid), want_even)
    # just above / below each midpoint
    for nudge in (np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))):
        assert_array_equal(co.float_to_half(nudge), nudge.astype(np.float16).view(np.uint16))
    rng = np.random.default_rng(0)
    r = (rng.standard_normal(1_000_000, dtype=np.float32)
         * 10.0 ** rng.integers(-9, 6, 1_000_000)).astype(np.float32)
    with np.errstate(over="ignore"):
        assert_array_equal(co.float_to_half(r), r.astype(np.float16).view(np.uint16))
    edge = np.array([65504, 65519.99, 65520, 1e6, np.inf, -np.inf, 2.0 ** -25, 2.0 ** -24,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 0.0, -0.0], np.float32)
    with np.errstate(over="ignore"):
        assert_array_equal(co.float_to_half(edge), edge.astype(np.float16).view(np.uint16))


def test_bf16_rounding_two_statements_and_ties():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1_000_000, dtype=np.float32)
    assert_array_equal(cf.f32_to_bf16_bits(x), co.float_to_bf16(x))
    # ties: low 16 bits exactly 0x8000 -> even upper half
    hi = rng.integers(0x3F00, 0x4100, 4096).astype(np.uint32)
    tie = ((hi << 16) | 0x8000).view(np.float32)
    want = np.where(hi & 1, hi + 1, hi).astype(np.uint16)
    assert_array_equal(cf.f32_to_bf16_bits(tie), want)
    assert_array_equal(co.float_to_bf16(tie), want)
    # exactness of representable values, infinities, NaN stays NaN
    rep = (hi << 16).view(np.float32)
    assert_array_equal(cf.f32_to_bf16_bits(rep), hi.astype(np.uint16))
    sp = np.array([np.inf, -np.inf, np.nan, 0.0, -0.0], np.float32)
    for fn in (cf.f32_to_bf16_bits, co.float_to_bf16):
        b = fn(sp)
        assert b[0] == 0x7F80 and b[1] == 0xFF80 and b[3] == 0 and b[4] == 0x8000
        assert np.isnan(cf.bf16_bits_to_f32(b[2:3]))[0]


def test_the_benchmark_builds_the_inputs_the_oracle_describes():
    """The package keeps its own statement of the shapes, the seeded inputs and
    the bf16 bit patterns for its benchmark (hc_amd/workloads.py); the oracle's
    are written independently.  Same figures, same bytes."""
    from hc_amd import workloads as W
    assert (W.C1_N, W.C2_SHAPE, W.C3_SHAPE, W.C4_SHAPE, W.C5_MNK) == \
        (cf.C1_N, cf.C2_SHAPE, cf.C3_SHAPE, cf.C4_SHAPE, cf.C5_MNK)
    for ours, theirs in ((cf.inputs_c1(1001), W.inputs_c1(1001)), (cf.inputs_c2((37, 41)), W.inputs_c2((37, 41))),
                         (cf.inputs_c3((9, 64)), W.inputs_c3((9, 64))), (cf.inputs_c4((33, 128)), W.inputs_c4((33, 128))),
                         (cf.inputs_c5((64, 32, 128)), W.inputs_c5((64, 32, 128)))):
        assert len(ours) == len(theirs)
        for a, b in zip(ours, theirs):
            assert a.dtype == b.dtype and a.shape == b.shape
            assert_array_equal(a.view(np.uint8), b.view(np.uint8))
    # every fp32 whose upper half word is one of 4096 and whose lower one is any of 65536
    hi = np.random.default_rng(2).integers(0, 1 << 16, 4096).astype(np.uint32)
    hi[:8] = (0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7FC0, 0x0000, 0x8000, 0x007F)
    x = ((hi[:, None] << 16) | np.arange(1 << 16, dtype=np.uint32)[None, :]).view(np.float32)
    assert_array_equal(cf.f32_to_bf16_bits(x), W.f32_to_bf16_bits(x))
    bits = np.arange(1 << 16, dtype=np.uint16)
    assert_array_equal(cf.bf16_bits_to_f32(bits).view(np.uint32), W.bf16_bits_to_f32(bits).view(np.uint32))
    assert_array_equal(cf.bf16_bits_to_f32(bits).view(np.uint32), bits.astype(np.uint32) << 16)


# ---------------------------------------------------------------------------
# W1 / W2
# ---------------------------------------------------------------------------
# --- W0 masked window copy ------------------------------------------------------
def test_copy_window_known_answers():
    # python/hckernel/tests/test_kernel_sim.py:91-104: twelve values stored into
    # sixteen cells of -1 leave the last four cells alone
    src, dst = np.arange(12), np.full(16, -1)
    want = np.array(list(range(12)) + [-1] * 4)
    assert np.array_equal(cf.np_copy_window(src, dst), want)
    assert np.array_equal(dst, np.full(16, -1)), "np_copy_window must not write its argument"
    d2 = dst.reshape(1, 16).copy()
    co.copy2d(src.reshape(1, 12), d2)
    assert np.array_equal(d2[0], want)
    # a source wider than the destination is cut, not wrapped
    assert np.array_equal(cf.np_copy_window(np.arange(20), np.full(16, -1)), np.arange(16))

    # 2-D, ragged both ways, written out by hand: 3 x 5 source into a 4 x 3
    # destination of -7 copies a 3 x 3 window
    src = np.array([[0, 1, 2, 3, 4], [10, 11, 12, 13, 14], [20, 21, 22, 23, 24]], np.int32)
    want = np.array([[0, 1, 2], [10, 11, 12], [20, 21, 22], [-7, -7, -7]], np.int32)
    dst = np.full((4, 3), -7, np.int32)
    assert np.array_equal(cf.np_copy_window(src, dst), want)
    co.copy2d(src, dst)
    assert np.array_equal(dst, want)


@pytest.mark.parametrize("itemsize_dtype", [np.int8, np.float16, np.int32, np.float64])
def test_copy2d_strided_views_leave_poison_alone(itemsize_dtype):
    # windows of larger poison-filled arrays, strided in both dimensions: every
    # byte outside the common window keeps its poison, inside it equals the source
    rng = np.random.default_rng(11)
    big_s = rng.integers(1, 100, (9, 14)).astype(itemsize_dtype)
    big_d = np.full((11, 17), 101, itemsize_dtype)
    src = big_s[1:8:2, 2:13:3]            # 4 x 4, strides (2 rows, 3 elements)
    dst = big_d[2:11:3, 1:16:2]           # 3 x 8, strides (3 rows, 2 elements)
    expect = big_d.copy()
    for r in range(3):
        for c in range(4):
            expect[2 + 3 * r, 1 + 2 * c] = big_s[1 + 2 * r, 2 + 3 * c]
    assert np.array_equal(cf.np_copy_window(src, dst), expect[2:11:3, 1:16:2])
    co.copy2d(src, dst)
    assert np.array_equal(big_d, expect)
    # transposed source (column-major walk)
    d2 = np.full((5, 5), 101, itemsize_dtype)
    co.copy2d(big_s.T[:3, :2], d2)
    assert np.array_equal(d2[:3, :2], big_s[:2, :3].T) and (d2[3:] == 101).all() and (d2[:, 2:] == 101).all()


def test_add_two_statements_bit_equal():
    a, b = cf.inputs_c1(100_003)
    assert_array_equal(co.add_f32(a, b).view(np.uint32), cf.np_add(a, b).view(np.uint32))


def test_fma_two_statements_bit_equal_and_exact_cases():
    a, b, c = cf.inputs_c2((97, 1031))
    assert_array_equal(co.fma_f16(a, b, c).view(np.uint16), cf.np_fma_f16(a, b, c).view(np.uint16))
    # the fp32 product of two halves is exact: compare with rational arithmetic
    rng = np.random.default_rng(7)
    idx = rng.integers(0, a.size, 300)
    d = cf.np_fma_f16(a, b, c).ravel()
    for i in idx:
        x, y, z = (Fraction(float(v.ravel()[i])) for v in (a, b, c))
        s32 = np.float32(float(x * y + z))   # one rounding: exact -> fp32 (via an exact double? see below)
        # x*y+z has at most 22+11 significant bits spread over < 2^40: exact in double
        assert np.float16(s32) == d[i]
    # specials: denormal results, overflow to inf, signed zero
    h = np.float16
    sa = np.array([[6e-8, 6e-8, 300, -300, 0.0, 1.0, 2.0 ** -14]], h)
    sb = np.array([[1.0, 0.5, 300, 300, -1.0, 1.0, 0.5]], h)
    sc = np.array([[0.0, 0.0, 0.0, 0.0, 0.0, 2.0 ** -11, 0.0]], h)
    with np.errstate(over="ignore"):
        want = cf.np_fma_f16(sa, sb, sc)
    got = co.fma_f16(sa, sb, sc)
    assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    assert want[0, 2] == np.inf and want[0, 3] == -np.inf
    assert want[0, 5] == h(1.0)              # 1 + 2^-11 is a tie -> even (1.0)


# ---------------------------------------------------------------------------
# W3 softmax
# ---------------------------------------------------------------------------
def test_softmax_statements_agree_and_invariants():
    (x,) = cf.inputs_c3((64, 1000))
    y_np = cf.np_softmax(x)
    y_c32 = co.softmax(x)
    y_c64 = co.softmax(x, f64=True)
    assert_allclose(y_np, y_c64, rtol=2e-6, atol=0)
    assert_allclose(y_c32, y_c64, rtol=2e-5, atol=0)
    assert_allclose(y_c64.astype(np.float64).sum(1), 1.0, atol=1e-6)
    # shift invariance: adding a constant per row changes nothing (up to the
    # rounding of x + c itself, so use a power of two)
    assert_allclose(co.softmax(x + np.float32(8.0), f64=True), y_c64, rtol=1e-5)
    # order preserved within a row
    r = 5
    order = np.argsort(x[r], kind="stable")
    assert (np.diff(y_c64[r][order]) >= 0).all()


def test_softmax_textbook_special_cases():
    # two-element rows: the logistic function
    d = np.linspace(-20, 20, 81, dtype=np.float32)
    x = np.stack([np.zeros_like(d), d], axis=1)
    want = 1.0 / (1.0 + np.exp(-d.astype(np.float64)))
    for y in (cf.np_softmax(x), co.softmax(x), co.softmax(x, f64=True)):
        assert_allclose(y[:, 1], want, rtol=3e-7)
    # constant rows: exactly 1/n when n is a power of two
    x = np.full((3, 64), 1.25, np.float32)
    for y in (cf.np_softmax(x), co.softmax(x), co.softmax(x, f64=True)):
        assert_array_equal(y, np.full((3, 64), 1 / 64, np.float32))
    # the reference's own input (test_examples.py:322-335), float64 there
    m, n = 30, 25
    a = (2 * np.arange(m * n).reshape(m, n) / (m * n)).astype(np.float32)
    assert_allclose(cf.np_softmax(a), co.softmax(a, f64=True), rtol=1e-6)


# ---------------------------------------------------------------------------
# W4 quantize
# ---------------------------------------------------------------------------
def rn32(fr: Fraction) -> float:
    """Correctly rounded (nearest even) binary32 value of a rational, by
    integer arithmetic; magnitudes here stay in the normal range."""
    if fr == 0:
        return 0.0
    s = -1 if fr < 0 else 1
    fr = abs(fr)
    e = fr.numerator.bit_length() - fr.denominator.bit_length()
    if Fraction(2) ** e > fr:
        e -= 1
    scaled = fr / Fraction(2) ** (e - 23)       # in [2^23, 2^24)
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n & 1):
        n += 1
    return s * float(n) * 2.0 ** (e - 23)


def rint_even(v: float) -> int:
    f = int(np.floor(v))
    d = v - f
    if d > 0.5 or (d == 0.5 and f & 1):
        return f + 1
    return f


def test_quantize_two_statements_bit_equal():
    (x,) = cf.inputs_c4((257, 1000))
    q_np, s_np = cf.np_quantize(x)
    q_c, s_c = co.quantize(x)
    assert_array_equal(q_np, q_c)
    assert_array_equal(s_np.view(np.uint32), s_c.view(np.uint32))
    assert np.abs(q_np).max() == 127          # every row attains +-127


def test_quantize_against_exact_rational_arithmetic():
    # every finite fp16 x with |x| <= amax, for three absmax values, against
    # fl32(amax/127), fl32(x/scale) and round-half-even computed with integers
    bits = np.arange(0x7C00, dtype=np.uint16)
    for amax in (np.float16(1.0), np.float16(3.141), np.float16(50.25)):
        pos = bits[bits.view(np.float16) <= amax].view(np.float16)
        row = np.concatenate([pos, -pos])[None, :]
        q, s = cf.np_quantize(row)
        scale = rn32(Fraction(float(amax)) / 127)
        assert float(s[0]) == scale
        step = max(1, row.size // 4000)       # every value would take minutes
        for i in range(0, row.size, step):
            quo = rn32(Fraction(float(row[0, i])) / Fraction(scale))
            assert int(q[0, i]) == max(-127, min(127, rint_even(quo))), (amax, row[0, i])


def test_quantize_constructed_ties_round_to_even():
    # amax = 127 * 2^e makes scale = 2^e exactly, so x = (k + 1/2) * 2^e hits
    # the tie for every k
    for e in (-3, 0, 2):
        ks = np.array([0, 1, 2, 3, 4, 125, 126], np.float32)
        x = np.concatenate([(ks + 0.5), -(ks + 0.5), [127.0]]).astype(np.float32) * np.float32(2.0 ** e)
        row = x.astype(np.float16)[None, :]
        assert_array_equal(row.astype(np.float32), x[None, :])      # representable
        want = np.array([0, 2, 2, 4, 4, 126, 126, 0, -2, -2, -4, -4, -126, -126, 127], np.int8)
        for q, s in (cf.np_quantize(row), co.quantize(row)):
            assert s[0] == np.float32(2.0 ** e)
            assert_array_equal(q[0], want)


def test_quantize_special_rows():
    h = np.float16
    rows = np.array([[0, 0, -0.0, 0],            # zero row: scale 0, q 0
                     [1, np.nan, -2, 0.5],       # NaN row: scale NaN, q 0
                     [np.inf, 1, -1, -np.inf],   # inf row: scale inf, q 0
                     [6e-8, -6e-8, 0, 3e-8]], h)  # subnormal absmax; 3e-8 rounds up to 2^-24
    for q, s in (cf.np_quantize(rows), co.quantize(rows)):
        assert s[0] == 0 and np.isnan(s[1]) and np.isinf(s[2])
        assert_array_equal(q[:3], np.zeros((3, 4), np.int8))
        assert_array_equal(q[3], [127, -127, 0, 127])
    qa, sa = cf.np_quantize(rows)
    qb, sb = co.quantize(rows)
    assert_array_equal(qa, qb)
    assert_array_equal(sa.view(np.uint32)[[0, 2, 3]], sb.view(np.uint32)[[0, 2, 3]])


def test_quotient_shortcut_is_exact_for_every_fp16_pair():
    """The kernel replaces x / scale by a reciprocal and one fma correction.
    Sweep every (x, absmax) pair of finite fp16 values with |x| <= absmax: the
    quotient never differs in value (only in the sign of zero for x = -0), the
    rounded integer never differs, and |rint| never exceeds 127."""
    edges = list(range(1, 0x7C00, 0x100)) + [0x7C00]
    co.lib()
    with ThreadPoolExecutor(8) as pool:
        res = list(pool.map(lambda i: co.quotient_shortcut_mismatches(edges[i], edges[i + 1]),
                            range(len(edges) - 1)))
    bad, zero, bad_int, checked, maxq = (sum(r[0] for r in res), sum(r[1] for r in res),
                                         sum(r[2] for r in res), sum(r[3] for r in res),
                                         max(r[4] for r in res))
    assert checked == 1_007_713_278
    assert bad == 0 and bad_int == 0
    assert zero == 0x7C00 - 1            # one -0 per absmax value
    assert maxq == 127.0


# ---------------------------------------------------------------------------
# W5 GEMM
# ---------------------------------------------------------------------------
def test_gemm_exact_integer_matrices():
    # small integers are exact in bf16, and every partial sum is an integer
    # below 2^24, so all statements must give the integer product bit for bit
    rng = np.random.default_rng(5)
    m, n, k = 33, 47, 96
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    bt = rng.integers(-8, 9, (n, k)).astype(np.float32)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    ab, bb = cf.f32_to_bf16_bits(a), cf.f32_to_bf16_bits(bt)
    assert_array_equal(cf.bf16_bits_to_f32(ab), a)
    for acc in (np.float32, np.float64):
        assert_array_equal(cf.np_gemm_bf16(ab, bb, acc).astype(np.float32), want)
    for f64 in (False, True):
        c16, c32 = co.gemm_bf16(ab, bb, f64=f64)
        assert_array_equal(c32, want)
        assert_array_equal(c16, cf.f32_to_bf16_bits(want))
    # a transposed operand or a dropped K tail would show
    assert not np.array_equal(cf.np_gemm_bf16(ab, bb[:, ::-1].copy()), want)


def test_gemm_reference_dot_recipe_and_statements():
    # input recipe of test_examples.py:113-121 (16 x 32 x 64), rounded to bf16
    m, n, k = 16, 32, 64
    a = (2 * np.arange(m * k).reshape(m, k) / (m * k)).astype(np.float32)
    b = (np.arange(n * k).reshape(k, n) / (n * k)).astype(np.float32)
    ab, bb = cf.f32_to_bf16_bits(a), cf.f32_to_bf16_bits(b.T.copy())
    exact = cf.np_gemm_bf16(ab, bb, np.float64)
    _, c64 = co.gemm_bf16(ab, bb, f64=True)
    _, c32 = co.gemm_bf16(ab, bb, f64=False)
    assert_allclose(c64, exact, rtol=1e-7)
    assert_allclose(c32, exact, rtol=1e-5)
    assert_allclose(cf.np_gemm_bf16(ab, bb), exact, rtol=1e-5)
    # against the unrounded fp64 dot the bf16 inputs cost at most ~2^-8 each
    assert_allclose(exact, np.dot(a.astype(np.float64), b.astype(np.float64)), rtol=1e-2)


def test_gemm_seeded_inputs_statistics():
    ab, bb = cf.inputs_c5((64, 48, 256))
    a = cf.bf16_bits_to_f32(ab)
    assert abs(a.std() - 0.02) < 2e-3
    c = cf.np_gemm_bf16(ab, bb, np.float64)
    assert abs(c.std() - 0.02 * 0.02 * 16) < 1.5e-3      # sigma^2 * sqrt(K)


# ---------------------------------------------------------------------------
# launch geometry
# ---------------------------------------------------------------------------
BLOCK_CASES = [   # x-first global sizes -> block, worked by hand from the rule
    ((16_777_259,), (1024,)),
    ((8193, 8191), (1024, 1)),
    ((27, 1), (27, 1)),
    ((27,), (27,)),
    ((64, 256), (64, 16)),
    ((813, 111), (813, 1)),
    ((20, 10), (20, 10)),
    ((72, 1, 1), (72, 1, 1)),
    ((1, 1, 1), (1, 1, 1)),
    ((3, 5, 7), (3, 5, 7)),
    ((100, 100, 100), (100, 8, 1)),
    ((1, 4096, 2), (1, 1024, 1)),
]


@pytest.mark.parametrize("global_sizes,block", BLOCK_CASES)
def test_suggest_block_size_table(global_sizes, block):
    assert cf.suggest_block_size(global_sizes) == block
    rc, got = co.suggest_block_size(global_sizes)
    assert rc == 0 and got == block
    assert np.prod(block) <= 1024


def test_suggest_block_size_rejects_bad_rank():
    assert co.suggest_block_size(())[0] == 1
    assert co.suggest_block_size((1, 2, 3, 4))[0] == 1
    with pytest.raises(ValueError):
        cf.suggest_block_size((1, 2, 3, 4))


@pytest.mark.parametrize("work,group,grid,block", [
    ((16_777_259,), (256,), (65537, 1, 1), (256, 1, 1)),
    ((8191, 8193), (1, 256), (33, 8191, 1), (256, 1, 1)),
    ((111, 813), (1, 813), (1, 111, 1), (813, 1, 1)),
    ((4, 5, 6), (2, 5, 4), (2, 1, 2), (4, 5, 2)),
])
def test_launch_geometry_reverses_python_dims(work, group, grid, block):
    assert cf.launch_geometry(work, group) == (grid, block)
    assert co.launch_geometry(work, group) == (grid, block)


def test_default_group_shape_examples():
    assert cf.default_group_shape((16_777_259,)) == (1024,)
    assert cf.default_group_shape((8191, 8193)) == (1, 1024)
    assert cf.default_group_shape((256, 64)) == (16, 64)
    assert cf.default_group_shape((1, 27)) == (1, 27)
