"""Kernels written against the reference's Python API, run on the GPU through
`@kernel` (tracing front-end -> typed C entry points) and checked against the
CPU oracle.  The three copy kernels are the bodies of the reference's own GPU
end-to-end tests (python/hckernel/tests/test_e2e.py:57-136), imported through
the reference's package name."""

import zlib

import numpy as np
import pytest
import sympy
from numpy.testing import assert_allclose, assert_array_equal

from hckernel.kernel import *          # noqa: F401,F403  (the reference's import line)
from hc_amd import runtime as rt
from oracle import closed_forms as cf
from oracle.hcsim import kernel as sim_kernel

pytestmark = pytest.mark.gpu

DT = typename.DT
_copy_shapes = [(1, 27), (1, 72), (1, 128), (10, 20), (111, 813), (256, 64), (256, 1024)]


def cdiv(a, b):
    return (a + b - 1) // b


def dev_pair(shape):
    a = np.arange(shape[0] * shape[1], dtype=np.int32).reshape(shape)
    return a, rt.to_device(a), rt.to_device(np.zeros_like(a))


@pytest.mark.parametrize("shape", _copy_shapes)
def test_copy(shape):
    W, H = sym.W, sym.H

    @kernel(work_shape=(W, H), backend="rocm", device="hip:0")
    def copy_kernel(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x, y = group.work_offset
        val = group.load(src[x:, y:], shape=group.shape)
        group.store(dst[x:, y:], val)

    a, da, db = dev_pair(shape)
    copy_kernel(da, db)
    assert_array_equal(db.to_host(), a)


@pytest.mark.parametrize("shape", _copy_shapes)
@pytest.mark.parametrize("unroll", [1, 2, 4])
@pytest.mark.parametrize("vec", [False, True])
def test_copy_unroll_and_vec(shape, unroll, vec):
    W, H, V = sym.W, sym.H, sym.V
    H1 = sympy.ceiling(H / V)

    @kernel(work_shape=(W, H1), backend="rocm", device="hip:0", literals=[V] if vec else ())
    def copy_kernel(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT], v: V):
        x, y = group.work_offset
        ld = group.vload if vec else group.load
        val = ld(src[x:, y * V:], shape=(group.shape[0], group.shape[1] * V))
        group.store(dst[x:, y * V:], val)

    a, da, db = dev_pair(shape)
    copy_kernel(da, db, unroll)
    assert_array_equal(db.to_host(), a)


def test_copy_with_torch_tensors():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    W, H = sym.W, sym.H

    @kernel(work_shape=(W, H))
    def copy_kernel(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x, y = group.work_offset
        group.store(dst[x:, y:], group.load(src[x:, y:], shape=group.shape))

    a = torch.arange(111 * 813, dtype=torch.int32).reshape(111, 813).to("cuda")
    b = torch.zeros_like(a)
    torch.cuda.synchronize()
    copy_kernel(a, b)
    torch.testing.assert_close(b, a)
    # a strided (non-contiguous) source window
    c = torch.zeros((111, 400), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    copy_kernel.plan(a[:, :400], c)
    W2, H2 = sym.W2, sym.H2

    @kernel(work_shape=(W2, H2))
    def copy_window(group: CurrentGroup, src: Buffer[W2, H2, DT], dst: Buffer[W2, H2, DT]):
        x, y = group.work_offset
        group.store(dst[x:, y:], group.load(src[x:, y:], shape=group.shape))

    copy_window(a[:, :400], c)
    torch.testing.assert_close(c, a[:, :400])


def test_elementwise_and_reduction_bodies_on_torch_tensors():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    R, Cc, N = sym.R, sym.C, sym.N

    @kernel(work_shape=(R, Cc))
    def gated(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta, tb = gr.load(a[x:, y:], shape=gr.shape), gr.load(b[x:, y:], shape=gr.shape)
        gr.store(out[x:, y:], np.maximum(ta, np.float32(0)) * tb + ta)

    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn(257, 1031, device="cuda", generator=g)
    b = torch.randn(257, 1031, device="cuda", generator=g)
    out = torch.full_like(a, 7.0)
    torch.cuda.synchronize()
    gated(a, b, out)
    want = torch.clamp_min(a, 0) * b + a              # two roundings, like the kernel
    assert torch.equal(out, want)
    # a column window of the tensors: strided rows
    out2 = torch.full_like(a, 7.0)
    torch.cuda.synchronize()
    gated(a[:, :500], b[:, :500], out2[:, :500])
    assert torch.equal(out2[:, :500], want[:, :500]) and bool((out2[:, 500:] == 7.0).all())

    @kernel(work_shape=N, group_shape=256)
    def sumsq(gr: CurrentGroup, x: Buffer[N, DT], result: Buffer[1, DT]):
        o, t = gr.work_offset[0], None
        t = gr.load(x[o:], shape=gr.shape[0])
        atomic_ref(result)[0] += (t * t).sum()

    v = torch.randn(1_000_003, device="cuda", generator=g, dtype=torch.float16)
    res = torch.zeros(1, device="cuda")
    torch.cuda.synchronize()
    sumsq(v, res)
    sq = (v * v).double()                              # fp16 products, as the tile arithmetic does
    assert abs(res.item() - sq.sum().item()) <= 64 * 2.0 ** -24 * sq.sum().item()


def test_vector_add_same_body_on_gpu_and_on_the_host_executor():
    N = sym.N

    def body(gr, a, b, c):
        o = gr.work_offset[0]
        gr.store(c[o:], gr.load(a[o:], shape=gr.shape[0]) + gr.load(b[o:], shape=gr.shape[0]))

    def annotated(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT]):
        body(gr, a, b, c)

    n = 100_003
    a, b = cf.inputs_c1(n)
    dc = rt.DeviceArray((n,), np.float32)
    kernel(work_shape=N, group_shape=256)(annotated)(rt.to_device(a), rt.to_device(b), dc)
    host = np.zeros(n, np.float32)
    sim_kernel(work_shape=N, group_shape=256)(annotated)(a, b, host)     # tile by tile on the CPU
    assert_array_equal(dc.to_host().view(np.uint32), host.view(np.uint32))
    assert_array_equal(host.view(np.uint32), cf.np_add(a, b).view(np.uint32))


def test_fused_multiply_add_2d_ragged():
    R, Cc = sym.R, sym.C
    f = np.float32

    @kernel(work_shape=(R, Cc))
    def fma(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], c: Buffer[R, Cc, DT],
            d: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta, tb, tc = (gr.load(v[x:, y:], shape=gr.shape) for v in (a, b, c))
        gr.store(d[x:, y:], (ta.astype(f) * tb.astype(f) + tc.astype(f)).astype(np.float16))

    a, b, c = cf.inputs_c2((127, 1031))
    dd = rt.DeviceArray(a.shape, np.float16)
    fma(rt.to_device(a), rt.to_device(b), rt.to_device(c), dd)
    assert_array_equal(dd.to_host().view(np.uint16), cf.np_fma_f16(a, b, c).view(np.uint16))


def test_softmax_body_of_the_reference_example():
    M, N, GM, MI = sym.M, sym.N, sym.GM, sym.MI

    @kernel(work_shape=cdiv(M, MI), group_shape=GM, tunables=TunableParam(MI, 1, range(1, 8)))
    def softmax(gr: CurrentGroup, a: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m_start = gr.work_offset[0] * MI
        m_block = gr.shape[0] * MI
        a_view = gr.load(a[m_start:, :], shape=(m_block, N))
        exp = np.exp(a_view - a_view.max(axis=1, keepdims=True))
        gr.store(out[m_start:, :], exp / (exp.sum(axis=1, keepdims=True)))

    m, n = 30, 25                      # the reference's input, in fp32
    a = (2 * np.arange(m * n).reshape(m, n) / (m * n)).astype(np.float32)
    out = rt.DeviceArray(a.shape, np.float32)
    softmax(rt.to_device(a), out, 8)
    assert_allclose(out.to_host(), cf.np_softmax(a.astype(np.float64)), rtol=2e-6)
    (x,) = cf.inputs_c3((257, 8192))
    out = rt.DeviceArray(x.shape, np.float32)
    softmax(rt.to_device(x), out, 8)
    assert_allclose(out.to_host(), cf.np_softmax(x), rtol=1e-5, atol=1e-9)


def test_row_quantize_bit_exact():
    M, N, GM = sym.M, sym.N, sym.GM

    @kernel(work_shape=M, group_shape=GM)
    def quant(gr: CurrentGroup, x: Buffer[M, N, DT], q: Buffer[M, N, DT], scale: Buffer[M, DT],
              g: GM):
        m0 = gr.work_offset[0]
        xf = gr.load(x[m0:, :], shape=(gr.shape[0], N)).astype(np.float32)
        s = np.abs(xf).max(axis=1, keepdims=True) / np.float32(127)
        gr.store(q[m0:, :], np.clip(np.rint(xf / s), -127, 127).astype(np.int8))
        gr.store(scale[m0:], s[:, 0])

    (x,) = cf.inputs_c4((513, 4096))
    dq, ds = rt.DeviceArray(x.shape, np.int8), rt.DeviceArray((x.shape[0],), np.float32)
    quant(rt.to_device(x), dq, ds, 4)
    q, s = cf.np_quantize(x)
    assert_array_equal(dq.to_host(), q)
    assert_array_equal(ds.to_host().view(np.uint32), s.view(np.uint32))


@pytest.mark.parametrize("mnk,gshape", [((512, 256, 256), (16, 16)), ((100, 200, 300), (8, 8))])
def test_blocked_dot_binds_to_the_mfma_gemm(mnk, gshape):
    M, N, K = sym.M, sym.N, sym.K
    GM, GN, MI, NI, KB = sym.GM, sym.GN, sym.MI, sym.NI, sym.KB
    tun = (TunableParam(MI, 4, range(1, 8)), TunableParam(NI, 4, range(1, 8)),
           TunableParam(KB, 64, range(8, 128)))
    KI = cdiv(K, KB)

    @kernel(work_shape=(cdiv(M, MI), cdiv(N, NI)), group_shape=(GM, GN), tunables=tun)
    def dot(gr: CurrentGroup, a: Buffer[M, K, DT], bt: Buffer[N, K, DT], out: Buffer[M, N, DT],
            gshape: (GM, GN)):
        m0, n0 = gr.work_offset[0] * MI, gr.work_offset[1] * NI
        mb, nb = gr.shape[0] * MI, gr.shape[1] * NI
        r = gr.zeros(shape=(mb, nb), dtype=np.float32)
        for k in range(KI):
            r += np.dot(gr.load(a[m0:, k * KB:], shape=(mb, KB)),
                        gr.load(bt[n0:, k * KB:], shape=(nb, KB)).T)
        gr.store(out[m0:, n0:], r)

    ab, bb = cf.inputs_c5(mnk)
    dc = rt.DeviceArray((mnk[0], mnk[1]), np.uint16, bf16=True)
    dot(rt.to_device(ab, bf16=True), rt.to_device(bb, bf16=True), dc, gshape)
    want = cf.np_gemm_bf16(ab, bb, np.float32)
    assert_allclose(cf.bf16_bits_to_f32(dc.to_host()), want, rtol=1e-2,
                    atol=1e-2 * 0.02 * 0.02 * np.sqrt(mnk[2]))


# ---------------------------------------------------------------------------
# arbitrary elementwise bodies: the same body on the GPU (fused map kernel) and
# on the host executor, bit for bit
# ---------------------------------------------------------------------------
def random_expression(rng, depth, dtype):
    """A Python function of three tiles built from operations whose fp32 / fp16
    results are exactly defined (no transcendental functions), together with its
    source text.  Denominators are kept away from zero: the host executor's
    masked arithmetic would otherwise leave those elements unwritten.  Scalars
    are written as K(value) with K the tiles' own type: a bare Python float
    would make numpy.ma, and with it the host executor, compute in float64."""
    def leaf():
        return rng.choice(["a", "b", "c"])

    def gen(d):
        if d == 0 or rng.random() < 0.15:
            return leaf()
        kind = rng.integers(0, 12)
        x = gen(d - 1)
        if kind <= 2:
            return f"({x} {rng.choice(['+', '-', '*'])} {gen(d - 1)})"
        if kind == 3:
            return f"({x} / (np.abs({gen(d - 1)}) + K(1.0)))"
        if kind == 4:
            return f"np.{rng.choice(['maximum', 'minimum'])}({x}, {gen(d - 1)})"
        if kind == 5:
            return f"(-{x})"
        if kind == 6:
            return f"np.abs({x})"
        if kind == 7:
            return f"np.sqrt(np.abs({x}))"
        if kind == 8:
            return f"np.rint({x} * K(3.0))"
        if kind == 9:
            return f"np.clip({x}, -1.5, 2.25)"
        if kind == 10:
            return f"(K({rng.choice(['0.3', '2.0', '-1.25'])}) {rng.choice(['+', '-', '*', '/'])} " \
                   f"(np.abs({x}) + K(0.5)))"
        return f"({x} {rng.choice(['+', '-', '*', '/'])} K({rng.choice(['0.7', '4.0', '-0.125'])}))"

    text = gen(depth)
    while text in ("a", "b", "c"):
        text = gen(depth)
    return eval(f"lambda a, b, c: {text}", {"np": np, "K": dtype}), text


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("layout", ["flat", "ragged2d", "window"])
def test_random_elementwise_bodies_match_the_host_executor(dtype, layout):
    rng = np.random.default_rng({"flat": 1, "ragged2d": 2, "window": 3}[layout] * 10 +
                                np.dtype(dtype).itemsize)
    N, R, Cc, R2, C2 = sym.N, sym.R, sym.C, sym.R2, sym.C2
    if layout == "flat":
        shape = big = (100_003,)
    elif layout == "ragged2d":
        shape = big = (37, 1031)
    else:
        shape, big = (36, 1024), (40, 1100)         # a window of larger arrays
    vals = [(rng.uniform(0.5, 2.0, big) * rng.choice([-1.0, 1.0], big)).astype(dtype)
            for _ in range(3)]
    tried = bound = 0
    while bound < 12:
        expr, text = random_expression(rng, 3, dtype)
        tried += 1

        if len(shape) == 1:
            def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT],
                     out: Buffer[N, DT]):
                o, g = gr.work_offset[0], gr.shape[0]
                gr.store(out[o:], expr(gr.load(a[o:], shape=g), gr.load(b[o:], shape=g),
                                       gr.load(c[o:], shape=g)))
            deco = dict(work_shape=N, group_shape=256)
        else:
            def body(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT],
                     c: Buffer[R, Cc, DT], out: Buffer[R2, C2, DT]):
                x, y = gr.work_offset
                gr.store(out[x:, y:], expr(*(gr.load(v[x:, y:], shape=gr.shape)
                                            for v in (a, b, c))))
            deco = dict(work_shape=(shape[0], shape[1]), group_shape=(4, 64))
        poison = np.full(shape if layout != "window" else (40, 1040), 7.5, dtype)
        host = poison.copy()
        with np.errstate(all="ignore"):
            sim_kernel(**deco)(body)(*vals, host)
        dout = rt.to_device(poison)
        try:
            kernel(**deco)(body)(*[rt.to_device(v) for v in vals], dout)
        except NoNativeKernel as exc:                  # deeper than the stack: not bound
            assert "stack" in str(exc) or "operations" in str(exc), text
            continue
        bound += 1
        got = dout.to_host()
        nan = np.isnan(host)
        assert (np.isnan(got) == nan).all(), text
        u = np.uint32 if dtype == np.float32 else np.uint16
        assert_array_equal(got.view(u)[~nan], host.view(u)[~nan], err_msg=text)
    assert tried < 40


def test_elementwise_body_with_transcendental_functions():
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        x, y = gr.load(a[o:], shape=g), gr.load(b[o:], shape=g)
        one = np.float32(1)
        gr.store(out[o:], x / (one + np.exp(-x)) + np.tanh(y) * np.log(np.abs(y) + one))

    rng = np.random.default_rng(21)
    n = 70_001
    a, b = (rng.standard_normal(n).astype(np.float32) * 3 for _ in range(2))
    host = np.zeros(n, np.float32)
    sim_kernel(work_shape=N, group_shape=256)(body)(a, b, host)
    dout = rt.DeviceArray((n,), np.float32)
    kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), dout)
    # exp / tanh / log are within 2 ulp of NumPy's; the sum of two terms of
    # either sign keeps that as an absolute error relative to the larger term
    assert_allclose(dout.to_host(), host, rtol=2e-6, atol=2e-6)


# ---------------------------------------------------------------------------
# reductions through atomic_ref (python/hckernel/tests/test_examples.py:31-71)
# ---------------------------------------------------------------------------
def _reduction_kernels(deco):
    WS, GS, N = sym.WS, sym.GS, sym.N
    TN = TunableParam(N, 2, range(1, 64))

    def reduction_1(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], gshape: GS):
        a_view = gr.load(a[gr.work_offset[0] * N:], shape=gr.size * N)
        atomic_ref(result)[0] += a_view.sum()

    def reduction_2(group: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], gshape: GS):
        temp_result = group.zeros(group.size, dtype=a.dtype)
        for i in range(N):
            work_offset = group.work_offset[0] * N + i * group.size
            a_view = group.load(a[work_offset:], shape=group.size)
            temp_result += a_view
        atomic_ref(result)[0] += temp_result.sum()

    args = dict(work_shape=cdiv(WS, N), group_shape=GS, tunables=TN)
    return [deco(**args)(f) for f in (reduction_1, reduction_2)]


def test_reference_reductions_known_answer():
    a = np.arange(0, 20).astype(np.float32)          # the reference's input; the sum is exact
    for gpu, host in zip(_reduction_kernels(kernel), _reduction_kernels(sim_kernel)):
        result = rt.to_device(np.zeros(1, np.float32))
        gpu(rt.to_device(a), result, 8)
        want = np.zeros(1, np.float32)
        host(a, want, 8)
        assert result.to_host()[0] == want[0] == a.sum() == 190.0
        gpu(rt.to_device(a), result, 8)               # += : accumulates on top
        assert result.to_host()[0] == 380.0


@pytest.mark.parametrize("n", [1, 7, 8, 2047, 100_003, 16_777_259])
def test_reductions_of_random_data_within_fp32_summation_error(n):
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(np.float32)
    exact = float(a.astype(np.float64).sum())
    # any order of n fp32 additions is within n * 2^-24 * sum|a| of the exact sum;
    # the kernel adds eight values per lane, then trees: far inside that bound
    bound = 64 * 2.0 ** -24 * float(np.abs(a).astype(np.float64).sum()) + 1e-30
    for k in _reduction_kernels(kernel):
        result = rt.to_device(np.zeros(1, np.float32))
        k.parametrize({sym.N: 4})(rt.to_device(a), result, 64)
        assert abs(float(result.to_host()[0]) - exact) <= bound


def test_dot_product_through_the_map_sum_kernel():
    WS = sym.WS

    def dot(gr: CurrentGroup, a: Buffer[WS, DT], b: Buffer[WS, DT], result: Buffer[4, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        atomic_ref(result)[2] += (gr.load(a[o:], shape=g) * gr.load(b[o:], shape=g)).sum()

    rng = np.random.default_rng(33)
    n = 1_000_003
    for dtype in (np.float32, np.float16):
        a, b = (rng.standard_normal(n).astype(dtype) for _ in range(2))
        result = rt.to_device(np.array([1, 2, 3, 4], np.float32))
        kernel(work_shape=WS, group_shape=256)(dot)(rt.to_device(a), rt.to_device(b), result)
        got = result.to_host()
        assert_array_equal(got[[0, 1, 3]], [1, 2, 4])            # neighbours untouched
        if dtype == np.float16:                                   # fp16 tiles: the product rounds
            prod = (a * b).astype(np.float64)
        else:
            prod = (a * b).astype(np.float64)                     # fp32 product, then summed
        assert abs(float(got[2]) - 3.0 - prod.sum()) <= 64 * 2.0 ** -24 * np.abs(prod).sum()


def test_pairwise_distance_body_of_the_reference_example():
    from test_kernel_frontend import _pairwise_kernel
    m, n, d = 16, 32, 8                                 # the reference's input, in fp32
    a = (2 * np.arange(m * d).reshape(m, d) / (m * d)).astype(np.float32)
    b = (np.arange(n * d).reshape(n, d) / (n * d)).astype(np.float32)
    out = rt.to_device(np.full((m, n), -1, np.float32))
    _pairwise_kernel(kernel)(rt.to_device(a), rt.to_device(b), out, (8, 8))
    host = np.zeros((m, n), np.float32)
    _pairwise_kernel(sim_kernel)(a, b, host, (8, 8))
    want = np.linalg.norm(a[:, None, :].astype(np.float64) - b[None, :, :], axis=2)
    assert_allclose(host, want, rtol=1e-6)
    assert_allclose(out.to_host(), want, rtol=1e-6, atol=1e-7)
    # ragged sizes, several panels of d, tunables
    rng = np.random.default_rng(41)
    m, n, d = 201, 333, 77
    a, b = rng.standard_normal((m, d)).astype(np.float32), rng.standard_normal((n, d)).astype(np.float32)
    out = rt.to_device(np.full((m, n), -1, np.float32))
    _pairwise_kernel(kernel).parametrize({sym.MI: 2, sym.NI: 3})(rt.to_device(a), rt.to_device(b),
                                                               out, (8, 4))
    want = np.linalg.norm(a[:, None, :].astype(np.float64) - b[None, :, :], axis=2)
    assert_allclose(out.to_host(), want, rtol=2e-6)
    # a point and itself: exactly zero, not the residue of a cancellation
    out = rt.to_device(np.full((m, m), -1, np.float32))
    _pairwise_kernel(kernel)(rt.to_device(a), rt.to_device(a), out, (8, 8))
    assert (np.diag(out.to_host()) == 0).all()


def test_autotune_flow_of_the_language_reference(tmp_path):
    # docs/langref.md:516-571: tunables on the decorator, autotune, parametrize, save / load
    from hc_amd.kernel import autotune
    WS, GS, N = sym.WS, sym.GS, sym.N
    TP = TunableParam

    @kernel(work_shape=cdiv(WS, N), group_shape=GS,
            tunables=(TP(GS, 64, range(64, 1024, 320)), TP(N, 16, range(16, 256, 80))))
    def reduction(group: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT]):
        temp_result = group.zeros(group.size, dtype=a.dtype)
        for i in range(N):
            work_offset = group.work_offset[0] * N + i * group.size
            temp_result += group.load(a[work_offset:], shape=group.size)
        atomic_ref(result)[0] += temp_result.sum()

    a = np.arange(200_000, dtype=np.float32) % 7
    scratch = rt.to_device(np.zeros(1, np.float32))
    tparams = autotune(reduction, rt.to_device(a), scratch, iters=3, warmup=1)
    assert tparams[GS] in range(64, 1024, 320) and tparams[N] in range(16, 256, 80)
    assert tparams.device.startswith("gfx950") and tparams.microseconds > 0
    tparams.save(tmp_path / "reduction.json")
    tuned = reduction.parametrize(autotune.load(tmp_path / "reduction.json"))
    result = rt.to_device(np.zeros(1, np.float32))
    tuned(rt.to_device(a), result)
    assert result.to_host()[0] == a.sum()               # small integers: exact in any order

    # a kernel family with variants: the chosen one is applied around the call
    Nn = sym.NN

    @kernel(work_shape=Nn, group_shape=256)
    def vadd(gr: CurrentGroup, x: Buffer[Nn, DT], y: Buffer[Nn, DT], z: Buffer[Nn, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        gr.store(z[o:], gr.load(x[o:], shape=g) + gr.load(y[o:], shape=g))

    x, y = cf.inputs_c1(1_000_003)
    dx, dy, dz = rt.to_device(x), rt.to_device(y), rt.DeviceArray(x.shape, np.float32)
    # the tuner tries variants for its own thread only: what the process has
    # selected is still selected afterwards
    rt.set_variant("add", 2)
    vadd(dx, dy, dz)
    selected = rt.last_kernel_name()
    tp = autotune(vadd, dx, dy, dz, iters=5, warmup=1)
    assert set(tp.variants) <= {"add"} and all(1 <= v <= 8 for v in tp.variants.values())
    vadd(dx, dy, dz)
    assert rt.last_kernel_name() == selected
    vadd.parametrize(tp)(dx, dy, dz)
    assert_array_equal(dz.to_host().view(np.uint32), cf.np_add(x, y).view(np.uint32))
    rt.set_variant("add", 0)
    vadd(dx, dy, dz)
    assert rt.last_kernel_name() == "hcamd_add_f32_v4_nt"     # the default is back


def test_blocked_dot_on_torch_bfloat16_tensors():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    M, N, K, KB = sym.M, sym.N, sym.K, sym.KB
    KI = cdiv(K, KB)

    @kernel(work_shape=(cdiv(M, 4), cdiv(N, 4)), group_shape=(16, 16),
            tunables=TunableParam(KB, 64, range(8, 128)))
    def dot(gr: CurrentGroup, a: Buffer[M, K, DT], bt: Buffer[N, K, DT], out: Buffer[M, N, DT]):
        m0, n0 = gr.work_offset[0] * 4, gr.work_offset[1] * 4
        mb, nb = gr.shape[0] * 4, gr.shape[1] * 4
        r = gr.zeros(shape=(mb, nb), dtype=np.float32)
        for k in range(KI):
            r += np.dot(gr.load(a[m0:, k * KB:], shape=(mb, KB)),
                        gr.load(bt[n0:, k * KB:], shape=(nb, KB)).T)
        gr.store(out[m0:, n0:], r)

    g = torch.Generator(device="cuda").manual_seed(5)
    a = (0.02 * torch.randn(512, 768, device="cuda", generator=g)).bfloat16()
    bt = (0.02 * torch.randn(256, 768, device="cuda", generator=g)).bfloat16()
    out = torch.zeros(512, 256, device="cuda", dtype=torch.bfloat16)
    torch.cuda.synchronize()
    dot(a, bt, out)
    assert rt.last_kernel_name().startswith("hcamd_gemm_bf16_p256x256")
    want = a.float() @ bt.float().T
    torch.testing.assert_close(out.float(), want, rtol=1e-2, atol=1e-2 * 0.02 * 0.02 * 768 ** 0.5)


def test_blocked_dot_fp16_same_body_on_gpu_and_host_executor():
    # the K-blocked dot of python/hckernel/tests/test_examples.py:124-165, with B given as Bt
    M, N, K = sym.M, sym.N, sym.K
    GM, GN, MI, NI, KB = sym.GM, sym.GN, sym.MI, sym.NI, sym.KB
    tun = (TunableParam(MI, 4, range(1, 8)), TunableParam(NI, 4, range(1, 8)),
           TunableParam(KB, 64, range(8, 128)))
    KI = cdiv(K, KB)

    def dot(gr: CurrentGroup, a: Buffer[M, K, DT], bt: Buffer[N, K, DT], out: Buffer[M, N, DT],
            gshape: (GM, GN)):
        m0, n0 = gr.work_offset[0] * MI, gr.work_offset[1] * NI
        mb, nb = gr.shape[0] * MI, gr.shape[1] * NI
        r = gr.zeros(shape=(mb, nb), dtype=np.float32)
        for k in range(KI):
            r += np.dot(gr.load(a[m0:, k * KB:], shape=(mb, KB)).astype(np.float32),
                        gr.load(bt[n0:, k * KB:], shape=(nb, KB)).astype(np.float32).T)
        gr.store(out[m0:, n0:], r)

    deco = dict(work_shape=(cdiv(M, MI), cdiv(N, NI)), group_shape=(GM, GN), tunables=tun)
    rng = np.random.default_rng(9)
    m, n, k = 256, 128, 192
    a = (0.5 * rng.standard_normal((m, k))).astype(np.float16)
    bt = (0.5 * rng.standard_normal((n, k))).astype(np.float16)
    host = np.zeros((m, n), np.float16)
    sim_kernel(**deco)(dot)(a, bt, host, (16, 16))
    out = rt.DeviceArray((m, n), np.float16)
    kernel(**deco)(dot)(rt.to_device(a), rt.to_device(bt), out, (16, 16))
    assert rt.last_kernel_name() == "hcamd_gemm_f16_p128x128_w2x2"
    # both accumulate in fp32 (in different orders) and round once to fp16
    assert_allclose(out.to_host().astype(np.float32), host.astype(np.float32),
                    rtol=2.0 ** -10, atol=2.0 ** -10)


def test_unsupported_body_raises_instead_of_running_on_the_cpu():
    N = sym.N

    @kernel(work_shape=N, group_shape=64)
    def scaled(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(c[o:], (gr.load(a[o:], shape=gr.shape[0]) * 3.0).sum())

    a = rt.to_device(np.ones(1000, np.float32))
    c = rt.to_device(np.zeros(1000, np.float32))
    with pytest.raises(NoNativeKernel):
        scaled(a, c)
    assert_array_equal(c.to_host(), np.zeros(1000, np.float32))     # untouched


# ---------------------------------------------------------------------------
# mapped loads and stores (python/hckernel/tests/test_examples.py:168-258)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n,c,nf,stride,tiles", [
    (1, 1, 1, 1, {}), (2, 3, 2, 2, {}), (4, 3, 8, 3, {}), (4, 1, 8, 1, {}),
    (3, 2, 5, 1, {sym.TN: 2, sym.TNF: 3}), (9, 3, 10, 2, {sym.TN: 4, sym.TNF: 7, sym.KB: 8})])
def test_implicit_gemm_convolution_of_the_reference_examples(n, c, nf, stride, tiles):
    from hc_amd.kernel import create_mapping
    from oracle import hcsim
    from test_kernel_frontend import _conv_kernel, conv_direct
    rng = np.random.default_rng(n + 10 * c + 100 * nf + stride)
    h = w = 4
    hf = wf = 2
    ho, wo = (h - hf) // stride + 1, (w - wf) // stride + 1
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    f = rng.standard_normal((nf, c, hf, wf)).astype(np.float32)
    out = rt.to_device(np.zeros((n, nf, ho, wo), np.float32))
    k = _conv_kernel(kernel, create_mapping, stride).parametrize(tiles)
    k(rt.to_device(x), rt.to_device(f), out)
    assert rt.last_kernel_name().startswith("hcamd_gather_gemm_f32_")
    want = np.zeros((n, nf, ho, wo), np.float32)
    _conv_kernel(sim_kernel, hcsim.create_mapping, stride).parametrize(tiles)(x, f, want)
    # K = c * hf * wf <= 12 products per output, summed in fp32 in another order
    assert_allclose(out.to_host(), want, rtol=1e-5, atol=1e-6)
    assert_allclose(out.to_host(), conv_direct(x, f, stride), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("fuse", [0, 1, 2, 4, 16])
def test_convolution_at_a_larger_size_with_full_tiles(fuse):
    from hc_amd.kernel import create_mapping
    from test_kernel_frontend import _conv_kernel, conv_direct
    rng = np.random.default_rng(2024)
    n, c, hw, nf, hf = 70, 6, 13, 66, 3          # (hw - hf) divisible by both strides
    x = rng.standard_normal((n, c, hw, hw)).astype(np.float32)
    f = rng.standard_normal((nf, c, hf, hf)).astype(np.float32)

    # the example's mappings assume 2 x 2 filters only through HF * WF; 3 x 3 works the same
    for stride, tiles in ((1, {sym.TN: 63, sym.TNF: 63, sym.KB: 16}), (2, {sym.TN: 32, sym.TNF: 40})):
        ho = (hw - hf) // stride + 1
        out = rt.to_device(np.full((n, nf, ho, ho), np.nan, np.float32))
        rt.set_variant("gather_fuse", fuse)
        try:
            _conv_kernel(kernel, create_mapping, stride).parametrize(tiles)(
                rt.to_device(x), rt.to_device(f), out)
        finally:
            rt.set_variant("gather_fuse", 0)
        if fuse:
            assert rt.last_kernel_name().endswith(f"_g{fuse}")
        got = out.to_host()
        assert not np.isnan(got).any()
        assert_allclose(got, conv_direct(x, f, stride), rtol=1e-4, atol=(c * hf * hf + 2) * 2.0 ** -22)


def test_float32_dot_with_row_major_b():
    """The blocked dot of python/hckernel/tests/test_examples.py:74-121 on fp32
    arrays: binds to the gathered product with identity mappings."""
    M, N, K, GM, GN, KB = sym.M, sym.N, sym.K, sym.GM, sym.GN, sym.KB
    KI = cdiv(K, KB)

    def make(deco):
        @deco(work_shape=(M, N), group_shape=(GM, GN), tunables=TunableParam(KB, 8, (8, 16)))
        def dot(gr: CurrentGroup, a: Buffer[M, K, DT], b: Buffer[K, N, DT], out: Buffer[M, N, DT],
                gshape: (GM, GN)):
            m0, n0 = gr.work_offset
            r = gr.zeros(shape=gr.shape, dtype=out.dtype)
            for k in range(KI):
                r += np.dot(gr.load(a[m0:, k * KB:], shape=(gr.shape[0], KB)),
                            gr.load(b[k * KB:, n0:], shape=(KB, gr.shape[1])))
            gr.store(out[m0:, n0:], r)
        return dot

    rng = np.random.default_rng(31)
    a = rng.standard_normal((130, 77)).astype(np.float32)
    b = rng.standard_normal((77, 95)).astype(np.float32)
    out = rt.to_device(np.zeros((130, 95), np.float32))
    make(kernel)(rt.to_device(a), rt.to_device(b), out, (64, 64))
    assert rt.last_kernel_name().startswith("hcamd_gather_gemm_f32_")
    want = np.zeros((130, 95), np.float32)
    make(sim_kernel)(a, b, want, (64, 64))
    assert_allclose(out.to_host(), want, rtol=1e-4, atol=79 * 2.0 ** -22)
    assert_allclose(out.to_host(), a.astype(np.float64) @ b, rtol=1e-4, atol=79 * 2.0 ** -22)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_convolution_on_16_bit_arrays(dtype):
    from hc_amd.kernel import create_mapping
    from test_kernel_frontend import _conv_kernel, conv_direct
    rng = np.random.default_rng(99)
    n, c, hw, nf, hf = 20, 5, 9, 12, 3
    x32 = rng.standard_normal((n, c, hw, hw)).astype(np.float32)
    f32 = rng.standard_normal((nf, c, hf, hf)).astype(np.float32)
    ho = hw - hf + 1
    if dtype == "float16":
        x, f = x32.astype(np.float16), f32.astype(np.float16)
        dx, df = rt.to_device(x), rt.to_device(f)
        out = rt.to_device(np.zeros((n, nf, ho, ho), np.float16))
        xv, fv = x.astype(np.float32), f.astype(np.float32)
    else:
        xb, fb = cf.f32_to_bf16_bits(x32), cf.f32_to_bf16_bits(f32)
        dx, df = rt.to_device(xb, bf16=True), rt.to_device(fb, bf16=True)
        out = rt.to_device(np.zeros((n, nf, ho, ho), np.uint16), bf16=True)
        xv, fv = cf.bf16_bits_to_f32(xb), cf.bf16_bits_to_f32(fb)
    _conv_kernel(kernel, create_mapping, 1)(dx, df, out)
    assert "_f16_" in rt.last_kernel_name() or "_bf16_" in rt.last_kernel_name()
    raw = out.to_host()
    got = raw.astype(np.float32) if dtype == "float16" else cf.bf16_bits_to_f32(raw)
    eps = 2.0 ** -11 if dtype == "float16" else 2.0 ** -8
    assert_allclose(got, conv_direct(xv, fv, 1), rtol=1.01 * eps, atol=(c * hf * hf + 2) * 2.0 ** -22)


def test_autotune_of_the_convolution_example():
    """The tunables of python/hckernel/tests/test_examples.py:216-218 (tile sizes
    and K block) and the block shapes of the kernel it binds to are timed; the
    tuned kernel computes the same convolution."""
    from hc_amd.kernel import autotune, create_mapping
    from test_kernel_frontend import _conv_kernel, conv_direct
    rng = np.random.default_rng(5)
    n, c, hw, nf, hf = 24, 4, 10, 16, 3
    x = rng.standard_normal((n, c, hw, hw)).astype(np.float32)
    f = rng.standard_normal((nf, c, hf, hf)).astype(np.float32)
    ho = hw - hf + 1
    dx, df = rt.to_device(x), rt.to_device(f)
    out = rt.to_device(np.zeros((n, nf, ho, ho), np.float32))
    conv = _conv_kernel(kernel, create_mapping, 1)
    tp = autotune(conv, dx, df, out, max_trials=6, iters=3, warmup=1)
    assert 1 <= tp[sym.TN] < 64 and 1 <= tp[sym.TNF] < 64 and 8 <= tp[sym.KB] < 128
    assert set(tp.variants) <= {"gather"}
    out2 = rt.to_device(np.full((n, nf, ho, ho), np.nan, np.float32))
    conv.parametrize(tp)(dx, df, out2)
    rt.set_variant("gather", 0)
    assert_allclose(out2.to_host(), conv_direct(x, f, 1), rtol=1e-4, atol=(c * hf * hf + 2) * 2.0 ** -22)


# ---------------------------------------------------------------------------
# bodies with reductions along rows -> hcamdLaunchRowProgram
# ---------------------------------------------------------------------------
# (one, two and four chunks per lane of the chain kernels, 64 ... 1024 lanes to a row, more rows
# than workgroups; 20,003 columns: the general kernel)
@pytest.mark.parametrize("rows,n", [(37, 200), (64, 4096), (9, 4104), (5, 20_003), (4400, 1000),
                                    (12, 16384), (3, 32768)])
@pytest.mark.parametrize("name", ["layernorm", "rmsnorm_half", "log_softmax_t", "row_norms", "spread",
                                  "unit_rows", "log_sum_exp"])
def test_row_reduction_bodies_match_the_simulator(name, rows, n):
    """The same body on the GPU and on the CPU simulator.  fp32 results agree
    to rtol 2e-5 (sums run in a different order, exp/log differ in the last
    bit); the fp16 output of rmsnorm_half to one fp16 ulp."""
    from test_kernel_frontend import _row_bodies, _row_case
    host = _row_case(name, rows, n, seed=rows)
    want = host[-1].copy()
    with np.errstate(all="ignore"):                     # masked rows of the last group
        _row_bodies(sim_kernel)[name](*host[:-1], want, 8)
    out = rt.DeviceArray(host[-1].shape, host[-1].dtype).fill_bytes32(0xA5A5A5A5)
    _row_bodies(kernel)[name](*[rt.to_device(a) for a in host[:-1]], out, 8)
    # (the two normalisations over dense rows of whole chunks have kernels of their own)
    assert rt.last_kernel_name().startswith(("hcamd_row_program", "hcamd_layer_norm_f32", "hcamd_rms_norm_f16"))
    if name == "layernorm" and n % 4 == 0 and n >= 8 and n <= 32768:
        assert rt.last_kernel_name().startswith("hcamd_layer_norm_f32")
    if name == "rmsnorm_half" and n % 8 == 0:
        assert rt.last_kernel_name().startswith("hcamd_rms_norm_f16")
    got = out.to_host()
    if got.dtype == np.float16:
        assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=1.1e-3)
    else:
        assert_allclose(got, want, rtol=2e-5, atol=2e-6)


# (a wave per row with and without 16-byte rows, a workgroup per row, rows past the last group)
@pytest.mark.parametrize("rows,n", [(8, 5), (37, 200), (21, 1031), (9, 4104), (70, 4608)])
def test_reductions_over_deactivated_elements_follow_numpy_ma_on_the_gpu(rows, n):
    """Row reductions over elements the data deactivates (zero divisors), row
    scalars that are deactivated themselves (a quotient of sums with a zero
    divisor, a root of a negative sum, a mean that is not finite), and what
    follows from them, on the GPU and on the CPU simulator: the same elements
    written (the rest keep the poison), the same values to the bound of sums
    added in another order, per-row results of deactivated rows included."""
    from test_kernel_frontend import POISON, _masked_row_bodies, _masked_row_case
    gpu, sim = _masked_row_bodies(kernel), _masked_row_bodies(sim_kernel)
    a, b = _masked_row_case(rows, n, seed=rows)
    da, db = rt.to_device(a), rt.to_device(b)
    for name, (body, per_row) in gpu.items():
        shape = (rows,) if per_row else (rows, n)
        want = np.full(shape, POISON)
        with np.errstate(all="ignore"):
            sim[name][0](a, b, want, 8)
        out = rt.to_device(np.full(shape, POISON))
        body(da, db, out, 8)
        elementwise = name in ("bare_scaled_quotient", "bare_one_minus_quotient",
                               "bare_python_one_minus_quotient", "bare_sqrt_of_quotient")
        assert rt.last_kernel_name().startswith(("hcamd_fmap", "hcamd_map") if elementwise
                                                else "hcamd_row_program_w"), (name, rt.last_kernel_name())
        got = out.to_host()
        assert_array_equal(got == POISON, want == POISON, err_msg=name)
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=name)
        assert_allclose(got, want, rtol=1e-4, atol=1e-5, err_msg=name)


@pytest.mark.parametrize("name", ["layernorm", "rmsnorm_half"])
@pytest.mark.parametrize("rows,n", [(64, 4096), (37, 200), (5, 20_003)])
def test_normalisations_of_rows_with_a_mean_that_is_not_finite(name, rows, n):
    """numpy.ma's mean of a row with an inf or a NaN is deactivated.  The layer
    normalisation computes from a tile: nothing of such a row is stored.  The
    root-mean-square one computes from x.astype(float32), a bare numpy.ma
    array, and is written in full: such a row gets what numpy.ma leaves in a
    deactivated quotient, the dividend x.  The kernels of their own (dense rows
    of whole chunks) and the general one do the same."""
    from test_kernel_frontend import _row_bodies, _row_case
    host = _row_case(name, rows, n, seed=rows)
    x = host[0]
    x[1, n // 3] = np.inf
    x[2, 0] = np.nan
    want = np.full(host[-1].shape, -77, host[-1].dtype)
    with np.errstate(all="ignore"):
        _row_bodies(sim_kernel)[name](*host[:-1], want, 8)
    out = rt.to_device(np.full(host[-1].shape, -77, host[-1].dtype))
    _row_bodies(kernel)[name](*[rt.to_device(v) for v in host[:-1]], out, 8)
    got = out.to_host()
    if name == "layernorm":
        assert (want[1] == -77).all() and (want[2] == -77).all() and (want[0] != -77).all()
    else:
        assert_array_equal(want[1].view(np.uint16), x[1].view(np.uint16))
        assert_array_equal(want[2].view(np.uint16), x[2].view(np.uint16))
    assert_array_equal(got == -77, want == -77)
    assert_array_equal(np.isnan(got), np.isnan(want))
    if got.dtype == np.float16:
        assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=1.1e-3)
    else:
        assert_allclose(got, want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("rows,n,gn", [(37, 200, 64), (3000, 4096, 512), (70_000, 24, 24),
                                       (513, 1031, 1031)])
@pytest.mark.parametrize("name", ["col_sums", "col_max_abs", "col_min", "col_means", "col_norms",
                                  "col_rms", "col_var", "col_std"])
def test_column_reduction_bodies_match_the_simulator(name, rows, n, gn):
    """The same body on the GPU and on the CPU simulator: maxima and minima bit
    for bit, sums within the fp32 bound of adding `rows` terms in another
    order, what is computed from a sum to the same relative bound.  The
    variance and the standard deviation are two reductions, the second reading
    the first one's result from a temporary vector."""
    from test_kernel_frontend import _col_bodies
    rng = np.random.default_rng(rows + n)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    y = rng.standard_normal((rows, n)).astype(np.float32)
    want = np.zeros(n, np.float32)
    _col_bodies(sim_kernel)[name](x, y, want, gn)
    out = rt.DeviceArray((n,), np.float32).fill_bytes32(0xA5A5A5A5)
    _col_bodies(kernel)[name](rt.to_device(x), rt.to_device(y), out, gn)
    # (the bands of a sum with a simple post program fold on a kernel of their own)
    assert rt.last_kernel_name().startswith(("hcamd_map_reduce_cols", "hcamd_cols_fold_f32"))
    got = out.to_host()
    if name in ("col_max_abs", "col_min"):
        assert_array_equal(got, want)
    else:
        x64, y64 = x.astype(np.float64), y.astype(np.float64)
        d64 = x64 - y64
        terms = {"col_sums": x64 * y64, "col_means": x64 + y64, "col_norms": d64 ** 2,
                 "col_rms": x64 * x64, "col_var": (x64 - x64.mean(axis=0)) ** 2,
                 "col_std": (d64 - d64.mean(axis=0)) ** 2}[name]
        rel = (rows + 2) * 2.0 ** -23 * np.abs(terms).sum(axis=0) / np.maximum(np.abs(terms.sum(axis=0)), 1e-30)
        assert (np.abs(got - want) <= (rel + 4e-7) * np.abs(want) + 1e-30).all()


@pytest.mark.parametrize("rows,n,gn", [(37, 200, 64), (2000, 1031, 256), (5000, 24, 24)])
@pytest.mark.parametrize("name", ["batch_norm", "col_softmax", "centre"])
def test_tiles_computed_from_their_own_column_reductions_match_the_simulator(name, rows, n, gn):
    """The reductions run first, each into a temporary vector; the tile is then
    one elementwise pass.  fp32 results agree with the simulator to the bound
    of sums added in another order."""
    from test_kernel_frontend import _col_tile_bodies
    rng = np.random.default_rng(rows + n)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    w = rng.standard_normal((rows, n)).astype(np.float32)
    want = np.zeros((rows, n), np.float32)
    _col_tile_bodies(sim_kernel)[name](x, w, want, gn)
    out = rt.DeviceArray((rows, n), np.float32).fill_bytes32(0xA5A5A5A5)
    _col_tile_bodies(kernel)[name](rt.to_device(x), rt.to_device(w), out, gn)
    assert rt.last_kernel_name().startswith(("hcamd_row_program", "hcamd_map"))
    got = out.to_host()
    assert_allclose(got, want, rtol=(rows + 8) * 2.0 ** -23, atol=(rows + 8) * 2.0 ** -23)


def test_softmax_with_a_temperature_is_a_row_program_and_plain_softmax_keeps_its_kernel():
    M, N, GM = sym.M, sym.N, sym.GM

    def make(deco, temperature):
        @deco(work_shape=M, group_shape=GM)
        def softmax(gr: CurrentGroup, a: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            t = gr.load(a[m0:, :], shape=(mb, N))
            if temperature != 1.0:
                t = t / np.float32(temperature)
            e = np.exp(t - t.max(axis=1, keepdims=True))
            gr.store(out[m0:, :], e / e.sum(axis=1, keepdims=True))
        return softmax

    x = (np.random.default_rng(3).standard_normal((100, 1000)) * 4).astype(np.float32)
    dx = rt.to_device(x)
    for temperature, name in ((1.0, "hcamd_softmax"), (0.7, "hcamd_row_program")):
        want = np.zeros_like(x)
        with np.errstate(all="ignore"):
            make(sim_kernel, temperature)(x, want, 8)
        out = rt.DeviceArray(x.shape, np.float32)
        make(kernel, temperature)(dx, out, 8)
        assert rt.last_kernel_name().startswith(name), rt.last_kernel_name()
        assert_allclose(out.to_host(), want, rtol=1e-5, atol=1e-30)


def test_random_row_expressions_match_the_simulator():
    """Random bodies mixing elementwise arithmetic and reductions along rows,
    on the GPU and on the CPU simulator (rtol 1e-4: sums in a different order,
    exp in the last bit, and cancellation in expressions like x - mean(x))."""
    from test_kernel_frontend import random_row_body, random_row_expression, random_row_operands
    rng = np.random.default_rng(77)
    shapes = [(1, 1), (3, 7), (21, 96), (40, 513), (17, 2048), (5, 4099), (3, 9001)]
    bound = tried = 0
    while bound < 28:
        expr, text, per_row = random_row_expression(rng, 3)
        tried += 1
        rows, n = shapes[tried % len(shapes)]
        host = random_row_operands(rng, rows, n, per_row)
        out = rt.DeviceArray(host[-1].shape, np.float32).fill_bytes32(0xA5A5A5A5)
        try:
            random_row_body(kernel, expr, per_row)(*[rt.to_device(a) for a in host[:-1]], out, 8)
        except NoNativeKernel as exc:
            assert any(w in str(exc) for w in ("stack", "row scalars", "operations", "passes", "numpy.ma leaves",
                                               "arrays")), (text, str(exc))
            continue
        assert rt.last_kernel_name().startswith("hcamd_row_program"), text
        bound += 1
        want = host[-1].copy()
        with np.errstate(all="ignore"):
            random_row_body(sim_kernel, expr, per_row)(*host[:-1], want, 8)
        scale = 1.0 + float(np.abs(want).max())
        assert_allclose(out.to_host(), want, rtol=1e-4, atol=1e-5 * scale,
                        err_msg=f"{text} on {rows} x {n}")
    assert tried < 90


# ---------------------------------------------------------------------------
# Asynchronous launches, events, vload, per-thread variants
# ---------------------------------------------------------------------------
def test_dependent_launches_without_synchronisation_between_two_events():
    """A chain of launches enqueued with sync=False on one queue, each reading
    what the one before wrote (the reference synchronises after every launch,
    python/cpp/py-runtime/src/GpuRuntime.cpp:60-69; here the queue keeps the
    order).  The events bracket the chain on the queue; the host waits once."""
    import time
    N = sym.N
    f = np.float32

    @kernel(work_shape=N, group_shape=256)
    def axpy(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(c[o:], gr.load(a[o:], shape=gr.shape[0]) * f(0.5) + gr.load(b[o:], shape=gr.shape[0]))

    @kernel(work_shape=N, group_shape=256)
    def total(gr: CurrentGroup, x: Buffer[N, DT], result: Buffer[1, DT]):
        o = gr.work_offset[0]
        atomic_ref(result)[0] += gr.load(x[o:], shape=gr.shape[0]).sum()

    n = 8_000_003
    x0, y0 = cf.inputs_c1(n)
    ctx = rt.default_context("hip:0")
    dx, dy = rt.to_device(x0), rt.to_device(y0)
    t1, t2, t3 = (rt.DeviceArray((n,), np.float32) for _ in range(3))
    cell = rt.to_device(np.zeros(1, np.float32))
    axpy(dx, dy, t1)                                   # traced and built outside the timed part
    total(t1, cell)
    cell2 = rt.to_device(np.zeros(1, np.float32))
    ctx.synchronize()
    start, stop = rt.Event(ctx), rt.Event(ctx)
    wall0 = time.perf_counter()
    start.record()
    axpy(dx, dy, t1, sync=False)                       # t1 = x/2 + y
    axpy(t1, dx, t2, sync=False)                       # t2 = t1/2 + x
    axpy(t2, t1, t3, sync=False)                       # t3 = t2/2 + t1
    total(t3, cell2, sync=False)                       # sum of t3
    stop.record()
    enqueued = time.perf_counter() - wall0
    stop.synchronize()
    wall = time.perf_counter() - wall0
    elapsed = start.elapsed_ms(stop) * 1e-3
    h = f(0.5)
    w1 = x0 * h + y0
    w2 = w1 * h + x0
    w3 = w2 * h + w1
    assert_array_equal(t3.to_host().view(np.uint32), w3.view(np.uint32))
    ref = w3.astype(np.float64)
    assert abs(float(cell2.to_host()[0]) - ref.sum()) <= 64 * 2.0 ** -24 * np.abs(ref).sum()
    assert 0.0 < elapsed < wall, (elapsed, wall)
    # three 96 MB passes and a reduction cannot be done before they were enqueued
    # unless the launches had blocked the host
    assert elapsed > 30e-6 and enqueued < wall


def test_vload_bodies_take_the_16_byte_per_lane_kernels():
    W, H, V = sym.W, sym.H, sym.V

    @kernel(work_shape=(W, sympy.ceiling(H / V)), literals=[V])
    def vcopy(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT], v: V):
        x, y = gr.work_offset
        gr.store(dst[x:, y * V:], gr.vload(src[x:, y * V:], shape=(gr.shape[0], gr.shape[1] * V)))

    a = np.arange(256 * 1024, dtype=np.int32).reshape(256, 1024)
    db = rt.to_device(np.zeros_like(a))
    vcopy(rt.to_device(a), db, 4)
    assert rt.last_kernel_name() == "hcamd_copy_flat_v4_nt"      # one 16-byte word per lane and step
    assert_array_equal(db.to_host(), a)

    N = sym.N

    @kernel(work_shape=N, group_shape=256)
    def vadd(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], z: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(z[o:], gr.vload(x[o:], shape=256) + gr.vload(y[o:], shape=256))

    x, y = cf.inputs_c1(100_003)
    dz = rt.DeviceArray(x.shape, np.float32)
    vadd(rt.to_device(x), rt.to_device(y), dz)
    assert rt.last_kernel_name() == "hcamd_add_f32_v4_nt"
    assert_array_equal(dz.to_host().view(np.uint32), cf.np_add(x, y).view(np.uint32))


def test_thread_variant_selects_the_kernel_for_this_thread_only():
    import threading
    ab, bb = cf.inputs_c5((256, 256, 256))
    da, dbt = rt.to_device(ab, bf16=True), rt.to_device(bb, bf16=True)
    dc = rt.DeviceArray((256, 256), np.uint16, bf16=True)
    plan = rt.plan_gemm_bf16(da, dbt, dc)
    names = {}

    def launch(tag, variant):
        if variant is not None:
            rt.set_thread_variant("gemm", variant)
        plan.launch(sync=True)
        names[tag] = rt.last_kernel_name()
        if variant is not None:
            rt.set_thread_variant("gemm", -1)

    rt.set_thread_variant("gemm", 14)
    t = threading.Thread(target=launch, args=("other", None))
    t.start()
    t.join()
    launch("mine", None)                       # still under this thread's override
    rt.set_thread_variant("gemm", -1)
    launch("after", None)
    assert names["other"] == "hcamd_gemm_bf16_p256x256_w2x4"
    assert names["mine"] == "hcamd_gemm_bf16_p256x256_w2x4_direct"
    assert names["after"] == "hcamd_gemm_bf16_p256x256_w2x4"


# ---------------------------------------------------------------------------
# Integer tiles (python/hckernel/kernel_api.py:157-211 on int32 data)
# ---------------------------------------------------------------------------
_I32 = np.int32
_INT_BIN = {
    "add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b,
    "floordiv": lambda a, b: a // (b | _I32(1)), "mod": lambda a, b: a % (b | _I32(1)),
    "min": lambda a, b: np.minimum(a, b), "max": lambda a, b: np.maximum(a, b),
    "and": lambda a, b: a & b, "or": lambda a, b: a | b, "xor": lambda a, b: a ^ b,
    "shl": lambda a, b: a << (b & _I32(31)), "shr": lambda a, b: a >> (b & _I32(31)),
    "lt": lambda a, b: (a < b) * _I32(3), "ge": lambda a, b: (a >= b) * a, "ne": lambda a, b: (a != b) * b,
}


def _random_int_tree(rng, depth):
    """A function tiles -> tile and its description."""
    if depth == 0 or rng.random() < 0.2:
        if rng.random() < 0.75:
            i = int(rng.integers(0, 3))
            return (lambda t, i=i: t[i]), f"t{i}"
        c = _I32(rng.integers(-50, 51))
        return (lambda t, c=c: c), str(int(c))
    if rng.random() < 0.15:
        f, d = _random_int_tree(rng, depth - 1)
        if rng.random() < 0.5:
            return (lambda t: -f(t)), f"-({d})"
        return (lambda t: abs(f(t))), f"abs({d})"
    name = list(_INT_BIN)[int(rng.integers(0, len(_INT_BIN)))]
    fa, da = _random_int_tree(rng, depth - 1)
    fb, db = _random_int_tree(rng, depth - 1)
    op = _INT_BIN[name]
    return (lambda t: op(fa(t), fb(t))), f"{name}({da}, {db})"


@pytest.mark.parametrize("seed", range(24))
def test_random_int32_expression_trees_equal_the_host_executor(seed):
    """(A tree that needs more than the integer map's four stack entries or 32
    instructions is drawn again, so that every seed runs one on the GPU.)"""
    rng = np.random.default_rng(1000 + seed)
    R, Cc = sym.R, sym.C
    shape = [(37, 130), (64, 256), (5, 1031)][seed % 3]
    big = seed % 4 == 0
    ins = [rng.integers(-2 ** 31 if big else -1000, 2 ** 31 if big else 1000, shape).astype(np.int32)
           for _ in range(3)]
    for _ in range(20):
        f, desc = _random_int_tree(rng, 3)
        if "t" not in desc or desc in ("t0", "t1", "t2"):
            continue

        def body(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], c: Buffer[R, Cc, DT],
                 out: Buffer[R, Cc, DT]):
            x, y = gr.work_offset
            tiles = [gr.load(v[x:, y:], shape=gr.shape) for v in (a, b, c)]
            value = f(tiles)
            if not hasattr(value, "shape") or value.shape == ():        # the tree folded to a constant
                value = tiles[0] * _I32(0) + value
            gr.store(out[x:, y:], value)

        host = np.full(shape, -777, np.int32)
        dout = rt.to_device(host)
        try:
            kernel(work_shape=(R, Cc), group_shape=(4, 64))(body)(*[rt.to_device(v) for v in ins], dout)
        except NoNativeKernel as e:
            if "too deep" in str(e) or "too long" in str(e):
                continue
            raise
        except TypeError:
            # a NumPy scalar on the left of a tile: a TypeError in the reference too
            # (its tile type has no reflected operators), and in the host executor
            with pytest.raises(TypeError), np.errstate(all="ignore"):
                sim_kernel(work_shape=(R, Cc), group_shape=(4, 64))(body)(*ins, host)
            continue
        break
    else:
        pytest.fail("no tree that fits the integer map in 20 draws")
    with np.errstate(all="ignore"):
        sim_kernel(work_shape=(R, Cc), group_shape=(4, 64))(body)(*ins, host)
    assert_array_equal(dout.to_host(), host, err_msg=desc)


def _gather_bodies(deco, make_mapping):
    """Bodies that load tiles through index mappings, or store one through a
    mapping, outside a matrix product (python/hckernel/kernel_api.py:304-310,
    319-335): indices that leave the window are inactive elements."""
    R, Cc = sym.R, sym.C
    TM, TN = 8, 16
    transpose = make_mapping(lambda i, j: (j, i))
    shifted = make_mapping(lambda i, j: (i - 1, j + 2))
    spread = make_mapping(lambda i, j: (2 * i, j))
    diagonal = make_mapping(lambda i, j: (i, (i + j) % TN))

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def gathered_copy(gr: CurrentGroup, a: Buffer[Cc, R, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        gr.store(out[x:, y:], gr.load(a[y:, x:], shape=(TM, TN), mapping=transpose))

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def gathered_expression(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta = gr.load(a[x:, y:], shape=(TM, TN), mapping=shifted)
        tb = gr.load(b[x:, y:], shape=(TM, TN))
        gr.store(out[x:, y:], (ta * np.float32(2) + tb) / gr.load(b[x:, y:], shape=(TM, TN), mapping=diagonal))

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def scattered_store(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[2 * R, Cc, DT]):
        x, y = gr.work_offset
        t = gr.load(a[x:, y:], shape=(TM, TN)) - gr.load(b[x:, y:], shape=(TM, TN))
        gr.store(out[2 * x:, y:], t, mapping=spread)

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def function_of_gathered(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta = gr.load(a[x:, y:], shape=(TM, TN), mapping=shifted)
        gr.store(out[x:, y:], np.exp(ta) + gr.load(b[x:, y:], shape=(TM, TN)))     # a bare array: stored in full

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def bare_array_scattered(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        # numpy.ma's own array, element by element: a deactivated element is the
        # masked constant, which NumPy turns into NaN (kernel_api.py:331-334)
        x, y = gr.work_offset
        ta = gr.load(a[x:, y:], shape=(TM, TN), mapping=diagonal)
        gr.store(out[x:, y:], np.sqrt(ta) / gr.load(b[x:, y:], shape=(TM, TN)), mapping=shifted)

    @deco(work_shape=(R, Cc), group_shape=(TM, TN))
    def bare_copy_scattered(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        gr.store(out[x:, y:], gr.load(a[x:, y:], shape=(TM, TN)).astype(a.dtype), mapping=shifted)

    return {"gathered_copy": gathered_copy, "gathered_expression": gathered_expression,
            "scattered_store": scattered_store, "function_of_gathered": function_of_gathered,
            "bare_array_scattered": bare_array_scattered, "bare_copy_scattered": bare_copy_scattered}


@pytest.mark.parametrize("rows,cols", [(16, 32), (37, 50), (8, 16)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int32])
def test_mapped_loads_and_stores_outside_a_product_match_the_simulator(rows, cols, dtype):
    """The same bodies on the GPU and on the simulator, on arrays that do not
    fill their last tiles: bit for bit, including which elements are left alone
    (indices past the window, deactivated quotients)."""
    gpu, sim = _gather_bodies(kernel, create_mapping), _gather_bodies(sim_kernel, __import__("oracle.hcsim", fromlist=["x"]).create_mapping)
    rng = np.random.default_rng(rows + cols)
    a = rng.integers(-5, 6, (rows, cols)).astype(dtype)
    b = rng.integers(-2, 3, (rows, cols)).astype(dtype)
    at = np.ascontiguousarray(a.T)
    cases = {"gathered_copy": ([at], (rows, cols))}
    if dtype != np.int32:
        cases.update({"gathered_expression": ([a, b], (rows, cols)), "scattered_store": ([a, b], (2 * rows, cols)),
                      "function_of_gathered": ([a, b], (rows, cols)),
                      "bare_array_scattered": ([a, b], (rows, cols)), "bare_copy_scattered": ([a, b], (rows, cols))})
    for name, (ins, shape) in cases.items():
        want = np.full(shape, 7, dtype)
        with np.errstate(all="ignore"):
            sim[name](*ins, want)
        out = rt.to_device(np.full(shape, 7, dtype))
        gpu[name](*[rt.to_device(v) for v in ins], out)
        assert rt.last_kernel_name() == "hcamd_gather_fmap", name
        got = out.to_host()
        if name == "function_of_gathered":          # exp: the last bit may differ
            assert_array_equal(got == 7, want == 7, err_msg=name)
            assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=2e-3 if dtype == np.float16 else 1e-6,
                            err_msg=name)
        else:
            bits = {2: np.uint16, 4: np.uint32}[np.dtype(dtype).itemsize]
            assert_array_equal(got.view(bits), want.view(bits), err_msg=name)
        if name in ("gathered_expression", "scattered_store"):
            assert (want == 7).any(), name               # something is left alone
        if name.startswith("bare_") and (rows, cols) == (37, 50):
            assert np.isnan(want).any() and (want == 7).any(), name     # masked constants, and places no index reaches


def _window_bodies(deco):
    """Elementwise bodies whose loads do not walk the store's window: a window
    shifted by a constant, a row vector and a column vector next to a 2-D tile,
    a transposed tile, a slice of a wider tile, a reshaped one."""
    M, N = sym.M, sym.N

    @deco(work_shape=N, group_shape=64)
    def stencil(gr: CurrentGroup, x: Buffer[N, DT], out: Buffer[N, DT]):
        o = gr.work_offset[0]
        left, mid, right = (gr.load(x[o + k:], shape=gr.shape) for k in (0, 1, 2))
        gr.store(out[o:], (left + right) * x.dtype.type(0.5) - mid)

    @deco(work_shape=(M, N), group_shape=(8, 32))
    def bias_and_scale(gr: CurrentGroup, x: Buffer[M, N, DT], b: Buffer[N, DT], s: Buffer[M, DT],
                       out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        t = gr.load(x[i:, j:], shape=gr.shape)
        row = gr.load(b[j:], shape=gr.shape[1])
        col = gr.load(s[i:], shape=gr.shape[0])
        gr.store(out[i:, j:], (t + row) * col[:, None] / row[None, :])

    @deco(work_shape=(M, N), group_shape=(8, 32))
    def transposed(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[N, M, DT]):
        i, j = gr.work_offset
        gr.store(out[j:, i:], gr.load(x[i:, j:], shape=gr.shape).T)

    @deco(work_shape=(M, N), group_shape=(8, 32))
    def symmetric_part(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[N, M, DT], out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        a = gr.load(x[i:, j:], shape=gr.shape)
        bt = gr.load(y[j:, i:], shape=gr.shape[::-1])
        gr.store(out[i:, j:], a * x.dtype.type(0.5) + bt.T * x.dtype.type(0.5))

    @deco(work_shape=(M, N), group_shape=(8, 32))
    def sliced(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        wide = gr.load(x[i:, j:], shape=(gr.shape[0] + 1, gr.shape[1] + 1))
        gr.store(out[i:, j:], wide[1:, 1:] - wide[:-1, :-1])

    @deco(work_shape=(M, N), group_shape=(8, 32))
    def reshaped(gr: CurrentGroup, x: Buffer[M, N, DT], flat: Buffer[sym.L, DT], out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        v = gr.load(flat[:], shape=(8 * 32,))
        gr.store(out[i:, j:], gr.load(x[i:, j:], shape=gr.shape) + v.reshape(8, 32))

    return {"stencil": stencil, "bias_and_scale": bias_and_scale, "transposed": transposed,
            "symmetric_part": symmetric_part, "sliced": sliced, "reshaped": reshaped}


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,cols", [(16, 64), (37, 50), (5, 131)])
def test_loads_that_do_not_walk_the_window_of_the_store_match_the_simulator(rows, cols, dtype):
    """Shifted, broadcast, transposed, sliced and reshaped tiles in elementwise
    bodies go to the gathered map with index tables the binder derives; the
    same bytes as the simulator writes, elements it leaves alone included
    (loads past the end of an array, zero divisors)."""
    gpu, sim = _window_bodies(kernel), _window_bodies(sim_kernel)
    rng = np.random.default_rng(rows * cols)
    x = rng.integers(-6, 7, (rows, cols)).astype(dtype)
    y = rng.integers(-6, 7, (cols, rows)).astype(dtype)
    b = rng.integers(-2, 3, cols).astype(dtype)          # zeros: deactivated quotients
    sc = rng.integers(-3, 4, rows).astype(dtype)
    flat = rng.integers(-6, 7, 8 * 32 - 3).astype(dtype)  # shorter than the tile it is reshaped into
    cases = {"stencil": ([x.reshape(-1)], (rows * cols,)), "bias_and_scale": ([x, b, sc], (rows, cols)),
             "transposed": ([x], (cols, rows)), "symmetric_part": ([x, y], (rows, cols)),
             "sliced": ([x], (rows, cols)), "reshaped": ([x, flat], (rows, cols))}
    bits = {2: np.uint16, 4: np.uint32}[np.dtype(dtype).itemsize]
    for name, (ins, shape) in cases.items():
        want = np.full(shape, 7, dtype)
        with np.errstate(all="ignore"):
            sim[name](*ins, want)
        out = rt.to_device(np.full(shape, 7, dtype))
        gpu[name](*[rt.to_device(v) for v in ins], out)
        # (a row vector and a per-row operand next to a tile are one stage of a row program)
        # and a tile's .T alone is a transposed copy)
        assert rt.last_kernel_name().startswith({"bias_and_scale": "hcamd_row_program",
                                                 "transposed": "hcamd_transpose2d"}.get(name, "hcamd_gather_fmap")), name
        assert_array_equal(out.to_host().view(bits), want.view(bits), err_msg=name)
        if name in ("stencil", "bias_and_scale", "sliced", "reshaped"):
            assert (want == 7).any(), name                 # something is left alone


@pytest.mark.parametrize("n,tile", [(1000, 256), (1024, 256), (77, 64), (5000, 1024), (300, 512)])
def test_one_result_per_group_from_reductions_of_whole_tiles(n, tile):
    """`out[group id] = tile.sum()` and `atomic_ref(out)[f(group id)] += ...`:
    the first stage of a two-stage reduction, every group with an element of
    its own; against the simulator, the last tile shorter than the others,
    elements no group owns left as they were."""
    N, G = sym.N, sym.G

    def bodies(deco):
        @deco(work_shape=N, group_shape=tile)
        def sums(gr: CurrentGroup, x: Buffer[N, DT], out: Buffer[G, DT]):
            o = gr.work_offset[0]
            t = gr.load(x[o:], shape=gr.shape)
            out[gr.id[0]] = (t * t).sum()

        @deco(work_shape=N, group_shape=tile)
        def spread(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], out: Buffer[G, DT]):
            o = gr.work_offset[0]
            t, u = gr.load(x[o:], shape=gr.shape), gr.load(y[o:], shape=gr.shape)
            atomic_ref(out)[gr.id[0] + 2] += (t + u).max() - np.minimum(t, u).min()
        return sums, spread

    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    y = rng.standard_normal(n).astype(np.float32)
    groups = -(-n // tile)
    (g_sums, g_spread), (s_sums, s_spread) = bodies(kernel), bodies(sim_kernel)
    want = np.full(groups + 3, 7, np.float32)
    s_sums(x, want)
    out = rt.to_device(np.full(groups + 3, 7, np.float32))
    g_sums(rt.to_device(x), out)
    assert rt.last_kernel_name().startswith("hcamd_row_program")
    got = out.to_host()
    assert_allclose(got, want, rtol=2e-6 * np.sqrt(tile))
    assert (got[groups:] == 7).all()
    start = rng.standard_normal(groups + 5).astype(np.float32)
    want = start.copy()
    s_spread(x, y, want)
    out = rt.to_device(start)
    g_spread(rt.to_device(x), rt.to_device(y), out)
    got = out.to_host()
    assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    assert_array_equal(got[:2], start[:2])
    assert_array_equal(got[groups + 2:], start[groups + 2:])


@pytest.mark.parametrize("rows,k", [(64, 128), (37, 1000), (300, 4097)])
def test_matrix_times_vector_is_a_row_sum_of_products(rows, k):
    """numpy.dot of a (rows, K) tile and a (K,) tile: the row program's sum of
    products along the rows; against the simulator's numpy.dot to the bound of a
    sum of K fp32 products added in another order."""
    M, K = sym.M, sym.K

    def body(gr: CurrentGroup, a: Buffer[M, K, DT], v: Buffer[K, DT], out: Buffer[M, DT]):
        i = gr.work_offset[0]
        gr.store(out[i:], np.dot(gr.load(a[i:, :], shape=(gr.shape[0], K)), gr.load(v[:], shape=(K,))))

    rng = np.random.default_rng(k)
    a = rng.standard_normal((rows, k)).astype(np.float32)
    v = rng.standard_normal(k).astype(np.float32)
    want = np.full(rows, 7, np.float32)
    sim_kernel(work_shape=M, group_shape=8)(body)(a, v, want)
    out = rt.to_device(np.full(rows, 7, np.float32))
    kernel(work_shape=M, group_shape=8)(body)(rt.to_device(a), rt.to_device(v), out)
    assert rt.last_kernel_name().startswith("hcamd_row_program")
    bound = 4 * np.finfo(np.float32).eps * (np.abs(a) @ np.abs(v))
    assert (np.abs(out.to_host() - want) <= bound).all()
    assert_allclose(out.to_host(), a.astype(np.float64) @ v.astype(np.float64), atol=float(bound.max()))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_selections_conversions_and_tanh_match_the_simulator(dtype):
    """numpy.where of tiles (a plain array chosen from the values, whatever their
    activity), numpy.tanh next to operations that deactivate, and an int32 tile
    converted with astype inside a float expression: the simulator's bytes,
    elements it leaves alone included (tanh to 1.5 ulp)."""
    M, N = sym.M, sym.N
    f = dtype
    forms = {
        "where_of_tiles": lambda a, b, ai: np.where(a > b, a, b),
        "where_with_numbers": lambda a, b, ai: np.where(a * b >= f(0), a, f(-1)),
        "where_of_quotient": lambda a, b, ai: np.where(b != f(0), a / b, f(9)),
        "where_nested": lambda a, b, ai: np.where(a < b, np.where(a < f(0), -a, a), b * f(2)),
        "tanh_of_quotient": lambda a, b, ai: np.tanh(a / b),
        "tanh_times_tile": lambda a, b, ai: a * np.tanh(b),
        "tanh_and_domain": lambda a, b, ai: np.sqrt(np.abs(a)) + np.tanh(b) - np.square(a),
    }
    if dtype == np.float32:
        forms.update({"int_astype": lambda a, b, ai: ai.astype(f) * f(0.5),
                      "int_astype_plus_tile": lambda a, b, ai: a + ai.astype(f),
                      "int_in_where": lambda a, b, ai: np.where(ai.astype(f) > a, b, ai.astype(f))})

    def make(deco, fn):
        @deco(work_shape=(M, N), group_shape=(8, 32))
        def body(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], xi: Buffer[M, N, DT],
                 out: Buffer[M, N, DT]):
            i, j = gr.work_offset
            a, b = gr.load(x[i:, j:], shape=gr.shape), gr.load(y[i:, j:], shape=gr.shape)
            gr.store(out[i:, j:], fn(a, b, gr.load(xi[i:, j:], shape=gr.shape)))
        return body

    rng = np.random.default_rng(31)
    rows, cols = 37, 50
    x = (rng.integers(-8, 9, (rows, cols)) / 4).astype(dtype)
    y = (rng.integers(-3, 4, (rows, cols)) / 2).astype(dtype)          # zeros among the divisors
    x[3, 4], y[5, 6], x[7, 7] = np.inf, np.nan, -0.0
    xi = rng.integers(-9, 10, (rows, cols)).astype(np.int32)
    bits = {2: np.uint16, 4: np.uint32}[np.dtype(dtype).itemsize]
    for name, fn in forms.items():
        want = np.full((rows, cols), 7, dtype)
        with np.errstate(all="ignore"):
            make(sim_kernel, fn)(x, y, xi, want)
        out = rt.to_device(np.full((rows, cols), 7, dtype))
        make(kernel, fn)(rt.to_device(x), rt.to_device(y), rt.to_device(xi), out)
        got = out.to_host()
        if "tanh" in name:
            assert_array_equal(got == 7, want == 7, err_msg=name)
            assert_array_equal(np.isnan(got), np.isnan(want), err_msg=name)
            ok = ~np.isnan(want)
            assert_allclose(got[ok].astype(np.float64), want[ok].astype(np.float64),
                            rtol=1.1e-3 if dtype == np.float16 else 4e-7,
                            atol=0 if dtype == np.float16 else 5e-7, err_msg=name)   # (sums of terms near +-2)
        else:
            assert_array_equal(got.view(bits), want.view(bits), err_msg=name)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_more_numpy_functions_of_tiles(dtype):
    """floor, ceil, trunc, sign, exp2, log2, log10, log1p, expm1, sin, cos and
    reciprocal of tiles and of quotients with deactivated elements, through the
    general float map: the same elements written as the simulator writes (numpy.ma
    keeps the activity, log2 / log10 have its domain), exact functions bit for
    bit, the others to a few units in the last place."""
    N = sym.N
    exact = ("floor", "ceil", "trunc", "sign", "reciprocal")
    names = exact + ("exp2", "log2", "log10", "log1p", "expm1", "sin", "cos")

    def make(deco, fn, quotient):
        @deco(work_shape=N, group_shape=256)
        def body(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], out: Buffer[N, DT]):
            o = gr.work_offset[0]
            a, b = gr.load(x[o:], shape=gr.shape), gr.load(y[o:], shape=gr.shape)
            gr.store(out[o:], a + fn(a / b) if quotient else fn(a))      # (a tile on the left: a tile again)
        return body

    rng = np.random.default_rng(17)
    n = 3001
    x = (rng.integers(-40, 41, n) / 8).astype(dtype)
    y = (rng.integers(-2, 3, n) / 2).astype(dtype)
    x[:6] = [np.inf, -np.inf, np.nan, 0.0, -0.0, 1.0]
    y[:6] = [1.0, 2.0, 1.0, 1.0, 1.0, 0.0]
    bits = {2: np.uint16, 4: np.uint32}[np.dtype(dtype).itemsize]
    for name in names:
        for quotient in (False, True):
            fn = getattr(np, name)
            want = np.full(n, 7, dtype)
            with np.errstate(all="ignore"):
                make(sim_kernel, fn, quotient)(x, y, want)
            out = rt.to_device(np.full(n, 7, dtype))
            make(kernel, fn, quotient)(rt.to_device(x), rt.to_device(y), out)
            assert rt.last_kernel_name() in ("hcamd_fmap", "hcamd_fmap_v8"), name
            got = out.to_host()
            tag = f"{name} quotient={quotient}"
            if name in exact:
                assert_array_equal(got.view(bits), want.view(bits), err_msg=tag)
            else:
                assert_array_equal(np.isnan(got), np.isnan(want), err_msg=tag)
                ok = ~np.isnan(want)
                assert_allclose(got[ok].astype(np.float64), want[ok].astype(np.float64),
                                rtol=2e-3 if dtype == np.float16 else 1e-6,
                                atol=2e-3 if dtype == np.float16 else 1e-6, err_msg=tag)
            if quotient:
                assert ((want == 7) & (y == 0)).sum() > 100, tag          # deactivated quotients are left alone


def test_tile_mask_is_stored_as_a_plain_bool_array():
    """`tile.mask` (python/hckernel/kernel_api.py:117-119: True = active) of
    float and int32 expressions that the data deactivates here and there: the
    same bytes as the simulator stores, every element written."""
    N = sym.N

    def fbody(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], q: Buffer[N, DT], m: Buffer[N, DT],
              m2: Buffer[N, DT]):
        o = gr.work_offset[0]
        ta, tb = gr.load(a[o:], shape=gr.shape), gr.load(b[o:], shape=gr.shape)
        t = ta / tb
        gr.store(q[o:], t)
        gr.store(m[o:], t.mask)
        gr.store(m2[o:], ((ta - tb) / (t * tb)).mask)

    def ibody(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], q: Buffer[N, DT], m: Buffer[N, DT],
              m2: Buffer[N, DT]):
        o = gr.work_offset[0]
        ta, tb = gr.load(a[o:], shape=gr.shape), gr.load(b[o:], shape=gr.shape)
        gr.store(q[o:], ta // tb)
        gr.store(m[o:], (ta % tb + ta).mask)
        gr.store(m2[o:], ta.mask)

    rng = np.random.default_rng(8)
    n = 1003
    for dtype, body in ((np.float32, fbody), (np.float16, fbody), (np.int32, ibody)):
        a = rng.integers(-4, 5, n).astype(dtype)
        b = rng.integers(-2, 3, n).astype(dtype)
        if dtype != np.int32:
            a[5], b[9] = np.inf, np.nan
        want = [np.full(n, 7, dtype), np.full(n, 7, np.bool_), np.full(n, 7, np.bool_)]
        with np.errstate(all="ignore"):
            sim_kernel(work_shape=N, group_shape=256)(body)(a, b, *want)
        got = [rt.to_device(np.full(n, 7, dtype)), rt.to_device(np.full(n, 7, np.bool_)),
               rt.to_device(np.full(n, 7, np.bool_))]
        kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), *got)
        assert 0 < want[1].sum() < n                       # some elements are deactivated, some are not
        for g, w in zip(got, want):
            assert_array_equal(g.to_host().view(np.uint8), w.view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int32])
def test_allocated_tiles_as_values(dtype):
    """CurrentGroup.full / zeros / ones / empty and their v-forms
    (python/hckernel/kernel_api.py:347-376,433-434) as values: a constant tile
    stored as it is (1-D, a ragged 2-D window, a bool buffer), as an operand, as an
    accumulator that loads are added to, and as a tile that is filled by
    assignment; the bytes the simulator leaves, untouched elements included."""
    N, M = sym.N, sym.M
    T = dtype

    def one_d(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT], s: Buffer[N, DT], acc: Buffer[N, DT],
              filled: Buffer[N, DT], flag: Buffer[N, DT]):
        o = gr.work_offset[0]
        x = gr.load(a[o:], shape=gr.shape)
        gr.store(c[o:], gr.full(gr.shape, dtype=T, fill_value=42))
        gr.store(s[o:], x * gr.vfull(gr.shape, dtype=T, fill_value=3) + gr.ones(gr.shape, dtype=T))
        t = gr.vzeros(gr.shape, dtype=T)
        t += x
        t += gr.vload(a[o:], shape=gr.shape)
        gr.store(acc[o:], t)
        e = gr.empty(gr.shape, dtype=T)
        e[:] = x - gr.vones(gr.shape, dtype=T)
        gr.store(filled[o:], gr.vec(e))
        gr.store(flag[o:], gr.zeros(gr.shape, dtype=np.bool_))

    n = 1003
    rng = np.random.default_rng(21)
    a = rng.integers(-50, 50, n).astype(dtype)
    want = [np.full(n, 7, dtype) for _ in range(4)] + [np.full(n, 1, np.bool_)]
    sim_kernel(work_shape=N, group_shape=256)(one_d)(a, *want)
    got = [rt.to_device(np.full(n, 7, dtype)) for _ in range(4)] + [rt.to_device(np.full(n, 1, np.bool_))]
    kernel(work_shape=N, group_shape=256)(one_d)(rt.to_device(a), *got)
    for g, w in zip(got, want):
        assert_array_equal(g.to_host().view(np.uint8), w.view(np.uint8))

    def two_d(gr: CurrentGroup, c: Buffer[M, N, DT]):
        i, j = gr.work_offset
        gr.store(c[i:, j:], gr.full(gr.shape, dtype=T, fill_value=5))

    want2 = np.full((61, 123), 9, dtype)            # ragged against the 8 x 32 groups
    sim_kernel(work_shape=(M, N), group_shape=(8, 32))(two_d)(want2)
    dev = rt.to_device(np.full((61, 123), 9, dtype))
    kernel(work_shape=(M, N), group_shape=(8, 32))(two_d)(dev)
    assert_array_equal(dev.to_host(), want2)
    assert (want2 == 5).all()
    torch = pytest.importorskip("torch")
    if torch.cuda.is_available():
        # a window of a larger tensor: the rest must stay as it was
        big = torch.full((70, 131), 9, dtype=getattr(torch, np.dtype(dtype).name), device="cuda")
        torch.cuda.synchronize()
        kernel(work_shape=(M, N), group_shape=(8, 32))(two_d)(big[3:64, 2:125])
        host = big.cpu().numpy()
        assert (host[3:64, 2:125] == 5).all() and (host == 9).sum() == 70 * 131 - 61 * 123


def test_fp16_maximum_and_minimum_of_signed_zeros_follow_numpy():
    """NumPy's fp16 maximum / minimum return the first of two equal values, its
    fp32 ones the second: +0 against -0 shows it.  Bits must equal the simulator's
    for both types."""
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], hi: Buffer[N, DT], lo: Buffer[N, DT]):
        o = gr.work_offset[0]
        ta, tb = gr.load(a[o:], shape=gr.shape), gr.load(b[o:], shape=gr.shape)
        gr.store(hi[o:], np.maximum(ta, tb))
        gr.store(lo[o:], np.minimum(ta * ta.dtype.type(1), tb))

    for dtype, bits in ((np.float16, np.uint16), (np.float32, np.uint32)):
        rng = np.random.default_rng(3)
        a = rng.standard_normal(1000).astype(dtype)
        b = rng.standard_normal(1000).astype(dtype)
        a[::4], b[::4] = 0.0, -0.0
        a[1::4], b[1::4] = -0.0, 0.0
        a[2], b[6] = np.nan, np.nan
        want_hi, want_lo = np.full(1000, 7, dtype), np.full(1000, 7, dtype)
        sim_kernel(work_shape=N, group_shape=256)(body)(a, b, want_hi, want_lo)
        hi, lo = rt.to_device(np.full(1000, 7, dtype)), rt.to_device(np.full(1000, 7, dtype))
        kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), hi, lo)
        assert_array_equal(hi.to_host().view(bits), want_hi.view(bits))
        assert_array_equal(lo.to_host().view(bits), want_lo.view(bits))


def test_int32_division_by_zero_deactivates_the_element_and_shift_counts():
    """numpy.ma masks x // 0 and x % 0, and everything computed from them: the
    store leaves those elements alone.  Shift counts outside 0..31 follow NumPy."""
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], q: Buffer[N, DT], r: Buffer[N, DT],
             s: Buffer[N, DT], flag: Buffer[N, DT]):
        o = gr.work_offset[0]
        ta, tb = gr.load(a[o:], shape=gr.shape[0]), gr.load(b[o:], shape=gr.shape[0])
        gr.store(q[o:], (ta // tb) * _I32(2) + _I32(1))
        gr.store(r[o:], ta % tb)
        gr.store(s[o:], (ta << tb) ^ (ta >> tb))
        gr.store(flag[o:], ta % _I32(7) == tb % _I32(7))

    rng = np.random.default_rng(77)
    n = 5000
    a = rng.integers(-10 ** 9, 10 ** 9, n).astype(np.int32)
    b = rng.integers(-6, 41, n).astype(np.int32)              # zeros, negatives, counts past 31
    a[:4] = [-2 ** 31, -2 ** 31, 2 ** 31 - 1, -7]
    b[:4] = [-1, 0, -1, 2]
    hosts = [np.full(n, -777, np.int32) for _ in range(3)] + [np.full(n, True)]
    hosts[3][::2] = False
    devs = [rt.to_device(h) for h in hosts]
    kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), *devs)
    with np.errstate(all="ignore"):
        sim_kernel(work_shape=N, group_shape=256)(body)(a, b, *hosts)
    for d, h, name in zip(devs, hosts, "qrsf"):
        assert_array_equal(d.to_host(), h, err_msg=name)
    zero = (b == 0) & (a != -2 ** 31)
    assert zero.sum() > 50 and (hosts[0][zero] == -777).all() and (hosts[1][zero] == -777).all()
    assert (hosts[0][b != 0] != -777).any()
    # numpy.ma's own corner: |INT_MIN| overflows in its divisor test, so INT_MIN // 0 stays
    # active with NumPy's quotient 0 (element 1 of the inputs)
    assert (a[1], b[1]) == (-2 ** 31, 0) and hosts[0][1] == 1 and hosts[1][1] == 0


def _special_floats(rng, shape, dtype):
    """Random values with zeros of both signs, infinities, NaNs, huge and tiny
    magnitudes mixed in, so that divisions fail in every way numpy.ma tests for."""
    big, tiny = (3.0e38, 1.5e-38) if dtype == np.float32 else (60000.0, 6.2e-5)
    x = (rng.standard_normal(shape) * 4).astype(dtype)
    special = np.array([0.0, -0.0, 1.0, -1.0, 2.5, -7.25, big, -big, tiny, np.inf, -np.inf, np.nan,
                        3.0, -3.0, 0.5], dtype)
    pick = rng.random(shape) < 0.35
    x[pick] = special[rng.integers(0, len(special), int(pick.sum()))]
    return x


_FLOAT_OPERATOR_BODIES = {
    # the tile operators go through numpy.ma: a failed division deactivates its element
    "a/b": lambda a, b, K: a / b,
    "a/b*2+1": lambda a, b, K: a / b * K(2) + K(1),
    "(a+b)/(a-b)": lambda a, b, K: (a + b) / (a - b),
    "a/3": lambda a, b, K: a / K(3),
    "a/0": lambda a, b, K: a / K(0),
    "a*a/b": lambda a, b, K: a * a / b,
    "a**2/b": lambda a, b, K: a ** K(2) / b,
    "a**0.5*b": lambda a, b, K: a ** K(0.5) * b,
    # a NumPy function reads the values, deactivated or not, and returns a plain array
    "np.divide(a,b)": lambda a, b, K: np.divide(a, b),
    "np.exp(a/b)": lambda a, b, K: np.exp(a / b),
    "np.abs(a/b)-b/a": lambda a, b, K: np.abs(a / b) - b / a,
    "np.abs(a/b*2)": lambda a, b, K: np.abs(a / b * K(2)),
    "a/b+np.abs(b/a)": lambda a, b, K: a / b + np.abs(b / a),
    "np.maximum(a/b,b/a)": lambda a, b, K: np.maximum(a / b, b / a),
    "np.sqrt(a**2)": lambda a, b, K: np.sqrt(a ** K(2)),
    # // and %, comparisons
    "a//b": lambda a, b, K: a // b,
    "a%b": lambda a, b, K: a % b,
    "a//b*b+a%b": lambda a, b, K: (a // b) * b + a % b,
    "a%3-b//2": lambda a, b, K: a % K(3) - b // K(2),
    "np.abs(a//b)": lambda a, b, K: np.abs(a // b),
    "(a<b)*a": lambda a, b, K: (a < b).astype(K) * a,
    "-(a/b)": lambda a, b, K: -(a / b),
    "abs(a/b)": lambda a, b, K: abs(a / b),
    # NumPy functions with a domain put numpy.ma's fill value where it fails
    "np.sqrt(a)": lambda a, b, K: np.sqrt(a),
    "np.log(a)": lambda a, b, K: np.log(a),
    "np.sqrt(a/b)": lambda a, b, K: np.sqrt(a / b),
    "a*np.sqrt(b)": lambda a, b, K: a * np.sqrt(b),
    "np.sqrt(a)*b": lambda a, b, K: np.sqrt(a) * b,
    "np.log(a)/b": lambda a, b, K: np.log(a) / b,
    "np.add(a/b,b)": lambda a, b, K: np.add(a / b, b),
    "np.remainder(a,b)": lambda a, b, K: np.remainder(a, b),
    "(a/b)*b": lambda a, b, K: (a / b) * b,
    "np.abs(a)*(b/a)": lambda a, b, K: np.abs(a) * (b / a),
    "(a/b)*K(2)": lambda a, b, K: (a / b) * K(2),
    "np.abs(a/b)+K(1)": lambda a, b, K: np.abs(a / b) + K(1),
    "np.rint(a//b)-a%b": lambda a, b, K: np.rint(a // b) - a % b,
}


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("name", list(_FLOAT_OPERATOR_BODIES))
def test_float_tile_operators_deactivate_like_numpy_ma(name, dtype):
    """/ // % ** on float tiles go through numpy.ma in the reference
    (python/hckernel/kernel_api.py:157-180): a zero divisor or a quotient that is
    not finite deactivates the element, the store leaves it alone, and a NumPy
    function applied afterwards sees the value numpy.ma left there.  Same body on
    the GPU and on the host executor, bit for bit, including which elements are
    written at all."""
    expr = _FLOAT_OPERATOR_BODIES[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()) % 1000 + np.dtype(dtype).itemsize)
    R, Cc = sym.R, sym.C
    shape = (37, 1031) if dtype == np.float32 else (19, 520)

    def body(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        gr.store(out[x:, y:], expr(gr.load(a[x:, y:], shape=gr.shape), gr.load(b[x:, y:], shape=gr.shape),
                                   dtype))

    a, b = _special_floats(rng, shape, dtype), _special_floats(rng, shape, dtype)
    host = np.full(shape, 7.5, dtype)
    dout = rt.to_device(host)
    deco = dict(work_shape=(R, Cc), group_shape=(4, 64))
    kernel(**deco)(body)(rt.to_device(a), rt.to_device(b), dout)
    with np.errstate(all="ignore"):
        sim_kernel(**deco)(body)(a, b, host)
    got = dout.to_host()
    nan = np.isnan(host)
    assert_array_equal(np.isnan(got), nan, err_msg=name)
    u = np.uint32 if dtype == np.float32 else np.uint16
    if "exp" in name or "log" in name or "**0.5" in name:
        # the library exp / log differ from NumPy's in the last bit, and numpy.ma computes
        # x ** 0.5 with NumPy's power (not correctly rounded) where the GPU takes the square
        # root; which elements are written, signs, zeros and infinities still have to agree
        # exactly
        tiny = float(np.finfo(dtype).tiny)
        fin = np.isfinite(host) & (np.abs(host) >= tiny)       # results near underflow: absolute
        assert_array_equal(got[~nan & ~np.isfinite(host)], host[~nan & ~np.isfinite(host)], err_msg=name)
        assert_allclose(got[~nan & np.isfinite(host) & ~fin].astype(np.float64),
                        host[~nan & np.isfinite(host) & ~fin].astype(np.float64), rtol=0, atol=tiny)
        assert_allclose(got[fin].astype(np.float64), host[fin].astype(np.float64),
                        rtol=4e-7 if dtype == np.float32 else 1e-3, err_msg=name)
    else:
        assert_array_equal(got.view(u)[~nan], host.view(u)[~nan], err_msg=name)
    if name in ("a/b", "a/0", "a**0.5*b", "a//b", "a%b", "a/b+np.abs(b/a)", "abs(a/b)"):
        assert (host.view(u) == np.array(7.5, dtype).view(u)).sum() > 100   # elements were left alone


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_float_comparisons_store_to_bool_buffers(dtype):
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], lt: Buffer[N, DT], le: Buffer[N, DT],
             eq: Buffer[N, DT], ne: Buffer[N, DT], ge: Buffer[N, DT], gt: Buffer[N, DT], mix: Buffer[N, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        ta, tb = gr.load(a[o:], shape=g), gr.load(b[o:], shape=g)
        gr.store(lt[o:], ta < tb)
        gr.store(le[o:], ta <= tb)
        gr.store(eq[o:], ta == tb)
        gr.store(ne[o:], ta != tb)
        gr.store(ge[o:], ta >= tb)
        gr.store(gt[o:], ta > tb)
        gr.store(mix[o:], ta / tb > dtype(0.5))        # inactive where the division failed

    rng = np.random.default_rng(5)
    n = 10_007
    a, b = _special_floats(rng, n, dtype), _special_floats(rng, n, dtype)
    b[::7] = a[::7]
    hosts = [np.zeros(n, bool) for _ in range(7)]
    for h in hosts:
        h[::3] = True
    devs = [rt.to_device(h) for h in hosts]
    kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), *devs)
    with np.errstate(all="ignore"):
        sim_kernel(work_shape=N, group_shape=256)(body)(a, b, *hosts)
    for d, h, name in zip(devs, hosts, ["lt", "le", "eq", "ne", "ge", "gt", "mix"]):
        assert_array_equal(d.to_host(), h, err_msg=name)


def test_sum_skips_elements_a_division_deactivated():
    """`acc += (a / b).sum()`: numpy.ma's sum leaves deactivated elements out."""
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], acc: Buffer[1, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        atomic_ref(acc)[0] += (gr.load(a[o:], shape=g) / gr.load(b[o:], shape=g) + np.float32(1)).sum()

    rng = np.random.default_rng(6)
    n = 100_003
    a = rng.standard_normal(n).astype(np.float32)
    b = rng.integers(-3, 4, n).astype(np.float32)          # a seventh of the divisors are zero
    host = np.zeros(1, np.float32)
    dacc = rt.to_device(host)
    kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), dacc)
    ok = b != 0
    want = (a[ok].astype(np.float64) / b[ok] + 1).sum()
    assert (~ok).sum() > 10_000
    assert_allclose(dacc.to_host()[0], want, rtol=1e-5)
    with np.errstate(all="ignore"):
        sim_kernel(work_shape=N, group_shape=256)(body)(a, b, host)
    assert_allclose(host[0], want, rtol=1e-4)


def test_row_programs_leave_deactivated_elements_alone():
    """Row reductions and stores under numpy.ma's rules: a row divided by its own
    zero sum is left as it was, a sum leaves out the elements a division or a
    domain function deactivated, and a result that is a bare numpy.ma array
    (a NumPy function on the left) is written in full."""
    M, N, GM = sym.M, sym.N, sym.GM
    f = np.float32

    def normalise(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        gr.store(out[m0:, :], t / t.sum(axis=1, keepdims=True))

    def sum_of_quotients(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], out: Buffer[M, DT],
                         gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        a, b = gr.load(x[m0:, :], shape=(mb, N)), gr.load(y[m0:, :], shape=(mb, N))
        gr.store(out[m0:], (a / b + f(1)).sum(axis=1))

    def log_then_max(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        lg = np.log(t)                                    # 1 where t <= 0, and inactive there
        gr.store(out[m0:, :], t * lg - (t * lg).max(axis=1, keepdims=True))

    def exp_over_sum(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        e = np.exp(t)
        gr.store(out[m0:, :], e / (t * f(0) + t.sum(axis=1, keepdims=True)))   # a bare array on the left

    rng = np.random.default_rng(12)
    rows, n = 37, 1000
    x = rng.standard_normal((rows, n)).astype(f)
    x[3] = 0
    x[5, ::2] = 1; x[5, 1::2] = -1                        # sums to zero exactly
    x[7, :10] = -np.abs(x[7, :10])
    y = rng.integers(-3, 4, (rows, n)).astype(f)
    deco = dict(work_shape=M, group_shape=4)
    for body, ins, shape, tol in ((normalise, (x,), (rows, n), 2e-5), (sum_of_quotients, (x, y), (rows,), 2e-4),
                                  (log_then_max, (x,), (rows, n), 2e-5), (exp_over_sum, (x,), (rows, n), 2e-5)):
        host = np.full(shape, 7.5, f)
        dout = rt.to_device(host)
        kernel(**deco)(body)(*[rt.to_device(v) for v in ins], dout, 4)
        assert rt.last_kernel_name().startswith("hcamd_row_program"), body.__name__
        with np.errstate(all="ignore"):
            sim_kernel(**deco)(body)(*ins, host, 4)
        got = dout.to_host()
        untouched = host == f(7.5)
        assert_array_equal(got == f(7.5), untouched, err_msg=body.__name__)
        nan = np.isnan(host)
        assert_array_equal(np.isnan(got), nan, err_msg=body.__name__)
        assert_allclose(got[~nan], host[~nan], rtol=tol, atol=tol, err_msg=body.__name__)
        if body is normalise:
            assert untouched[3].all() and untouched[5].all() and not untouched[0].any()


@pytest.mark.parametrize("rows,n", [(37, 1000), (300, 8192), (41, 64)])
def test_row_bodies_whose_row_scalars_can_fail_take_two_launches(rows, n):
    """Bodies whose only deactivations are failed operations on row scalars (the
    mean's division, a root, a logarithm): the chain kernel runs every row and
    leaves a row on which one failed to the general kernel.  Rows of zeros (a
    zero norm: nothing of the row is stored), rows with an infinity (a mean that
    is not finite), rows whose squares overflow; against the host executor,
    including which elements are written, and against the general kernel alone."""
    M, N, GM = sym.M, sym.N, sym.GM
    f = np.float32

    def make(fn):
        def body(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            t = gr.load(x[m0:, :], shape=(mb, N))
            gr.store(out[m0:, :], fn(t))
        return body

    bodies = {
        "centre": lambda t: t - t.mean(axis=1, keepdims=True),
        "l2": lambda t: t / np.sqrt((t * t).sum(axis=1, keepdims=True)),
        "rms": lambda t: t / np.sqrt((t * t).mean(axis=1, keepdims=True) + f(1e-6)),
        "log_softmax": lambda t: (t - t.max(axis=1, keepdims=True))
        - np.log(np.exp(t - t.max(axis=1, keepdims=True)).sum(axis=1, keepdims=True)),
        "log_of_sum": lambda t: t - np.log(t.sum(axis=1, keepdims=True)),
    }
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, n)).astype(f)
    x[3] = 0
    x[5, 7] = np.inf
    x[6] *= f(1e25)                                       # squares overflow
    x[9] = -np.abs(x[9])                                  # a negative sum under the logarithm
    x[11, 2] = -np.inf
    deco = dict(work_shape=M, group_shape=4)
    for name, fn in bodies.items():
        body = make(fn)
        host = np.full((rows, n), 7.5, f)
        with np.errstate(all="ignore"):
            sim_kernel(**deco)(body)(x, host, 4)
        results = {}
        for variant in (0, 3):
            rt.set_variant("rows", variant)
            try:
                dout = rt.to_device(np.full((rows, n), 7.5, f))
                kernel(**deco)(body)(rt.to_device(x), dout, 4)
            finally:
                rt.set_variant("rows", 0)
            assert rt.last_kernel_name().startswith("hcamd_row_program_w"), name   # the general kernel ran last
            got = results[variant] = dout.to_host()
            untouched = host == f(7.5)
            assert_array_equal(got == f(7.5), untouched, err_msg=f"{name} variant {variant}")
            nan = np.isnan(host)
            assert_array_equal(np.isnan(got), nan, err_msg=f"{name} variant {variant}")
            # (the host executor continues in float64 after a mean; the large row shows it)
            assert_allclose(got[~nan], host[~nan], rtol=3e-4, atol=2e-4, err_msg=f"{name} variant {variant}")
        assert_allclose(results[0], results[3], rtol=3e-4, atol=2e-4, equal_nan=True, err_msg=name)
        if name == "l2":
            assert (host[3] == f(7.5)).all() and not (host[0] == f(7.5)).any()
        if name == "log_of_sum":
            assert (host[9] == f(7.5)).all()


def test_column_reductions_leave_deactivated_elements_out():
    """`(a / b).sum(axis=0)` and `(a / b).max(axis=0)`: numpy.ma's reductions skip
    the elements a zero divisor deactivated; same body on the GPU and on the host
    executor."""
    M, N, GN = sym.M, sym.N, sym.GN

    def body(fn):
        def k(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], out: Buffer[N, DT], gn: GN):
            n0 = gr.id[0] * GN
            tx, ty = gr.load(x[:, n0:], shape=(M, GN)), gr.load(y[:, n0:], shape=(M, GN))
            gr.store(out[n0:], fn(tx, ty))
        return k

    rng = np.random.default_rng(21)
    rows, n, gn = 777, 200, 64
    x = rng.standard_normal((rows, n)).astype(np.float32)
    y = rng.integers(-2, 3, (rows, n)).astype(np.float32)          # a fifth of the divisors are zero
    y[:, 7] = 0              # a column without an active quotient: numpy.ma stores 0 for its sum, 1e20 for its maximum
    y[:, 130] = 0
    deco = dict(work_shape=cdiv(n, gn), group_shape=1, literals={GN})
    for name, fn in (("sum", lambda a, b: (a / b).sum(axis=0)), ("max", lambda a, b: (a / b).max(axis=0)),
                     ("sum_sqrt", lambda a, b: np.sqrt(a * b).sum(axis=0)),
                     ("min_log", lambda a, b: np.log(a * b).min(axis=0))):
        want = np.zeros(n, np.float32)
        with np.errstate(all="ignore"):
            sim_kernel(**deco)(body(fn))(x, y, want, gn)
        out = rt.DeviceArray((n,), np.float32).fill_bytes32(0xA5A5A5A5)
        kernel(**deco)(body(fn))(rt.to_device(x), rt.to_device(y), out, gn)
        assert rt.last_kernel_name().startswith(("hcamd_map", "hcamd_cols_fold_f32")), name
        assert np.isfinite(want).all(), name
        assert_allclose(out.to_host(), want, rtol=2e-4, atol=2e-4, err_msg=name)


# forms of the fixture's case that have no native kernel: a scalar result, `&`
# of two plain bool arrays
_PLAIN_AND_BARE_REFUSED = {"w_sum", "mask_and_mask"}


def test_plain_and_bare_arrays_next_to_tiles_match_the_reference_simulator():
    """numpy.where returns a plain NumPy array and a NumPy function of a tile a
    bare numpy.ma array; what they do next to numbers, each other and tiles
    (NumPy's own arithmetic, numpy.ma's operators, TypeError for a plain array
    or a NumPy scalar on the left of a tile) is pinned by vectors written by the
    reference simulator (tests/golden/sim_cases.py,
    case_plain_and_bare_arrays_next_to_tiles); the same bodies run here through
    @kernel and every stored value is compared with those vectors bit for bit
    (numpy.log: 2 ulp)."""
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
    import sim_cases
    from hc_amd.binding import NoNativeKernel
    golden = sim_cases.load(os.path.join(os.path.dirname(__file__), "golden", "sim_golden.json"))
    case = "plain_and_bare_arrays_next_to_tiles/"
    f = np.float32
    x = np.array([1.0, 0.0, -0.0, np.inf, np.nan, 4.0, -2.0, 0.5, -1.0, 3.0, -np.inf, 2.5], f)
    y = np.array([2.0, 0.0, 1.0, 1.0, 1.0, 0.0, 0.0, -1.0, 1.0, -2.0, 2.0, 0.0], f)
    N = sym.N
    dx, dy = rt.to_device(x[:11].copy()), rt.to_device(y[:11].copy())
    refused = set()
    for i, (name, fn) in enumerate(sim_cases.PLAIN_AND_BARE_FORMS.items()):
        is_bool = case + name + ".dtype" in golden and bytes(golden[case + name + ".dtype"]) == b"bool"
        # (the arrays end one element before the tiles do, as in the fixture: the
        # last element of every tile is inactive)
        want = golden[case + ("dst_bool" if is_bool else "dst")][i][:11]
        out = rt.to_device(np.full(11, True) if is_bool else np.full(11, sim_cases.POISON, f))

        @kernel(work_shape=N, group_shape=12)
        def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, typename.DT2]):
            gr.store(out[0:], fn(gr.load(a[0:], shape=12), gr.load(b[0:], shape=12)))

        if case + name + ".raises" in golden:
            with pytest.raises(TypeError):
                body(dx, dy, out)
            continue
        try:
            body(dx, dy, out)
        except NoNativeKernel:
            refused.add(name)
            continue
        got = out.to_host()
        if name == "log_w":
            assert_array_equal(np.isnan(got), np.isnan(want), err_msg=name)
            assert_allclose(got, want, rtol=3e-7, err_msg=name)
        elif is_bool:
            assert_array_equal(got, want, err_msg=name)
        else:
            nan = np.isnan(want)
            assert_array_equal(np.isnan(got), nan, err_msg=f"{name}: got {got.tolist()} want {want.tolist()}")
            assert_array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan],
                               err_msg=f"{name}: got {got.tolist()} want {want.tolist()}")
    assert refused == _PLAIN_AND_BARE_REFUSED, refused


def test_random_bodies_match_the_simulator():
    """Random elementwise bodies that lean on numpy.ma's rules
    (tests/random_bodies.py: zero divisors, domains, numpy.where, bare and plain
    arrays next to tiles, signed zeros, NaN, infinities), 1-D and 2-D, fp32 and
    fp16, on the device against the host executor: the same NaNs, the same bits
    elsewhere (a few ulp for transcendental functions).  Whatever kernel the
    binder picks runs; a body either side refuses is refused by both or has no
    native kernel."""
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    N, M = sym.N, sym.M
    tally = {"ok": 0, "refused": 0, "both raise": 0}
    for seed in range(600):
        fn, text, dtype, vals, shape = random_bodies.case(seed)
        if len(shape) == 1:
            def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT], out: Buffer[N, DT]):
                o = gr.work_offset[0]
                gr.store(out[o:], fn(*(gr.load(v[o:], shape=gr.shape) for v in (a, b, c))))
            deco = dict(work_shape=N, group_shape=256)
        else:
            def body(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], c: Buffer[M, N, DT],
                     out: Buffer[M, N, DT]):
                i, j = gr.work_offset
                gr.store(out[i:, j:], fn(*(gr.load(v[i:, j:], shape=gr.shape) for v in (a, b, c))))
            deco = dict(work_shape=(M, N), group_shape=(4, 64))
        want = np.full(shape, 7.5, dtype)
        sim_raises = False
        try:
            with np.errstate(all="ignore"), warnings.catch_warnings():
                warnings.simplefilter("ignore")
                sim_kernel(**deco)(body)(*vals, want)
        except TypeError:                      # a NumPy scalar or plain array on the left of a tile
            sim_raises = True
        out = rt.to_device(np.full(shape, 7.5, dtype))
        try:
            kernel(**deco)(body)(*[rt.to_device(v) for v in vals], out)
        except NoNativeKernel:
            tally["refused"] += 1
            continue
        except TypeError:
            assert sim_raises, f"seed {seed}: {text}: only the front-end raises TypeError"
            tally["both raise"] += 1
            continue
        assert not sim_raises, f"seed {seed}: {text}: only the simulator raises TypeError"
        diff = random_bodies.difference(out.to_host(), want, text)
        assert diff is None, f"seed {seed}: {text} ({np.dtype(dtype).name}, {rt.last_kernel_name()}): {diff}"
        tally["ok"] += 1
    assert tally["ok"] > 400, tally


def test_random_row_bodies_match_the_simulator():
    """Random elementwise expressions of two tiles and of reductions along their
    rows (tests/random_bodies.py: sums, maxima, minima, means, variances,
    standard deviations; divisions by zero, roots of negative numbers, NumPy
    functions next to operators; data with zeros of both signs, and infinities
    and NaN where no mean, var or std is taken) on the device against the host
    executor: the same elements stored, NaN where it has NaN, values to 1e-4."""
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    from test_fmap_programs_against_oracle import row_body
    poison = np.float32(-77.0)
    tally = {"ok": 0, "refused": 0}
    for seed in range(500):
        fn, text, per_row, (a, b) = random_bodies.row_case(seed)
        shape = (a.shape[0],) if per_row else a.shape
        want = np.full(shape, poison)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            row_body(sim_kernel, fn, per_row)(a, b, want, 4)
        out = rt.to_device(np.full(shape, poison))
        try:
            row_body(kernel, fn, per_row)(rt.to_device(a), rt.to_device(b), out, 4)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        got = out.to_host()
        where = f"seed {seed}: {text} ({rt.last_kernel_name()})"
        assert_array_equal(got == poison, want == poison, err_msg=where)
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=where)
        assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=where)
        tally["ok"] += 1
    assert tally["ok"] > 400, tally


def test_random_column_bodies_match_the_simulator():
    """Random reductions down the columns of elementwise expressions, with what
    may follow them per column (tests/random_bodies.py: a root, a logarithm, a
    division by zero, a second fold), on the device against the host executor:
    the same NaNs, values to 1e-4.  numpy.sqrt / numpy.log of a fold give
    numpy.ma's fill values where the domain fails and a failed division leaves
    its dividend, as the result is a bare array that is written in full."""
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    M, N, GN = sym.M, sym.N, sym.GN
    poison = np.float32(-77.0)
    tally = {"ok": 0, "refused": 0}
    for seed in range(400):
        fn, text, (a, b), gn = random_bodies.col_case(seed)
        n = a.shape[1]

        def body(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], out: Buffer[N, DT], g: GN):
            n0 = gr.id[0] * GN
            gr.store(out[n0:], fn(gr.load(x[:, n0:], shape=(M, GN)), gr.load(y[:, n0:], shape=(M, GN))))

        deco = dict(work_shape=cdiv(n, gn), group_shape=1, literals={GN})
        want = np.full(n, poison)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            sim_kernel(**deco)(body)(a, b, want, gn)
        out = rt.to_device(np.full(n, poison))
        try:
            kernel(**deco)(body)(rt.to_device(a), rt.to_device(b), out, gn)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        got = out.to_host()
        where = f"seed {seed}: {text} ({rt.last_kernel_name()})"
        assert_array_equal(got == poison, want == poison, err_msg=where)
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=where)
        assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=where)
        tally["ok"] += 1
    assert tally["ok"] > 200, tally


def test_random_bodies_with_a_row_vector_and_a_per_row_operand_match_the_simulator():
    """The random row bodies with two more operands that broadcast: a row vector
    (a weight, a bias) and a per-row operand (a scale per row), as in the
    reference's normalisation and softmax-with-temperature bodies.  A per-row
    result that is a tile (the per-row operand on the left of the tile operators)
    keeps its deactivated rows out of the store."""
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    M, N, GM = sym.M, sym.N, sym.GM
    poison = np.float32(-77.0)

    def bodies(deco, fn, per_row):
        if per_row:
            @deco(work_shape=M, group_shape=GM)
            def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], w: Buffer[N, DT], s: Buffer[M, DT],
                  out: Buffer[M, DT], g: GM):
                m0, mb = gr.work_offset[0], gr.shape[0]
                gr.store(out[m0:], fn(gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N)),
                                      gr.load(w[:], shape=(N,)), gr.load(s[m0:], shape=(mb,))))
        else:
            @deco(work_shape=M, group_shape=GM)
            def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], w: Buffer[N, DT], s: Buffer[M, DT],
                  out: Buffer[M, N, DT], g: GM):
                m0, mb = gr.work_offset[0], gr.shape[0]
                gr.store(out[m0:, :], fn(gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N)),
                                         gr.load(w[:], shape=(N,)), gr.load(s[m0:], shape=(mb,))))
        return k

    tally = {"ok": 0, "refused": 0}
    for seed in range(400):
        fn, text, per_row, vals = random_bodies.vector_case(seed)
        shape = (vals[0].shape[0],) if per_row else vals[0].shape
        want = np.full(shape, poison)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            bodies(sim_kernel, fn, per_row)(*vals, want, 4)
        out = rt.to_device(np.full(shape, poison))
        try:
            bodies(kernel, fn, per_row)(*[rt.to_device(v) for v in vals], out, 4)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        got = out.to_host()
        where = f"seed {seed}: {text} ({rt.last_kernel_name()})"
        assert_array_equal(got == poison, want == poison, err_msg=where)
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=where)
        assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=where)
        tally["ok"] += 1
    assert tally["ok"] > 300, tally


def test_numpy_where_of_int32_tiles():
    """numpy.where of integer tiles as the stored value (the guarded division
    `numpy.where(b != 0, a // b, 0)` among them): picked from the values, the
    dividend under a failed //, 1 under a failed %, every element stored; same
    bodies on the host executor.  Arithmetic on top of a quotient inside the
    selection is refused."""
    from hc_amd.binding import NoNativeKernel
    N = sym.N
    I = np.int32
    rng = np.random.default_rng(31)
    n = 5003
    a = rng.integers(-40, 41, n).astype(I)
    b = rng.integers(-3, 4, n).astype(I)            # a seventh of the divisors are zero
    a[:3] = [np.iinfo(I).min, np.iinfo(I).min, 7]
    b[:3] = [0, -1, 0]
    forms = {
        "guarded": lambda x, y: np.where(y != I(0), x // y, I(0)),
        "unguarded": lambda x, y: np.where(x < y, x // y, x % y),
        "plain": lambda x, y: np.where(x * y > I(10), x - y, y),
        "numbers": lambda x, y: np.where(x >= y, I(1), I(-1)),
    }
    for name, fn in forms.items():
        def body(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], out: Buffer[N, DT]):
            o = gr.work_offset[0]
            gr.store(out[o:], fn(gr.load(x[o:], shape=gr.shape), gr.load(y[o:], shape=gr.shape)))
        want = np.full(n, -777, I)
        with np.errstate(all="ignore"):
            sim_kernel(work_shape=N, group_shape=256)(body)(a, b, want)
        out = rt.to_device(np.full(n, -777, I))
        kernel(work_shape=N, group_shape=256)(body)(rt.to_device(a), rt.to_device(b), out)
        assert rt.last_kernel_name() == "hcamd_imap_i32"
        assert_array_equal(out.to_host(), want, err_msg=name)
        assert (want != -777).all()

    def on_top(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], out: Buffer[N, DT]):
        o = gr.work_offset[0]
        tx, ty = gr.load(x[o:], shape=gr.shape), gr.load(y[o:], shape=gr.shape)
        gr.store(out[o:], np.where(tx < ty, tx // ty + I(1), ty))
    with pytest.raises(NoNativeKernel, match="numpy.where of integer tiles"):
        kernel(work_shape=N, group_shape=256)(on_top)(rt.to_device(a), rt.to_device(b), rt.to_device(a))


def test_random_statement_sequences_match_the_simulator():
    """In-place operators and `tile[:] = value` (python/hckernel/kernel_api.py:123-145:
    tile op= x is tile[:] = tile op x, which takes the value's active elements
    only -- an element whose result is deactivated keeps its value and its
    activity), allocated tiles, rebinding: random sequences of such statements
    on the device against the host executor, bit for bit (exp: a few ulp)."""
    import sys
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    api = sys.modules["hckernel.kernel"]
    tally = {"ok": 0, "refused": 0, "both raise": 0}
    for seed in range(600):
        body, text, deco, vals = random_bodies.statement_body(seed, api)
        want = np.full(vals[0].shape, np.float32(-77))
        sim_raises = False
        try:
            with np.errstate(all="ignore"), warnings.catch_warnings():
                warnings.simplefilter("ignore")
                sim_kernel(**deco)(body)(*vals, want)
        except TypeError:
            sim_raises = True
        out = rt.to_device(np.full(vals[0].shape, np.float32(-77)))
        try:
            kernel(**deco)(body)(*[rt.to_device(v) for v in vals], out)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        except TypeError:
            assert sim_raises, f"seed {seed}: {text}: only the front-end raises TypeError"
            tally["both raise"] += 1
            continue
        assert not sim_raises, f"seed {seed}: {text}: only the simulator raises TypeError"
        got = out.to_host()
        if "exp" in text:                      # exp of exp amplifies the last bits
            assert_array_equal(np.isnan(got), np.isnan(want), err_msg=f"seed {seed}: {text}")
            assert_allclose(got, want, rtol=2e-5, atol=1e-6, err_msg=f"seed {seed}: {text}")
        else:
            diff = random_bodies.difference(got, want, text)
            assert diff is None, f"seed {seed}: {text} ({rt.last_kernel_name()}): {diff}"
        tally["ok"] += 1
    assert tally["ok"] > 300, tally


def test_random_int32_statement_sequences_match_the_simulator():
    """Random statements and expressions of int32 tiles (tests/random_bodies.py) on
    the device against the host executor, exactly: zero divisors, INT_MIN as a
    dividend and as a divisor (numpy.ma's test deactivates every quotient by
    INT_MIN), bare arrays written in full with numpy.ma's leftovers, numpy.where."""
    import sys
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    api = sys.modules["hckernel.kernel"]
    tally = {"ok": 0, "refused": 0, "both raise": 0}
    for seed in range(600):
        body, text, deco, vals = random_bodies.int_statement_body(seed, api)
        want = np.full(vals[0].shape, np.int32(-777))
        sim_raises = False
        try:
            with np.errstate(all="ignore"), warnings.catch_warnings():
                warnings.simplefilter("ignore")
                sim_kernel(**deco)(body)(*vals, want)
        except TypeError:
            sim_raises = True
        out = rt.to_device(np.full(vals[0].shape, np.int32(-777)))
        try:
            kernel(**deco)(body)(*[rt.to_device(v) for v in vals], out)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        except TypeError:
            assert sim_raises, f"seed {seed}: {text}: only the front-end raises TypeError"
            tally["both raise"] += 1
            continue
        assert not sim_raises, f"seed {seed}: {text}: only the simulator raises TypeError"
        assert_array_equal(out.to_host(), want, err_msg=f"seed {seed}: {text}")
        tally["ok"] += 1
    assert tally["ok"] > 350, tally


def test_random_statement_sequences_in_row_bodies_match_the_simulator():
    """In-place operators with row scalars (`t -= t.max(axis=1, keepdims=True)`,
    `t /= u.sum(axis=1, keepdims=True)`: where the divisor is zero the element
    keeps its value and stays active), rebinding to NumPy functions, then a store:
    random sequences on the device against the host executor."""
    import sys
    import warnings
    import random_bodies
    from hc_amd.binding import NoNativeKernel
    from hc_amd.kernel_api import TraceError
    api = sys.modules["hckernel.kernel"]
    poison = np.float32(-7777.25)
    tally = {"ok": 0, "refused": 0}
    for seed in range(300):
        body, text, deco, vals = random_bodies.row_statement_body(seed, api)
        want = np.full(vals[0].shape, poison)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            sim_kernel(**deco)(body)(*vals, want, 4)
        out = rt.to_device(np.full(vals[0].shape, poison))
        try:
            kernel(**deco)(body)(*[rt.to_device(v) for v in vals], out, 4)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        got = out.to_host()
        where = f"seed {seed}: {text} ({rt.last_kernel_name()})"
        assert_array_equal(got == poison, want == poison, err_msg=where)
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=where)
        assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=where)
        tally["ok"] += 1
    assert tally["ok"] > 200, tally


def test_expressions_of_several_column_reductions():
    """`(x * x).mean(axis=0) - x.mean(axis=0) ** 2` and the like: every reduction
    down the columns runs into a temporary vector and the general float map
    combines them under numpy.ma's rules (a zero divisor leaves the dividend,
    the result is written in full); same bodies on the host executor."""
    M, N, GN = sym.M, sym.N, sym.GN
    f = np.float32
    rng = np.random.default_rng(77)
    rows, n, gn = 300, 200, 64
    x = rng.standard_normal((rows, n)).astype(f)
    y = (np.abs(rng.standard_normal((rows, n))) + 0.1).astype(f)       # (sums without cancellation)
    y[:, 5] = 0                                  # a column whose sum is zero: a / 0 leaves a
    forms = {
        "variance": lambda a, b: (a * a).mean(axis=0) - a.mean(axis=0) ** f(2),
        "ratio": lambda a, b: a.sum(axis=0) / b.sum(axis=0),
        "range": lambda a, b: a.max(axis=0) - a.min(axis=0),
        "cosine": lambda a, b: (a * b).sum(axis=0) / np.sqrt((a * a).sum(axis=0) * (b * b).sum(axis=0)),
        "same_twice": lambda a, b: a.sum(axis=0) * a.sum(axis=0) + b.std(axis=0),
    }
    for name, fn in forms.items():
        def body(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[N, DT], g: GN):
            n0 = gr.id[0] * GN
            gr.store(out[n0:], fn(gr.load(a[:, n0:], shape=(M, GN)), gr.load(b[:, n0:], shape=(M, GN))))
        deco = dict(work_shape=cdiv(n, gn), group_shape=1, literals={GN})
        want = np.full(n, f(-77))
        with np.errstate(all="ignore"):
            sim_kernel(**deco)(body)(x, y, want, gn)
        out = rt.to_device(np.full(n, f(-77)))
        kernel(**deco)(body)(rt.to_device(x), rt.to_device(y), out, gn)
        assert rt.last_kernel_name() in ("hcamd_fmap", "hcamd_fmap_v8"), name
        got = out.to_host()
        assert (got != f(-77)).all(), name
        assert_array_equal(np.isnan(got), np.isnan(want), err_msg=name)
        assert_allclose(got, want, rtol=2e-4, atol=2e-4, err_msg=name)
