"""The `@kernel` front-end without a GPU: symbol binding, launch-geometry
defaults, tracing of kernel bodies written against the reference's API, and the
binding of the traced program to the typed C entry points (which entry point,
which pointers, leading dimensions and window sizes).  Arrays are stand-ins
that expose __cuda_array_interface__ with made-up device addresses; nothing is
launched."""

import numpy as np
import pytest
import sympy

from hc_amd import runtime as rt
from hc_amd.kernel import (Buffer, CurrentGroup, NoNativeKernel, TunableParam, atomic_ref, kernel,
                           suggest_group_shape, sym, typename)
from oracle import closed_forms as cf

DT = typename.DT
CODES = {"float32": "<f4", "float16": "<f2", "int8": "|i1", "int32": "<i4", "bfloat16": "<u2",
         "bool": "|b1"}


class FakeDev:
    """Device-array stand-in: shape, dtype and a fake address."""
    _next = 0x7F00_0000_0000

    def __init__(self, shape, dtype, ld=None):
        self.shape = tuple(shape)
        self.bf16 = dtype == "bfloat16"
        self.dtype = np.dtype("uint16" if self.bf16 else dtype)
        item = self.dtype.itemsize
        FakeDev._next += 1 << 32
        self.ptr = FakeDev._next
        strides = None
        if ld is not None:
            strides = (ld * item, item)
        self.__cuda_array_interface__ = {"shape": self.shape, "typestr": CODES[str(dtype)],
                                         "data": (self.ptr, False), "strides": strides,
                                         "version": 2}


@pytest.fixture
def ctx():
    c = rt.Context.__new__(rt.Context)      # no device behind it: plans are built, never launched
    c.queue, c.device, c.messages = 0x1234, 0x5678, []
    return c


def cdiv(a, b):
    return (a + b - 1) // b


def test_default_group_shape_comes_from_the_block_size_suggestion():
    for work in [(16_777_259,), (8191, 8193), (256, 64), (1, 27), (111, 813), (4, 5, 6)]:
        assert suggest_group_shape(work) == cf.default_group_shape(work)


def test_copy_kernel_of_the_reference_e2e_test_binds_to_copy2d(ctx):
    W, H = sym.W, sym.H

    @kernel(work_shape=(W, H))
    def copy_kernel(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x, y = group.work_offset
        val = group.load(src[x:, y:], shape=group.shape)
        group.store(dst[x:, y:], val)

    for shape in [(1, 27), (10, 20), (111, 813), (256, 1024)]:
        a, b = FakeDev(shape, "int32"), FakeDev(shape, "int32")
        (p,) = copy_kernel.plan(a, b, ctx=ctx)
        assert p.fn is rt.hcamdLaunchCopy2D
        assert p.args == (ctx.queue, 4, a.ptr, shape[0], shape[1], shape[1], 1,
                          b.ptr, shape[0], shape[1], shape[1], 1)


@pytest.mark.parametrize("literal", [False, True])
@pytest.mark.parametrize("unroll", [1, 2, 4])
def test_unrolled_copy_kernels_cover_the_same_window(ctx, unroll, literal):
    W, H, V = sym.W, sym.H, sym.V
    H1 = sympy.ceiling(H / V)

    @kernel(work_shape=(W, H1), literals=[V] if literal else ())
    def copy_kernel(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT], v: V):
        x, y = group.work_offset
        load = group.vload if literal else group.load
        val = load(src[x:, y * V:], shape=(group.shape[0], group.shape[1] * V))
        group.store(dst[x:, y * V:], val)

    a, b = FakeDev((111, 813), "int32"), FakeDev((111, 813), "int32")
    (p,) = copy_kernel.plan(a, b, unroll, ctx=ctx)
    assert p.fn is rt.hcamdLaunchCopy2D and p.args[3:5] == (111, 813)


def test_copy_into_a_larger_destination_copies_the_common_window(ctx):
    W, H, W2, H2 = sym.W, sym.H, sym.W2, sym.H2

    @kernel(work_shape=(W2, H2), group_shape=(4, 64))
    def k(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W2, H2, DT]):
        x, y = group.work_offset
        group.store(dst[x:, y:], group.load(src[x:, y:], shape=group.shape))

    a, b = FakeDev((37, 101), "float16"), FakeDev((50, 130), "float16", ld=136)
    (p,) = k.plan(a, b, ctx=ctx)
    assert p.args == (ctx.queue, 2, a.ptr, 37, 101, 101, 1, b.ptr, 37, 101, 136, 1)


def test_vector_add_binds_to_add_f32(ctx):
    N = sym.N

    @kernel(work_shape=N, group_shape=256)
    def vadd(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(c[o:], gr.load(a[o:], shape=gr.shape[0]) + gr.load(b[o:], shape=gr.shape[0]))

    n = 16_777_259
    a, b, c = (FakeDev((n,), "float32") for _ in range(3))
    (p,) = vadd.plan(a, b, c, ctx=ctx)
    assert p.fn is rt.hcamdLaunchAddF32 and p.args == (ctx.queue, a.ptr, b.ptr, c.ptr, n)
    # second call: cached binding, fresh pointers
    a2 = FakeDev((n,), "float32")
    (p2,) = vadd.plan(a2, b, c, ctx=ctx)
    assert p2.args[1] == a2.ptr and len(vadd._cache) == 1
    # fp16 arrays: no dedicated kernel, the fused map runs "add, round to fp16"
    (p3,) = vadd.plan(*(FakeDev((n,), "float16") for _ in range(3)), ctx=ctx)
    assert p3.fn is rt.hcamdLaunchMap
    assert map_program(p3) == [("in", 0, 0.0), ("add_in", 1, 0.0), ("r16", 0, 0.0)]
    # int32 arrays: the integer map kernel
    (p4,) = vadd.plan(*(FakeDev((n,), "int32") for _ in range(3)), ctx=ctx)
    assert p4.fn is rt.hcamdLaunchIMap and imap_program(p4) == [("in", 0, 0), ("in", 1, 0), ("add", 0, 0)]
    with pytest.raises(NoNativeKernel):
        vadd.plan(*(FakeDev((n,), "int8") for _ in range(3)), ctx=ctx)


def imap_program(plan):
    """(opname, arg, int immediate) triples of a hcamdLaunchIMap plan."""
    import ctypes as C
    names = {v: k for k, v in rt.IMAP_OPS.items()}
    prog, n = plan.args[1], plan.args[2]
    out = []
    for i in range(n):
        imm = C.c_int32.from_buffer_copy(bytes(C.string_at(C.addressof(prog[i]) + rt.MapInstr.imm.offset, 4)))
        out.append((names[prog[i].op], prog[i].arg, imm.value))
    return out


def test_integer_tile_operators_bind_to_the_integer_map(ctx):
    """The operators the reference's tile wrapper forwards for integer tiles
    (python/hckernel/kernel_api.py:157-180): arithmetic, floor division and
    remainder, bitwise, shifts, comparisons."""
    R, Cc = sym.R, sym.C
    i32 = np.int32

    @kernel(work_shape=(R, Cc), group_shape=(4, 64))
    def k(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT],
          flag: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta, tb = gr.load(a[x:, y:], shape=gr.shape), gr.load(b[x:, y:], shape=gr.shape)
        gr.store(out[x:, y:], ((ta * tb - i32(7)) // (tb | i32(1))) % i32(13) + (ta >> i32(2) ^ tb << i32(3)))
        gr.store(flag[x:, y:], np.minimum(ta, tb) <= -abs(tb) & i32(255))

    a, b, out = (FakeDev((37, 130), "int32") for _ in range(3))
    flag = FakeDev((37, 130), "bool")
    p1, p2 = k.plan(a, b, out, flag, ctx=ctx)
    assert p1.fn is rt.hcamdLaunchIMap and p2.fn is rt.hcamdLaunchIMap
    assert imap_program(p1) == [
        ("in", 0, 0), ("in", 1, 0), ("mul", 0, 0), ("const", 0, 7), ("sub", 0, 0),
        ("in", 1, 0), ("const", 0, 1), ("or", 0, 0), ("floordiv", 0, 0), ("const", 0, 13),
        ("mod", 0, 0), ("in", 0, 0), ("const", 0, 2), ("shr", 0, 0), ("in", 1, 0), ("const", 0, 3),
        ("shl", 0, 0), ("xor", 0, 0), ("add", 0, 0)]
    assert p1.args[7] == rt.I32 and p1.args[9:11] == (37, 130)
    assert imap_program(p2) == [("in", 0, 0), ("in", 1, 0), ("min", 0, 0), ("in", 1, 0), ("abs", 0, 0),
                                ("neg", 0, 0), ("const", 0, 255), ("and", 0, 0), ("le", 0, 0)]
    assert p2.args[7] == rt.U8

    # what has no native form says so
    @kernel(work_shape=(R, Cc), group_shape=(4, 64))
    def truediv(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        gr.store(out[x:, y:], gr.load(a[x:, y:], shape=gr.shape) / gr.load(b[x:, y:], shape=gr.shape))

    @kernel(work_shape=(R, Cc), group_shape=(4, 64))
    def uses_mask(gr: CurrentGroup, a: Buffer[R, Cc, DT], out: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        gr.store(out[x:, y:], gr.load(a[x:, y:], shape=gr.shape).mask)

    with pytest.raises(NoNativeKernel):
        truediv.plan(a, b, out, ctx=ctx)
    with pytest.raises(NoNativeKernel, match="float64 in NumPy"):
        truediv.plan(a, b, out, ctx=ctx)
    (p,) = uses_mask.plan(a, out, ctx=ctx)              # tile.mask: 0 / 1, every element stored
    assert p.fn is rt.hcamdLaunchIMap and imap_program(p) == [("in", 0, 0), ("active", 0, 0)]


def map_program(plan):
    """(opname, arg, imm) triples of a hcamdLaunchMap plan."""
    names = {v: k for k, v in rt.MAP_OPS.items()}
    prog, n = plan.args[1], plan.args[2]
    return [(names[prog[i].op], prog[i].arg, prog[i].imm) for i in range(n)]


def stack_depth(program):
    sp = deepest = 0
    for name, _, _ in program:
        code = rt.MAP_OPS[name]
        sp += 1 if code <= 2 else (-1 if code <= 10 or code in (35, 36) else 0)   # the rest: one in, one out
        deepest = max(deepest, sp)
    assert sp == 1
    return deepest


def test_elementwise_expressions_compile_to_postfix_programs(ctx):
    N = sym.N
    f = np.float32

    def kern(expr):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT],
              out: Buffer[N, DT]):
            o, g = gr.work_offset[0], gr.shape[0]
            gr.store(out[o:], expr(gr.load(a[o:], shape=g), gr.load(b[o:], shape=g),
                                   gr.load(c[o:], shape=g)))
        return k

    arrs = [FakeDev((1000,), "float32") for _ in range(4)]
    # constants fold into immediates; a reversed immediate form where the
    # constant is on the left
    (p,) = kern(lambda a, b, c: (2.0 - a) * b / 4).plan(*arrs, ctx=ctx)
    # (the tile operator / is numpy.ma's division: the m* forms deactivate failed quotients)
    assert map_program(p) == [("in", 0, 0.0), ("rsubi", 0, 2.0), ("mul_in", 1, 0.0),
                              ("mdivi", 0, 4.0)]
    assert p.args[6] == 2 and p.args[10:] == (1, 1000)        # two operands, 1 x 1000
    # an operand on one side of a binary operation is read by the operation
    # itself: a - (b*c + a/b) evaluates the right side, then "a minus top"
    (p,) = kern(lambda a, b, c: a - (b * c + a / b)).plan(*arrs, ctx=ctx)
    prog = map_program(p)
    assert [i[0] for i in prog] == ["in", "mul_in", "in", "mdiv_in", "add", "rsub_in"]
    assert stack_depth(prog) == 2
    assert p.args[3][prog[-1][1]] == arrs[0].ptr       # operands are numbered by first use
    # the deeper side goes first: (a*b - c*a) / (exp(a) / (b*c + a*a))
    (p,) = kern(lambda a, b, c: (a * b - c * a) / (np.exp(a) / (b * c + a * a))).plan(
        *arrs, ctx=ctx)
    prog = map_program(p)
    assert [i[0] for i in prog] == ["in", "mul_in", "in", "mul_in", "sub",        # numerator
                                    "in", "mul_in", "in", "mul_in", "add",        # b*c + a*a
                                    "in", "exp", "rmdiv", "mdiv"]
    assert stack_depth(prog) == 3
    # ufuncs, clip, maximum with NaN propagation left to the kernel
    (p,) = kern(lambda a, b, c: np.clip(np.exp(-np.abs(a)) + np.maximum(b, c), 0, 6)).plan(
        *arrs, ctx=ctx)
    assert [i[0] for i in map_program(p)] == ["in", "abs", "neg", "exp", "in", "max_in", "add",
                                              "maxi", "mini"]
    # mixed storage: fp16 operands, fp32 math, fp16 result -> one rounding, at the store
    half = [FakeDev((1000,), "float16") for _ in range(4)]
    (p,) = kern(lambda a, b, c: (a.astype(f) * b.astype(f) - c.astype(f)).astype(np.float16)
                ).plan(*half, ctx=ctx)
    assert [i[0] for i in map_program(p)] == ["in", "mul_in", "sub_in", "r16"]
    assert list(p.args[4][:3]) == [rt.F16] * 3 and p.args[8] == rt.F16
    # arithmetic on fp16 tiles rounds after every operation, and a Python
    # scalar is first rounded to fp16 like NumPy does
    (p,) = kern(lambda a, b, c: a * 0.1 + b).plan(*half, ctx=ctx)
    assert map_program(p) == [("in", 0, 0.0), ("muli", 0, float(np.float32(np.float16(0.1)))),
                              ("r16", 0, 0.0), ("add_in", 1, 0.0), ("r16", 0, 0.0)]
    # too deep for the four-entry stack: a balanced tree over 16 sub-expressions
    def deep(a, b, c):
        l = [np.abs(v) for v in (a, b, c) * 5 + (a,)]
        while len(l) > 1:
            l = [x / y for x, y in zip(l[::2], l[1::2])]
        return l[0]
    with pytest.raises(NoNativeKernel, match="stack"):
        kern(deep).plan(*arrs, ctx=ctx)


def test_fused_multiply_add_binds_to_fma_f16(ctx):
    R, Cc = sym.R, sym.C
    f = np.float32

    @kernel(work_shape=(R, Cc))
    def fma(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], c: Buffer[R, Cc, DT],
            d: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta, tb, tc = (gr.load(v[x:, y:], shape=gr.shape) for v in (a, b, c))
        gr.store(d[x:, y:], (ta.astype(f) * tb.astype(f) + tc.astype(f)).astype(np.float16))

    arrs = [FakeDev((8191, 8193), "float16") for _ in range(4)]
    (p,) = fma.plan(*arrs, ctx=ctx)
    assert p.fn is rt.hcamdLaunchFmaF16
    assert p.args == (ctx.queue, arrs[0].ptr, 8193, arrs[1].ptr, 8193, arrs[2].ptr, 8193,
                      arrs[3].ptr, 8193, 8191, 8193)

    # without the fp32 casts the arithmetic rounds to fp16 after the multiply as
    # well: not the fma kernel, but the fused map with an extra rounding step
    @kernel(work_shape=(R, Cc))
    def fma_half(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT],
                 c: Buffer[R, Cc, DT], d: Buffer[R, Cc, DT]):
        x, y = gr.work_offset
        ta, tb, tc = (gr.load(v[x:, y:], shape=gr.shape) for v in (a, b, c))
        gr.store(d[x:, y:], ta * tb + tc)

    (p,) = fma_half.plan(*arrs, ctx=ctx)
    assert p.fn is rt.hcamdLaunchMap
    assert [i[0] for i in map_program(p)] == ["in", "mul_in", "r16", "add_in", "r16"]


def test_softmax_of_the_reference_example_binds_to_softmax_f32(ctx):
    # body of python/hckernel/tests/test_examples.py:304-321
    M, N, GM, MI = sym.M, sym.N, sym.GM, sym.MI

    @kernel(work_shape=cdiv(M, MI), group_shape=GM, tunables=TunableParam(MI, 1, range(1, 8)))
    def softmax(gr: CurrentGroup, a: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m_start = gr.work_offset[0] * MI
        m_block = gr.shape[0] * MI
        a_view = gr.load(a[m_start:, :], shape=(m_block, N))
        exp = np.exp(a_view - a_view.max(axis=1, keepdims=True))
        gr.store(out[m_start:, :], exp / (exp.sum(axis=1, keepdims=True)))

    x, y = FakeDev((4096, 8192), "float32"), FakeDev((4096, 8192), "float32")
    (p,) = softmax.plan(x, y, 8, ctx=ctx)
    assert p.fn is rt.hcamdLaunchSoftmaxF32
    assert p.args == (ctx.queue, x.ptr, 8192, y.ptr, 8192, 4096, 8192)
    y2 = FakeDev((30, 25), "float32")
    (p,) = softmax.parametrize({MI: 4}).plan(FakeDev((30, 25), "float32", ld=32), y2, 8, ctx=ctx)
    assert p.args[2] == 32 and p.args[4] == 25 and p.args[5:] == (30, 25)


def test_row_quantize_binds_to_quantize_f16_i8(ctx):
    M, N, GM = sym.M, sym.N, sym.GM

    @kernel(work_shape=M, group_shape=GM)
    def quant(gr: CurrentGroup, x: Buffer[M, N, DT], q: Buffer[M, N, DT], scale: Buffer[M, DT],
              g: GM):
        m0 = gr.work_offset[0]
        xf = gr.load(x[m0:, :], shape=(gr.shape[0], N)).astype(np.float32)
        s = np.abs(xf).max(axis=1, keepdims=True) / np.float32(127)
        gr.store(q[m0:, :], np.clip(np.rint(xf / s), -127, 127).astype(np.int8))
        gr.store(scale[m0:], s[:, 0])

    x, q, s = FakeDev((16384, 4096), "float16"), FakeDev((16384, 4096), "int8"), \
        FakeDev((16384,), "float32")
    (p,) = quant.plan(x, q, s, 1, ctx=ctx)
    assert p.fn is rt.hcamdLaunchQuantizeF16I8
    assert p.args == (ctx.queue, x.ptr, 4096, q.ptr, 4096, s.ptr, 16384, 4096)


@pytest.mark.parametrize("blocked", [True, False])
def test_dot_kernel_binds_to_gemm_bf16(ctx, blocked):
    # structure of python/hckernel/tests/test_examples.py:74-165 with B column-major
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
        if blocked:
            for k in range(KI):
                r += np.dot(gr.load(a[m0:, k * KB:], shape=(mb, KB)),
                            gr.load(bt[n0:, k * KB:], shape=(nb, KB)).T)
        else:
            r += np.dot(gr.load(a[m0:, :], shape=(mb, K)), gr.load(bt[n0:, :], shape=(nb, K)).T)
        gr.store(out[m0:, n0:], r)

    a, bt, c = (FakeDev((4096, 4096), "bfloat16") for _ in range(3))
    (p,) = dot.plan(a, bt, c, (16, 16), ctx=ctx)
    assert p.fn is rt.hcamdLaunchGemmBF16
    assert p.args == (ctx.queue, a.ptr, 4096, bt.ptr, 4096, c.ptr, 4096, 4096, 4096, 4096)
    a2, bt2, c2 = FakeDev((100, 300), "bfloat16"), FakeDev((200, 300), "bfloat16"), \
        FakeDev((100, 200), "bfloat16")
    (p,) = dot.plan(a2, bt2, c2, (8, 8), ctx=ctx)
    assert p.args[7:] == (100, 200, 300)


def test_symbol_conflicts_and_rank_errors_are_reported():
    W, H = sym.W, sym.H

    @kernel(work_shape=(W, H))
    def k(group: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x, y = group.work_offset
        group.store(dst[x:, y:], group.load(src[x:, y:], shape=group.shape))

    with pytest.raises(RuntimeError, match="Symbol value conflict"):
        k.plan(FakeDev((3, 4), "int32"), FakeDev((3, 5), "int32"), ctx=object())
    with pytest.raises(RuntimeError, match="Invalid rank"):
        k.plan(FakeDev((3,), "int32"), FakeDev((3, 5), "int32"), ctx=object())
    with pytest.raises(RuntimeError, match="host array"):
        k.plan(np.zeros((3, 4), np.int32), np.zeros((3, 4), np.int32), ctx=object())
    with pytest.raises(RuntimeError, match="backend"):
        kernel(work_shape=(W, H), backend="nvvm")(k.func).plan(FakeDev((3, 4), "int32"),
                                                               FakeDev((3, 4), "int32"))


def test_bodies_without_a_native_kernel_fail_loudly(ctx, monkeypatch):
    N = sym.N

    @kernel(work_shape=N, group_shape=64)
    def shifted(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(c[o:], gr.load(a[o + 1:], shape=gr.shape[0]))       # not a disjoint tiling: a gathered copy

    @kernel(work_shape=N, group_shape=64)
    def scaled(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(c[o:], (gr.load(a[o:], shape=gr.shape[0]) * 3.0).sum())   # a reduction

    @kernel(work_shape=N, group_shape=64)
    def nothing(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT]):
        pass

    @kernel(work_shape=N, group_shape=64)
    def scoped(gr: CurrentGroup, a: Buffer[N, DT], c: Buffer[N, DT]):
        @gr.workitems
        def inner(wi):
            pass
        inner()

    a, c = FakeDev((1000,), "float32"), FakeDev((1000,), "float32")
    for k in (scaled, nothing, scoped):
        with pytest.raises(NoNativeKernel):
            k.plan(a, c, ctx=ctx)
    monkeypatch.setattr(rt, "GatherMap", MapTablesOnly)
    (p,) = shifted.plan(a, c, ctx=ctx)
    assert p.fn is rt.hcamdGatherMapLaunch and p.args[-1] == 4          # copy mode, 4-byte elements
    assert MapTablesOnly.last.operands[0][2][:2, 0].tolist() == [1, 65]


def test_decorator_argument_checks():
    with pytest.raises(AssertionError):
        kernel(work_shape=(1, 2, 3, 4))
    with pytest.raises(AssertionError):
        kernel(work_shape=(4, 4), group_shape=(2,))
    with pytest.raises(AssertionError, match="Subgroup size"):
        kernel(work_shape=4, subgroup_size=sym.SG)


def test_reference_reduction_bodies_bind_to_the_map_sum_kernel(ctx):
    # bodies of python/hckernel/tests/test_examples.py:31-71
    WS, GS, N = sym.WS, sym.GS, sym.N
    TN = TunableParam(N, 2, range(1, 64))

    @kernel(work_shape=cdiv(WS, N), group_shape=GS, tunables=TN)
    def reduction_1(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], gshape: GS):
        a_view = gr.load(a[gr.work_offset[0] * N:], shape=gr.size * N)
        atomic_ref(result)[0] += a_view.sum()

    @kernel(work_shape=cdiv(WS, N), group_shape=GS, tunables=TN)
    def reduction_2(group: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], gshape: GS):
        temp_result = group.zeros(group.size, dtype=a.dtype)
        for i in range(N):
            work_offset = group.work_offset[0] * N + i * group.size
            a_view = group.load(a[work_offset:], shape=group.size)
            temp_result += a_view
        atomic_ref(result)[0] += temp_result.sum()

    a, res = FakeDev((20,), "float32"), FakeDev((1,), "float32")
    for k in (reduction_1, reduction_2, reduction_2.parametrize({N: 4})):
        (p,) = k.plan(a, res, 8, ctx=ctx)
        assert p.fn is rt.hcamdLaunchMapSum
        assert map_program(p) == [("in", 0, 0.0)]
        assert p.args[3][0] == a.ptr and p.args[7] == res.ptr and p.args[8:] == (1, 20)

    # a dot product: one pass, the product is formed by the program
    @kernel(work_shape=WS, group_shape=256)
    def dot(gr: CurrentGroup, a: Buffer[WS, DT], b: Buffer[WS, DT], result: Buffer[4, DT]):
        o, g = gr.work_offset[0], gr.shape[0]
        atomic_ref(result)[2] += (gr.load(a[o:], shape=g) * gr.load(b[o:], shape=g)).sum()

    res4 = FakeDev((4,), "float32")
    (p,) = dot.plan(a, FakeDev((20,), "float32"), res4, ctx=ctx)
    assert map_program(p) == [("in", 0, 0.0), ("mul_in", 1, 0.0)] and p.args[7] == res4.ptr + 8

    # what has no kernel says so
    @kernel(work_shape=WS, group_shape=256)
    def per_group(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[4, DT]):
        atomic_ref(result)[gr.id[0]] += gr.load(a[gr.work_offset[0]:], shape=gr.shape[0]).sum()

    @kernel(work_shape=WS, group_shape=256)
    def not_a_sum(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[4, DT]):
        atomic_ref(result)[0] += gr.load(a[gr.work_offset[0]:], shape=gr.shape[0]).max()

    @kernel(work_shape=WS, group_shape=256)
    def assigned(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[4, DT]):
        atomic_ref(result)[0] = gr.load(a[gr.work_offset[0]:], shape=gr.shape[0]).sum()

    for k in (not_a_sum, assigned):
        with pytest.raises(NoNativeKernel):
            k.plan(a, res4, ctx=ctx)
    # an element per group: the groups' tiles are the rows of a row program with a per-row result
    # (20 elements in tiles of 256: one short row)
    (p,) = per_group.plan(a, res4, ctx=ctx)
    assert p.fn is rt.hcamdLaunchRowProgram and p.args[-2:] == (1, 20)
    # (slot 0: the element's old value, read as a per-row operand; slot 1: the row's sum)
    assert row_stages(p) == [("sum", 1, [("in", 0, 0.0)]), ("store_col", 0, [("red", 0, 0.0), ("add_red", 1, 0.0)])]
    big = FakeDev((1000,), "float32")
    plans = per_group.plan(big, res4, ctx=ctx)
    assert [q.args[-2:] for q in plans] == [(3, 256), (1, 232)]
    assert plans[1].args[4][0] == big.ptr + 3 * 256 * 4 and plans[1].args[11] == res4.ptr + 3 * 4
    with pytest.raises(NoNativeKernel, match="consecutive elements"):
        per_group.plan(FakeDev((2000,), "float32"), res4, ctx=ctx)         # eight groups, four elements
    with pytest.raises(NoNativeKernel, match="float32"):
        reduction_1.plan(a, FakeDev((1,), "float16"), 8, ctx=ctx)


def _pairwise_kernel(deco):
    # body of python/hckernel/tests/test_examples.py:270-292
    M, N, D, GM, GN, MI, NI = sym.M, sym.N, sym.D, sym.GM, sym.GN, sym.MI, sym.NI
    tun = (TunableParam(MI, 1, range(1, 8)), TunableParam(NI, 1, range(1, 8)))

    @deco(work_shape=(cdiv(M, MI), cdiv(N, NI)), group_shape=(GM, GN), tunables=tun)
    def pw_distance(gr: CurrentGroup, a: Buffer[M, D, DT], b: Buffer[N, D, DT],
                    out: Buffer[M, N, DT], gshape: (GM, GN)):
        m_start, n_start = gr.work_offset[0] * MI, gr.work_offset[1] * NI
        m_block, n_block = gr.shape[0] * MI, gr.shape[1] * NI
        a_view = gr.load(a[m_start:, :], shape=(m_block, D))
        b_view = gr.load(b[n_start:, :], shape=(n_block, D))
        diff = a_view[:, None, :] - b_view[None, :, :]
        gr.store(out[m_start:, n_start:], np.linalg.norm(diff, axis=2))
    return pw_distance


def test_pairwise_distance_example_binds_to_the_distance_kernel(ctx):
    k = _pairwise_kernel(kernel)
    a, b, out = FakeDev((16, 8), "float32"), FakeDev((32, 8), "float32"), FakeDev((16, 32), "float32")
    (p,) = k.plan(a, b, out, (8, 8), ctx=ctx)
    assert p.fn is rt.hcamdLaunchPairwiseDistF32
    assert p.args == (ctx.queue, a.ptr, 8, b.ptr, 8, out.ptr, 32, 16, 32, 8)
    (p,) = k.parametrize({sym.MI: 2, sym.NI: 4}).plan(a, b, out, (4, 2), ctx=ctx)
    assert p.args[7:] == (16, 32, 8)
    with pytest.raises(NoNativeKernel, match="float32"):
        k.plan(*(FakeDev(s, "float16") for s in ((16, 8), (32, 8), (16, 32))), (8, 8), ctx=ctx)


def test_tuned_params_round_trip_and_parametrize(tmp_path, ctx):
    from hc_amd.kernel import TunedParams, autotune
    WS, GS, N = sym.WS, sym.GS, sym.N
    t = TunedParams({N: 4, GS: 128}, {"add": 7}, "gfx950", 12.5)
    t.save(tmp_path / "tuned.json")
    back = autotune.load(tmp_path / "tuned.json")
    assert dict(back) == {N: 4, GS: 128} and back.variants == {"add": 7}
    assert back.device == "gfx950" and back.microseconds == 12.5

    @kernel(work_shape=cdiv(WS, N), group_shape=GS,
            tunables=(TunableParam(GS, 64, range(64, 1024, 64)), TunableParam(N, 16, range(16, 256, 16))))
    def reduction(group: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT]):
        temp_result = group.zeros(group.size, dtype=a.dtype)
        for i in range(N):
            work_offset = group.work_offset[0] * N + i * group.size
            temp_result += group.load(a[work_offset:], shape=group.size)
        atomic_ref(result)[0] += temp_result.sum()

    tuned = reduction.parametrize(back)          # the spelling of docs/langref.md:540-550
    assert tuned.tuned == {N: 4, GS: 128} and tuned.variants == {"add": 7}
    (p,) = tuned.plan(FakeDev((5000,), "float32"), FakeDev((1,), "float32"), ctx=ctx)
    assert p.fn is rt.hcamdLaunchMapSum and p.args[8:] == (1, 5000)


# ---------------------------------------------------------------------------
# Mapped loads / stores: products of gathered tiles
# ---------------------------------------------------------------------------
def _conv_kernel(deco, make_mapping, stride):
    """The implicit-GEMM convolution of python/hckernel/tests/test_examples.py:203-252:
    a group owns TN images x TNF filters at one output position; the im2col
    row of an image and the flattened filter are gathered through mappings."""
    N, C, H, W, NF, HF, WF, KB = (sym.N, sym.C, sym.H, sym.W, sym.NF, sym.HF, sym.WF, sym.KB)
    TN, TNF = sym.TN, sym.TNF
    HO = (H - HF) / stride + 1
    WO = (W - WF) / stride + 1
    SZ = HF * WF * C
    KI = cdiv(SZ, KB)
    tun = (TunableParam(TN, 8, range(1, 64)), TunableParam(TNF, 8, range(1, 64)),
           TunableParam(KB, 16, range(8, 128)))
    x_map = make_mapping(lambda i, j: (i, j // (HF * WF), (j % (HF * WF)) % WF,
                                       (j % (HF * WF)) // WF))
    f_map = make_mapping(lambda i, j: (j, i // (HF * WF), i % WF, (i % (HF * WF)) // WF))
    o_map = make_mapping(lambda i, j: (i, j, 0, 0))

    @deco(work_shape=(N, NF, HO * WO), group_shape=(TN, TNF, 1), tunables=tun)
    def conv(gr: CurrentGroup, xs: Buffer[N, C, H, W, DT], fs: Buffer[NF, C, HF, WF, DT],
             out: Buffer[N, NF, HO, WO, DT]):
        i0, o0, idx = gr.work_offset
        p, q = idx % WO, idx // WO
        xv = gr.load(xs[i0:, :, p * stride:, q * stride:], shape=(TN, SZ), mapping=x_map)
        fv = gr.load(fs[o0:, :, :, :], shape=(SZ, TNF), mapping=f_map)
        r = gr.zeros(shape=(xv.shape[0], fv.shape[1]), dtype=out.dtype)
        for k in range(KI):
            r += np.dot(gr.vload(xv[:, k * KB:], shape=(TN, KB)),
                        gr.vload(fv[k * KB:, :], shape=(KB, TNF)))
        gr.store(out[i0:, o0:, p:, q:], r, mapping=o_map)
    return conv


def conv_direct(x, f, stride):
    """Valid cross-correlation, NCHW, square output walk as in the example."""
    n, c, h, w = x.shape
    nf, _, hf, wf = f.shape
    ho, wo = (h - hf) // stride + 1, (w - wf) // stride + 1
    out = np.zeros((n, nf, ho, wo), np.float64)
    for p in range(ho):
        for q in range(wo):
            win = x[:, :, p * stride:p * stride + hf, q * stride:q * stride + wf]
            out[:, :, p, q] = np.einsum("nchw,fchw->nf", win.astype(np.float64),
                                        f.astype(np.float64))
    return out


class TablesOnly:
    """Stands in for hc_amd.runtime.GatherGemm: keeps the host tables."""
    last = None

    def __init__(self, ctx, a, b, out, n_groups, tm, tn, k):
        self.ctx, self.handle = ctx, 0xABCD
        self.ops, self.n_groups, self.tm, self.tn, self.k = (a, b, out), n_groups, tm, tn, k
        self.layouts = [(tuple(o[0]), tuple(o[1])) for o in (a, b, out)]
        TablesOnly.last = self

    def run(self, a, b, out):
        """The meaning of the tables (include/hc_amd_runtime.h, HcamdGatherOperand):
        element (r, c) of a group's tile sits at index rows[r] + cols[c] of the
        window that starts at starts[g]; it is active while every index is
        inside the window.  Products are summed in float64."""
        def tile(op, arr, g, nr, nc):
            shape, _, starts, rows, cols = op
            idx = rows[:nr, None, :] + cols[None, :nc, :]
            ok = ((idx >= 0) & (idx < np.asarray(shape) - starts[g])).all(-1)
            src = np.where(ok[..., None], idx + starts[g], 0)
            vals = arr[tuple(src[..., d] for d in range(len(shape)))]
            return np.where(ok, vals, 0), ok, src

        for g in range(self.n_groups):
            ta, _, _ = tile(self.ops[0], a, g, self.tm, self.k)
            tb, _, _ = tile(self.ops[1], b, g, self.k, self.tn)
            _, ok, dst = tile(self.ops[2], out, g, self.tm, self.tn)
            prod = ta.astype(np.float64) @ tb.astype(np.float64)
            out[tuple(dst[ok][:, d] for d in range(dst.shape[-1]))] = prod[ok]


@pytest.mark.parametrize("n,c,nf,stride,tiles", [
    (1, 1, 1, 1, {}), (2, 3, 2, 2, {}), (4, 3, 8, 3, {}), (3, 2, 5, 1, {sym.TN: 2, sym.TNF: 3}),
    (5, 3, 4, 1, {sym.TN: 4, sym.TNF: 4, sym.KB: 8})])
def test_convolution_example_binds_to_the_gathered_product(ctx, monkeypatch, n, c, nf, stride, tiles):
    from hc_amd.kernel import create_mapping
    from oracle import hcsim
    monkeypatch.setattr(rt, "GatherGemm", TablesOnly)
    rng = np.random.default_rng(5)
    h = w = 4
    hf = wf = 2
    ho, wo = (h - hf) // stride + 1, (w - wf) // stride + 1
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    f = rng.standard_normal((nf, c, hf, wf)).astype(np.float32)

    k = _conv_kernel(kernel, create_mapping, stride).parametrize(tiles)
    dx, df, do = FakeDev(x.shape, "float32"), FakeDev(f.shape, "float32"), \
        FakeDev((n, nf, ho, wo), "float32")
    (p,) = k.plan(dx, df, do, ctx=ctx)
    assert p.fn is rt.hcamdGatherGemmLaunchF32
    t = TablesOnly.last
    assert p.args == (ctx.queue, t.handle, dx.ptr, df.ptr, do.ptr)
    tn, tnf = tiles.get(sym.TN, 8), tiles.get(sym.TNF, 8)

    def merged(extent, count):
        # neighbouring groups are joined while the tile stays within 64 and the count divides
        return extent * max(d for d in range(1, count + 1) if count % d == 0 and d * extent <= 64)
    assert (t.tm, t.tn, t.k) == (merged(tn, cdiv(n, tn)), merged(tnf, cdiv(nf, tnf)), c * hf * wf)
    assert t.n_groups == cdiv(n, t.tm) * cdiv(nf, t.tn) * ho * wo if stride < 3 else True
    got = np.full((n, nf, ho, wo), np.nan, np.float32)
    t.run(x, f, got)

    sim = hcsim.kernel
    want = np.zeros((n, nf, ho, wo), np.float32)
    _conv_kernel(sim, hcsim.create_mapping, stride).parametrize(tiles)(x, f, want)
    assert not np.isnan(got).any()                       # every output was written
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got, conv_direct(x, f, stride), rtol=1e-5, atol=1e-5)


def test_plain_float32_dot_binds_to_the_gathered_product(ctx, monkeypatch):
    monkeypatch.setattr(rt, "GatherGemm", TablesOnly)
    M, N, K, GM, GN, KB = sym.M, sym.N, sym.K, sym.GM, sym.GN, sym.KB
    KI = cdiv(K, KB)

    @kernel(work_shape=(M, N), group_shape=(GM, GN), tunables=TunableParam(KB, 8, (8, 16)))
    def dot(gr: CurrentGroup, a: Buffer[M, K, DT], b: Buffer[K, N, DT], out: Buffer[M, N, DT],
            gshape: (GM, GN)):
        m0, n0 = gr.work_offset
        r = gr.zeros(shape=gr.shape, dtype=out.dtype)
        for k in range(KI):
            r += np.dot(gr.load(a[m0:, k * KB:], shape=(gr.shape[0], KB)),
                        gr.load(b[k * KB:, n0:], shape=(KB, gr.shape[1])))
        gr.store(out[m0:, n0:], r)

    rng = np.random.default_rng(6)
    a = rng.standard_normal((13, 21)).astype(np.float32)
    b = rng.standard_normal((21, 10)).astype(np.float32)
    (p,) = dot.plan(FakeDev(a.shape, "float32"), FakeDev(b.shape, "float32"),
                    FakeDev((13, 10), "float32"), (8, 4), ctx=ctx)
    assert p.fn is rt.hcamdGatherGemmLaunchF32
    t = TablesOnly.last
    # 2 x 3 groups of 8 x 4 are joined into one 16 x 12 tile
    assert (t.n_groups, t.tm, t.tn, t.k) == (1, 16, 12, 24)
    got = np.full((13, 10), np.nan, np.float32)
    t.run(a, b, got)
    np.testing.assert_allclose(got, a.astype(np.float64) @ b.astype(np.float64), rtol=1e-5, atol=1e-5)


def test_mappings_that_no_table_can_express_are_refused(ctx, monkeypatch):
    from hc_amd.kernel import create_mapping
    monkeypatch.setattr(rt, "GatherGemm", TablesOnly)
    M, N, K = sym.M, sym.N, sym.K

    def make(a_func, dtype="float32", store_func=None):
        a_map = create_mapping(a_func)
        o_map = create_mapping(store_func) if store_func else None

        @kernel(work_shape=(M, N), group_shape=(4, 4))
        def body(gr: CurrentGroup, a: Buffer[M, K, DT], b: Buffer[K, N, DT], out: Buffer[M, N, DT]):
            m0, n0 = gr.work_offset
            av = gr.load(a[m0:, :], shape=(4, K), mapping=a_map)
            bv = gr.load(b[:, n0:], shape=(K, 4))
            gr.store(out[m0:, n0:], np.dot(av, bv), mapping=o_map)
        return body.plan(FakeDev((8, 6), dtype), FakeDev((6, 8), dtype), FakeDev((8, 8), dtype),
                         ctx=ctx)

    (p,) = make(lambda i, j: (i, j))
    assert p.fn is rt.hcamdGatherGemmLaunchF32
    (p,) = make(lambda i, j: (i, 5 - j), store_func=lambda i, j: (3 - i, j))   # reversed K, flipped rows
    assert p.fn is rt.hcamdGatherGemmLaunchF32
    with pytest.raises(NoNativeKernel, match="both tile coordinates"):
        make(lambda i, j: (i + j, j))
    with pytest.raises(NoNativeKernel, match="one destination"):
        make(lambda i, j: (i, j), store_func=lambda i, j: (i // 2, j))
    with pytest.raises(NoNativeKernel, match="float32, float16 or bfloat16"):
        make(lambda i, j: (i, j), dtype="int32", store_func=lambda i, j: (i, j))
    for dtype, code in (("float16", rt.F16), ("bfloat16", rt.BF16)):
        (p,) = make(lambda i, j: (i, j), dtype=dtype, store_func=lambda i, j: (i, j))
        assert p.fn is rt.hcamdGatherGemmLaunch and p.args[2] == code
    with pytest.raises(NoNativeKernel, match="must return 2 indices"):
        make(lambda i, j: (i, j, 0))
    with pytest.raises(NoNativeKernel, match="cannot be evaluated"):
        make(lambda i, j: (i, j if j < 3 else 0))


class MapTablesOnly:
    """Stands in for hc_amd.runtime.GatherMap: keeps the host tables and runs
    them in NumPy."""
    last = None

    def __init__(self, ctx, operands, n_groups, tile_elems):
        self.ctx, self.handle = ctx, 0xABCE
        self.operands, self.n_groups, self.tile_elems = operands, n_groups, tile_elems
        self.layouts = [(tuple(o[0]), tuple(o[1])) for o in operands]
        MapTablesOnly.last = self

    def gather(self, k, arr, g):
        """(values, active) of operand k's tile for group g (HcamdGatherMapOperand:
        element e sits at index[e] of the window that starts at starts[g] and is
        active while every index is inside it)."""
        shape, _, starts, index = self.operands[k]
        ok = ((index >= 0) & (index < np.asarray(shape) - starts[g])).all(-1)
        src = np.where(ok[:, None], index + starts[g], 0)
        return np.where(ok, arr[tuple(src[:, d] for d in range(len(shape)))], 0), ok, src


def test_mapped_loads_and_stores_outside_a_product_bind_to_the_gathered_map(ctx, monkeypatch):
    from hc_amd.kernel import create_mapping
    monkeypatch.setattr(rt, "GatherMap", MapTablesOnly)
    R, Cc = sym.R, sym.C
    rows, cols, TM, TN = 19, 21, 4, 8

    def body(load_func=None, store_func=None, fn=lambda t, u: t * np.float32(3) - u, stretch=1):
        lm = create_mapping(load_func) if load_func else None
        sm = create_mapping(store_func) if store_func else None

        @kernel(work_shape=(R, Cc), group_shape=(TM, TN))
        def k(gr: CurrentGroup, a: Buffer[R, Cc, DT], b: Buffer[R, Cc, DT], out: Buffer[sym.RO, sym.CO, DT]):
            x, y = gr.work_offset
            t = gr.load(a[x:, y:], shape=(TM, TN), mapping=lm)
            u = gr.load(b[x:, y:], shape=(TM, TN))
            gr.store(out[stretch * x:, y:], fn(t, u), mapping=sm)
        return k

    def plan(k, dtype="float32", out_shape=(rows, cols)):
        return k.plan(FakeDev((rows, cols), dtype), FakeDev((rows, cols), dtype), FakeDev(out_shape, dtype), ctx=ctx)

    # a gathered expression: the tables say where every tile element comes from
    (p,) = plan(body(load_func=lambda i, j: (i + 1, j - 1)))
    assert p.fn is rt.hcamdGatherMapLaunch
    names = {v: k for k, v in rt.FMAP_OPS.items()}
    prog = [(names[p.args[2][i].op], p.args[2][i].arg, p.args[2][i].imm) for i in range(p.args[3])]
    assert prog == [("in", 0, 0.0), ("const", 0, 3.0), ("mul", 0, 0.0), ("in", 1, 0.0), ("sub", 0, 0.0)]
    t = MapTablesOnly.last
    assert (t.n_groups, t.tile_elems) == (5 * 3, TM * TN)
    rng = np.random.default_rng(0)
    a = rng.standard_normal((rows, cols)).astype(np.float32)
    g = 4                                              # group (1, 1): rows 4.., columns 8..
    vals, ok, src = t.gather(0, a, g)
    assert tuple(t.operands[0][2][g]) == (4, 8)
    assert_eq = np.testing.assert_array_equal
    assert_eq(ok.reshape(TM, TN)[:, 0], False)          # column index -1: outside the window
    assert_eq(vals.reshape(TM, TN)[:, 1:], a[5:9, 8:15])
    # a scattered store past the destination's end is not written: the bounds test is the table's
    (p,) = plan(body(store_func=lambda i, j: (2 * i, j), stretch=2), out_shape=(2 * rows - 1, cols))
    t = MapTablesOnly.last
    _, ok, dst = t.gather(2, np.zeros((2 * rows - 1, cols)), 14)   # the last group: from row 32 of 37
    assert ok.reshape(TM, TN)[:, 0].tolist() == [True, True, True, False]
    # a copy takes any element type
    (p,) = plan(body(load_func=lambda i, j: (i, j), fn=lambda t, u: t), dtype="int32")
    assert p.args[-1] == 4 and p.args[3] == 0
    # what has no native code says why
    with pytest.raises(NoNativeKernel, match="stored to one place"):
        plan(body(store_func=lambda i, j: (i // 2, j)))
    with pytest.raises(NoNativeKernel, match="float32 / float16"):
        plan(body(load_func=lambda i, j: (i, j)), dtype="int32")
    with pytest.raises(NoNativeKernel, match="must return 2 indices"):
        plan(body(load_func=lambda i, j: (i, j, 0)))
    with pytest.raises(NoNativeKernel, match="cannot be evaluated"):
        plan(body(load_func=lambda i, j: (i, j if j < 3 else 0)))


def run_gathered_plan(p, tables, host_of, out):
    """A gathered-map plan in NumPy: operands gathered by the host tables
    (host_of: device address -> host array), the program on (value, active)
    pairs (the operations these tests use), active elements inside the
    destination stored."""
    names = {v: k for k, v in rt.FMAP_OPS.items()}
    prog = [(names[p.args[2][i].op], p.args[2][i].arg, p.args[2][i].imm) for i in range(p.args[3])]
    arrays = [host_of[p.args[4][i]] for i in range(len(tables.operands) - 1)]
    for g in range(tables.n_groups):
        stack = []
        for op, arg, imm in prog:
            if op == "in":
                v, ok, _ = tables.gather(arg, arrays[arg], g)
                stack.append((v.astype(np.float32), ok))
            elif op == "const":
                stack.append((np.full(tables.tile_elems, imm, np.float32), np.ones(tables.tile_elems, bool)))
            else:
                (b, bok), (a, aok) = stack.pop(), stack.pop()
                with np.errstate(all="ignore"):
                    v = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op]
                ok = aok & bok
                if op == "div":
                    ok &= (b != 0) & np.isfinite(v)
                stack.append((v.astype(np.float32), ok))
        (v, ok), = stack
        _, inside, dst = tables.gather(len(arrays), out, g)
        keep = ok & inside
        out[tuple(dst[keep, d] for d in range(out.ndim))] = v[keep]


def test_loads_that_do_not_walk_the_window_of_the_store_become_gathered_operands(ctx, monkeypatch):
    """Windows shifted by a constant, row and column vectors broadcast over a
    2-D tile, transposed, sliced and reshaped tiles: no kernel that walks one
    window takes them; the binder derives an index table per load and hands the
    expression to the gathered map.  The tables, run in NumPy, give what the
    simulator gives."""
    from oracle.hcsim import kernel as sim_kernel
    monkeypatch.setattr(rt, "GatherMap", MapTablesOnly)
    M, N = sym.M, sym.N
    f = np.float32

    def bodies(deco):
        @deco(work_shape=N, group_shape=16)
        def shifted(gr: CurrentGroup, x: Buffer[N, DT], out: Buffer[N, DT]):
            o = gr.work_offset[0]
            gr.store(out[o:], gr.load(x[o + 1:], shape=gr.shape) - gr.load(x[o:], shape=gr.shape))

        @deco(work_shape=(M, N), group_shape=(4, 8))
        def broadcast(gr: CurrentGroup, x: Buffer[M, N, DT], b: Buffer[N, DT], s: Buffer[M, DT], out: Buffer[M, N, DT]):
            i, j = gr.work_offset
            t = gr.load(x[i:, j:], shape=gr.shape)
            gr.store(out[i:, j:], (t + gr.load(b[j:], shape=gr.shape[1])) / gr.load(s[i:], shape=gr.shape[0])[:, None])

        @deco(work_shape=(M, N), group_shape=(4, 8))
        def transposed(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[N, M, DT], out: Buffer[N, M, DT]):
            i, j = gr.work_offset
            t = gr.load(x[i:, j:], shape=gr.shape)
            gr.store(out[j:, i:], gr.load(y[j:, i:], shape=gr.shape[::-1]) * t.T)

        @deco(work_shape=(M, N), group_shape=(4, 8))
        def sliced(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT]):
            i, j = gr.work_offset
            wide = gr.load(x[i:, j:], shape=(5, 9))
            gr.store(out[i:, j:], wide[1:, 1:] - wide[:-1, :-1].reshape(32).reshape(4, 8))
        return {"shifted": shifted, "broadcast": broadcast, "transposed": transposed, "sliced": sliced}

    rng = np.random.default_rng(5)
    rows, cols = 11, 21
    x = rng.integers(-5, 6, (rows, cols)).astype(f)
    y = rng.integers(-5, 6, (cols, rows)).astype(f)
    b = rng.integers(-5, 6, cols).astype(f)
    sc = rng.integers(-1, 2, rows).astype(f)                 # zeros: rows whose quotients are deactivated
    cases = {"shifted": ([x.reshape(-1)], (rows * cols,)), "broadcast": ([x, b, sc], (rows, cols)),
             "transposed": ([x, y], (cols, rows)), "sliced": ([x], (rows, cols))}
    gpu, sim = bodies(kernel), bodies(sim_kernel)
    for name, (ins, shape) in cases.items():
        want = np.full(shape, 77, f)
        with np.errstate(all="ignore"):
            sim[name](*ins, want)
        fake = [FakeDev(v.shape, "float32") for v in ins]
        (p,) = gpu[name].plan(*fake, FakeDev(shape, "float32"), ctx=ctx)
        if name == "broadcast":
            # a row vector and a per-row operand next to a tile: one store stage of a row
            # program over the whole window, whatever the groups' tiling
            assert p.fn is rt.hcamdLaunchRowProgram and p.args[-2:] == (rows, cols)
            assert (p.args[7], p.args[10]) == (2, 1)          # the tile and the vector; one per-row operand
            got = run_row_stages(row_stages(p), [x, b], [sc], f, init=np.full(shape, 77, f))
        else:
            assert p.fn is rt.hcamdGatherMapLaunch, name
            got = np.full(shape, 77, f)
            run_gathered_plan(p, MapTablesOnly.last, {d.ptr: v for d, v in zip(fake, ins)}, got)
        np.testing.assert_array_equal(got, want, err_msg=name)
        assert (want == 77).any() or name == "transposed", name
    # the shifted window is a window start, the broadcast vector a table that ignores a dimension
    (p,) = gpu["shifted"].plan(FakeDev((200,), "float32"), FakeDev((200,), "float32"), ctx=ctx)
    t = MapTablesOnly.last
    assert t.operands[0][2][:3, 0].tolist() == [1, 17, 33] and t.operands[1][2][:3, 0].tolist() == [0, 16, 32]
    # (a vector that the row program cannot take, here one shorter than the tiles are wide, stays gathered)
    @kernel(work_shape=(M, N), group_shape=(4, 8))
    def short_vector(gr: CurrentGroup, x: Buffer[M, N, DT], b: Buffer[sym.NB, DT], s: Buffer[M, DT], out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        t = gr.load(x[i:, j:], shape=gr.shape)
        gr.store(out[i:, j:], (t + gr.load(b[j:], shape=gr.shape[1])) * gr.load(s[i:], shape=gr.shape[0])[:, None])
    (p,) = short_vector.plan(FakeDev((12, 21), "float32"), FakeDev((19,), "float32"), FakeDev((12,), "float32"),
                             FakeDev((12, 21), "float32"), ctx=ctx)
    assert p.fn is rt.hcamdGatherMapLaunch
    t = MapTablesOnly.last
    assert t.operands[1][3][:, 0].tolist() == list(range(8)) * 4         # the row vector: the column index
    assert t.operands[2][3][:, 0].tolist() == [r for r in range(4) for _ in range(8)]
    # a bare array (a transposed tile is one) is stored in full: refused where that would write what the
    # reference initialises tiles with
    T2 = sym.T2

    @kernel(work_shape=(M, N), group_shape=(4, 8))
    def wider(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[T2, T2, DT]):
        i, j = gr.work_offset
        gr.store(out[j:, i:], gr.load(x[i:, j:], shape=gr.shape).T)
    with pytest.raises(NoNativeKernel, match="written in full"):
        wider.plan(FakeDev((11, 21), "float32"), FakeDev((24, 24), "float32"), ctx=ctx)
    # other element types: copies only
    @kernel(work_shape=(M, N), group_shape=(4, 8))
    def int_transpose(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[N, M, DT]):
        i, j = gr.work_offset
        gr.store(out[j:, i:], gr.load(x[i:, j:], shape=gr.shape).T)
    # a tile's .T alone, stored to the transposed window, is one transposed copy of the whole window
    (p,) = int_transpose.plan(FakeDev((11, 21), "int32"), FakeDev((21, 11), "int32"), ctx=ctx)
    assert p.fn is rt.hcamdLaunchTranspose2D and p.args[1] == 4 and p.args[-2:] == (11, 21)
    (p,) = int_transpose.plan(FakeDev((11, 21), "int8", ld=32), FakeDev((21, 11), "int8", ld=16), ctx=ctx)
    assert p.args[1] == 1 and p.args[-2:] == (11, 21) and (p.args[3], p.args[5]) == (32, 16)
    @kernel(work_shape=(M, N), group_shape=(4, 8))
    def wider_transpose(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[N, T2, DT]):
        i, j = gr.work_offset
        gr.store(out[j:, i:], gr.load(x[i:, j:], shape=gr.shape).T)
    with pytest.raises(NoNativeKernel, match="written in full"):
        wider_transpose.plan(FakeDev((11, 21), "int32"), FakeDev((21, 12), "int32"), ctx=ctx)


def test_offsets_with_division_are_for_mapped_accesses_only(ctx):
    W, H = sym.W, sym.H

    @kernel(work_shape=(W, H), group_shape=(4, 4))
    def body(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x, y = gr.work_offset
        gr.store(dst[x:, y:], gr.load(src[x // 2:, y:], shape=gr.shape))

    with pytest.raises(NoNativeKernel, match="mapped loads and stores only"):
        body.plan(FakeDev((8, 8), "float32"), FakeDev((8, 8), "float32"), ctx=ctx)


def test_groups_are_joined_only_when_that_is_exact(ctx, monkeypatch):
    """Row index -1 of a tile is inactive in its own window but would be the last
    row of the window before it: such tables keep the user's tiling."""
    from hc_amd.kernel import create_mapping
    monkeypatch.setattr(rt, "GatherGemm", TablesOnly)
    M, N, K = sym.M, sym.N, sym.K
    shifted = create_mapping(lambda i, j: (i - 1, j))

    @kernel(work_shape=(M, N), group_shape=(4, 4))
    def body(gr: CurrentGroup, a: Buffer[M, K, DT], b: Buffer[K, N, DT], out: Buffer[M, N, DT]):
        m0, n0 = gr.work_offset
        av = gr.load(a[m0:, :], shape=(4, K), mapping=shifted)
        bv = gr.load(b[:, n0:], shape=(K, 4))
        gr.store(out[m0:, n0:], np.dot(av, bv))

    rng = np.random.default_rng(3)
    a = rng.standard_normal((8, 6)).astype(np.float32)
    b = rng.standard_normal((6, 8)).astype(np.float32)
    body.plan(FakeDev((8, 6), "float32"), FakeDev((6, 8), "float32"), FakeDev((8, 8), "float32"),
              ctx=ctx)
    t = TablesOnly.last
    assert (t.tm, t.tn, t.n_groups) == (4, 8, 2)      # columns joined, rows not
    got = np.full((8, 8), np.nan, np.float32)
    t.run(a, b, got)
    want = np.zeros((8, 8))
    want[1:4], want[5:8] = a[0:3] @ b, a[4:7] @ b     # row 0 of each group reads nothing
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------------------
# Row programs: elementwise arithmetic mixed with reductions along the rows
# ---------------------------------------------------------------------------
def row_stages(plan):
    """[(kind, slot, [(opname, arg, imm)])] of a hcamdLaunchRowProgram plan."""
    assert plan.fn is rt.hcamdLaunchRowProgram
    names = {v: k for k, v in rt.MAP_OPS.items()}
    kinds = {v: k for k, v in rt.ROW_KINDS.items()}
    prog, st, n = plan.args[1], plan.args[2], plan.args[3]
    out, pc = [], 0
    for i in range(n):
        out.append((kinds[st[i].kind], st[i].dst,
                    [(names[prog[j].op], prog[j].arg, prog[j].imm)
                     for j in range(pc, pc + st[i].nInstr)]))
        pc += st[i].nInstr
    return out


def run_row_stages(stages, inputs, columns=(), out_dtype=np.float32, init=None):
    """What hcamdLaunchRowProgram computes, in NumPy fp32 (reductions with
    NumPy's own summation order): enough to check on the CPU that the stages
    the front-end emits mean what the kernel body says.  Elements carry an
    "inactive" flag per stage, row scalars a "deactivated" flag, as in the
    kernel; `init` is what the output holds before (elements that are not
    stored keep it)."""
    f = np.float32
    rows = next(x.shape[0] for x in inputs if x.ndim == 2)
    n = next(x.shape[1] for x in inputs if x.ndim == 2)
    red = {k: (c.astype(f).reshape(rows, 1), np.zeros((rows, 1), bool)) for k, c in enumerate(columns)}
    FUNC, SWAPPED, KEEP_DEAD = 0x200, 0x400, 0x800
    plain = {"add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b,
             "div": lambda a, b: a / b, "max": np.maximum, "min": np.minimum}
    unary = {"neg": np.negative, "abs": np.abs, "sqrt": np.sqrt, "rint": np.rint, "exp": np.exp,
             "log": np.log, "tanh": np.tanh, "r16": lambda a: a.astype(np.float16).astype(f)}

    def r16(q, half):
        return q.astype(np.float16).astype(f) if half else q

    def quotient(a, b, half):
        """numpy.ma's division: (value, failed)."""
        q = r16((a / b).astype(f), half)
        good = np.isfinite(q)
        return np.where(good, q + f(0) * a, f(0) + a).astype(f), ~good

    def domain(name, x):
        """(value, failed) of the functions that can deactivate."""
        if name == "msqrt":
            out = x < 0
            return np.where(out, f(0), np.sqrt(np.where(out, f(0), x))).astype(f), out
        if name == "mlog":
            out = x <= 0
            return np.where(out, f(1), np.log(np.where(out, f(1), x))).astype(f), out
        if name == "masqrt":
            y = np.sqrt(x)
            out = ~np.isfinite(y) | (x < 0)
            return np.where(out, x, y).astype(f), out
        assert name == "powchk"
        out = ~np.isfinite(x)
        return np.where(out, f(1e20), x).astype(f), out

    def split(name):
        """(operation, form) of an in-place instruction: form i, _in, _red."""
        for form in ("_in", "_red"):
            if name.endswith(form):
                return name[:-len(form)], form
        assert name.endswith("i"), name
        return name[:-1], "i"

    result = None if init is None else init.copy()
    if result is None:
        result = np.zeros((rows, n) if stages[-1][0] == "store" else rows, out_dtype)
    with np.errstate(all="ignore"):
        for kind, dst, program in stages:
            scalar_stage = kind in ("scalar", "store_col")
            stack = []                    # values; scalar stages: (value, dead)
            bad = np.zeros((rows, n), bool)
            live_slot = None
            # a frozen stage keeps what numpy.ma leaves in deactivated elements
            # (one running value; the instructions carry the form flags)
            frozen = program[-1][0] == "frozen"
            for name, arg, imm in program:
                if name == "livepos":
                    live_slot = arg & 0xff
                    continue
                if name == "frozen":
                    bad[:] = False
                    continue
                if scalar_stage:
                    half, func, swapped = bool(arg & 0x100), bool(arg & FUNC), bool(arg & SWAPPED)
                    never = np.zeros((rows, 1), bool)
                    if name in ("red", "red0"):
                        v, d = red[arg & 0xff]
                        stack.append((v, never if name == "red0" else d))
                        continue
                    if name == "const":
                        stack.append((np.full((rows, 1), imm, f), never))
                        continue
                    if name in unary:
                        v, d = stack.pop()
                        keep = d if arg & KEEP_DEAD else never     # x ** 0.5 keeps a deactivated operand
                        stack.append((np.where(keep, v, unary[name](v)).astype(f), d))
                        continue
                    if name in ("msqrt", "mlog", "masqrt", "powchk"):
                        v, d = stack.pop()
                        if name in ("msqrt", "mlog"):
                            # numpy.sqrt / numpy.log of a deactivated value: the fill value too
                            v = np.where(d, f(-1), v)
                        v, failed = domain(name, v)
                        stack.append((v, d | failed))
                        continue
                    if name in ("add", "sub", "mul", "div", "max", "min", "rsub", "rdiv", "mdiv", "rmdiv"):
                        right, left = stack.pop(), stack.pop()
                        op = name
                    else:
                        op, form = split(name)
                        running = stack.pop()
                        other = (np.full((rows, 1), imm, f), never) if form == "i" else red[arg & 0xff]
                        left, right = running, other
                    if op.startswith("r"):        # rsub, rdiv, rmdiv: the other operand comes first
                        op, left, right = op[1:], right, left
                    elif swapped:
                        left, right = right, left
                    dead = left[1] | right[1]
                    if op == "mdiv":
                        v, failed = quotient(left[0], right[0], half or (name in ("mdiv", "rmdiv") and arg & 1))
                        v = np.where(dead, f(0) + left[0], v)
                        dead = dead | failed
                    else:
                        v = plain[op](left[0], right[0]).astype(f)
                        if not func and op in ("add", "sub", "mul"):
                            v = np.where(dead, left[0], v)      # numpy.ma keeps the first operand's value
                    stack.append((v.astype(f), dead))
                    continue
                # element-wise stages
                half = bool(arg & 0x100)
                if name == "in":
                    stack.append(np.broadcast_to(inputs[arg].astype(f), (rows, n)))
                elif name == "red":
                    stack.append(np.broadcast_to(red[arg][0], (rows, n)))
                    bad |= red[arg][1]
                elif name == "const":
                    stack.append(np.full((rows, n), imm, f))
                elif name == "clear":
                    bad[:] = False
                elif name in unary:
                    x = stack.pop()
                    y = unary[name](x).astype(f)
                    stack.append(np.where(bad, x, y) if frozen and arg & KEEP_DEAD else y)
                elif name in ("msqrt", "mlog", "powchk"):
                    x = stack.pop()
                    if frozen and name != "powchk":
                        x = np.where(bad, f(-1), x)       # deactivated already: the fill value too
                    v, failed = domain(name, x)
                    stack.append(v)
                    bad |= failed
                elif name in ("add", "sub", "mul", "div", "max", "min", "rsub", "rdiv", "mdiv", "rmdiv"):
                    b = stack.pop()
                    a = stack.pop()
                    if name.startswith("r"):
                        name, a, b = name[1:], b, a
                    if name == "mdiv":
                        v, failed = quotient(a, b, arg != 0)
                        bad |= failed
                    else:
                        v = plain[name](a, b).astype(f)
                    stack.append(v)
                else:
                    op, form = split(name)
                    a = stack.pop()
                    if form == "i":
                        b = np.full((rows, n), imm, f)
                    elif form == "_red":
                        b = np.broadcast_to(red[arg & 0xf][0], (rows, n))
                        bad = bad | red[arg & 0xf][1]
                    else:
                        b = np.broadcast_to(inputs[arg & 0x3].astype(f), (rows, n))
                    if op.startswith("r"):
                        op, a, b = op[1:], b, a
                    elif frozen and arg & SWAPPED:
                        a, b = b, a
                    if op == "mdiv":
                        v, failed = quotient(a, b, half)
                        if frozen:
                            v = np.where(bad, f(0) + a, v)
                        bad = bad | failed
                    else:
                        v = plain[op](a, b).astype(f)
                        if frozen and not arg & FUNC and op in ("add", "sub", "mul"):
                            v = np.where(bad, a, v)           # numpy.ma keeps the first operand's value
                    stack.append(v)
            (top,) = stack
            if scalar_stage:
                v, dead = top
                v, dead = np.broadcast_to(v, (rows, 1)).astype(f), np.broadcast_to(dead, (rows, 1)).copy()
                if live_slot is not None:
                    dead = ~(red[live_slot][0] > 0)
                if kind == "scalar":
                    red[dst] = (v, dead)
                elif dst == 1 and result is not None:      # a tile: deactivated rows are not stored
                    result = np.where(dead.reshape(rows), result, v.reshape(rows).astype(out_dtype))
                else:
                    result = v.reshape(rows).astype(out_dtype)
                continue
            top = np.broadcast_to(np.asarray(top, f), (rows, n))
            if kind == "store":
                result = np.where(bad, result, top.astype(out_dtype))
                continue
            count = (~bad).sum(axis=1, keepdims=True)
            if kind == "count":
                red[dst] = (count.astype(f), np.zeros((rows, 1), bool))
            elif kind == "sum":
                red[dst] = (np.where(bad, f(0), top).sum(axis=1, keepdims=True).astype(f), count == 0)
            else:
                fill = f(-np.inf) if kind == "max" else f(np.inf)
                folded = getattr(np.where(bad, fill, top), kind)(axis=1, keepdims=True).astype(f)
                red[dst] = (np.where(count == 0, f(1e20), folded), count == 0)
    return result


def _row_bodies(deco):
    """Kernel bodies with reductions along rows, written against the reference's
    API; `deco` is hc_amd's kernel or the CPU simulator's."""
    M, N, GM = sym.M, sym.N, sym.GM
    f = np.float32

    @deco(work_shape=M, group_shape=GM)
    def layernorm(gr: CurrentGroup, x: Buffer[M, N, DT], g: Buffer[N, DT], b: Buffer[N, DT],
                  out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        w, bias = gr.load(g[:], shape=(N,)), gr.load(b[:], shape=(N,))
        mean = t.mean(axis=1, keepdims=True)
        var = t.var(axis=1, keepdims=True)
        gr.store(out[m0:, :], (t - mean) / np.sqrt(var + f(1e-5)) * w + bias)

    @deco(work_shape=M, group_shape=GM)
    def rmsnorm_half(gr: CurrentGroup, x: Buffer[M, N, DT], g: Buffer[N, DT],
                     out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N)).astype(f)
        ms = np.mean(np.square(t), axis=1, keepdims=True)
        gr.store(out[m0:, :], (t / np.sqrt(ms + f(1e-6)) * gr.load(g[:], shape=(N,))).astype(np.float16))

    @deco(work_shape=M, group_shape=GM)
    def log_softmax_t(gr: CurrentGroup, x: Buffer[M, N, DT], temp: Buffer[M, DT],
                      out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        s = gr.load(temp[m0:], shape=(mb,))
        z = (t - t.max(axis=1, keepdims=True)) * s[:, None]
        gr.store(out[m0:, :], z - np.log(np.exp(z).sum(axis=1, keepdims=True)))

    @deco(work_shape=M, group_shape=GM)
    def row_norms(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        gr.store(out[m0:], np.sqrt((t * t).sum(axis=1)))

    @deco(work_shape=M, group_shape=GM)
    def spread(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        lo, hi = t.min(axis=1), np.max(t, axis=1)
        gr.store(out[m0:, :], (t - lo[:, None]) / (hi - lo)[:, None])

    @deco(work_shape=M, group_shape=GM)
    def unit_rows(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        gr.store(out[m0:, :], t / np.linalg.norm(t, axis=1, keepdims=True))

    @deco(work_shape=M, group_shape=GM)
    def log_sum_exp(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        top = t.max(axis=1)
        gr.store(out[m0:], top + np.log(np.exp(t - top[:, None]).sum(axis=-1)))

    return {"layernorm": layernorm, "rmsnorm_half": rmsnorm_half, "log_softmax_t": log_softmax_t,
            "row_norms": row_norms, "spread": spread, "unit_rows": unit_rows,
            "log_sum_exp": log_sum_exp}


def _row_case(name, rows, n, seed=0):
    """Host operands of a body, in argument order, the last one the output."""
    rng = np.random.default_rng(seed)
    f = np.float32
    x = (rng.standard_normal((rows, n)) * 2 + 0.25).astype(f)
    if name == "layernorm":
        return [x, rng.standard_normal(n).astype(f), rng.standard_normal(n).astype(f),
                np.zeros((rows, n), f)]
    if name == "rmsnorm_half":
        return [x.astype(np.float16), rng.standard_normal(n).astype(f), np.zeros((rows, n), np.float16)]
    if name == "log_softmax_t":
        return [x, rng.uniform(0.5, 2.0, rows).astype(f), np.zeros((rows, n), f)]
    if name in ("row_norms", "log_sum_exp"):
        return [x, np.zeros(rows, f)]
    return [x, np.zeros((rows, n), f)]


def test_bodies_with_row_reductions_compile_to_row_programs(ctx):
    from oracle.hcsim import kernel as sim_kernel
    rows, n = 37, 200
    gpu, sim = _row_bodies(kernel), _row_bodies(sim_kernel)
    want_stages = {
        # sum(x) is computed once for the mean and the variance
        # (the mean, the variance and the scale are a row scalar each)
        "layernorm": ["sum", "scalar", "sum", "scalar", "scalar", "store"],
        "rmsnorm_half": ["sum", "scalar", "store"],
        "log_softmax_t": ["max", "sum", "scalar", "store"],
        "row_norms": ["sum", "store_col"],
        "spread": ["min", "max", "scalar", "store"],
        "unit_rows": ["sum", "scalar", "store"],
        "log_sum_exp": ["max", "sum", "store_col"],
    }
    for name, body in gpu.items():
        host = _row_case(name, rows, n)
        fake = [FakeDev(a.shape, a.dtype.name) for a in host]
        (p,) = body.plan(*fake, 8, ctx=ctx)
        stages = row_stages(p)
        assert [k for k, _, _ in stages] == want_stages[name], (name, stages)
        assert p.args[-2:] == (rows, n)
        n_in, n_col = p.args[7], p.args[10]
        # the stages mean what the body says: run them in NumPy, run the body
        # on the simulator
        tiles = [a for a in host[:-1] if not (a.ndim == 1 and a.shape[0] == rows)]
        cols = [a for a in host[:-1] if a.ndim == 1 and a.shape[0] == rows]
        assert (n_in, n_col) == (len(tiles), len(cols)), name
        got = run_row_stages(stages, tiles, cols, host[-1].dtype)
        want = host[-1].copy()
        sim[name](*host[:-1], want, 8)
        if host[-1].dtype == np.float16:
            np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3)
        else:
            np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6, err_msg=name)
    # details of one program: the row scalars are read by the operations themselves
    (p,) = gpu["layernorm"].plan(*[FakeDev(a.shape, a.dtype.name)
                                   for a in _row_case("layernorm", rows, n)], 8, ctx=ctx)
    st = row_stages(p)
    assert [i[0] for i in st[-1][2]] == ["in", "sub_red", "mdiv_red", "mul_in", "add_in"]   # the tile operator /: numpy.ma's rule
    assert st[1][2] == [("red", 0, 0.0), ("mdivi", 0, float(n))]              # numpy.ma's division
    assert st[3][2] == [("red0", 2, 0.0), ("divi", 0, float(n))]             # the variance: active whatever it is
    assert list(p.args[6][:3]) == [n, 0, 0]                 # tile, then two vectors (stride 0)


POISON = np.float32(-77.0)


def _masked_row_bodies(deco):
    """Bodies whose reductions along rows run over elements that the data can
    deactivate (a zero divisor), or whose row scalars can be deactivated
    themselves (a division of two sums, a root of a negative sum, a mean that is
    not finite): numpy.ma's rules decide what is folded, what is stored and what a
    deactivated per-row result holds (python/hckernel/kernel_api.py:150-180 forwards
    all of it to numpy.ma).  name -> (kernel, result is one value per row)."""
    M, N, GM = sym.M, sym.N, sym.GM
    f = np.float32

    def tile_body(fn):
        @deco(work_shape=M, group_shape=GM)
        def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, N, DT], g: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            ta, tb = gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N))
            gr.store(out[m0:, :], fn(ta, tb))
        return k

    def row_body(fn):
        @deco(work_shape=M, group_shape=GM)
        def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, DT], g: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            ta, tb = gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N))
            gr.store(out[m0:], fn(ta, tb))
        return k

    def zscore(ta, tb):
        q = ta / tb
        return (q - q.mean(axis=1, keepdims=True)) / q.std(axis=1, keepdims=True, ddof=1)

    def layernorm(ta, tb):
        return (ta - ta.mean(axis=1, keepdims=True)) / np.sqrt(ta.var(axis=1, keepdims=True) + f(1e-5)) * tb

    tiles = {
        "ratio": lambda ta, tb: ta * (ta.sum(axis=1, keepdims=True) / tb.sum(axis=1, keepdims=True)),
        "centre": lambda ta, tb: (ta / tb) - (ta / tb).mean(axis=1, keepdims=True),
        "divsqrt": lambda ta, tb: ta / np.sqrt(tb.sum(axis=1, keepdims=True)),
        "mullog": lambda ta, tb: ta * np.log(tb.sum(axis=1, keepdims=True)),
        "xvar": lambda ta, tb: tb * ta.var(axis=1, keepdims=True),
        "xstd": lambda ta, tb: tb * ta.std(axis=1, keepdims=True),
        "xmaskedvar": lambda ta, tb: tb * (ta / tb).var(axis=1, keepdims=True, ddof=2),
        "rms": lambda ta, tb: ta / np.sqrt(np.mean(np.square(ta), axis=1, keepdims=True) + f(1e-6)) * tb,
        "layernorm": layernorm,
        "zscore": zscore,
        "square_of_sum": lambda ta, tb: ta * (tb * f(1e10)).sum(axis=1, keepdims=True) ** 2,
        "over_max": lambda ta, tb: ta / (ta / tb).max(axis=1, keepdims=True),
        # tile.astype gives a bare numpy.ma array: what is computed from it is stored in
        # full, deactivated elements with what numpy.ma leaves in them
        "bare_scaled_quotient": lambda ta, tb: (ta.astype(f) / tb.astype(f)) * f(3) - f(1),
        "bare_rms": lambda ta, tb: ta.astype(f) / np.sqrt(np.mean(np.square(ta.astype(f)), axis=1, keepdims=True)
                                                          + f(1e-6)) * tb.astype(f),
        "bare_centre_over_sum": lambda ta, tb: (ta.astype(f) - ta.astype(f).mean(axis=1, keepdims=True)) /
        tb.astype(f).sum(axis=1, keepdims=True),
        "bare_one_minus_quotient": lambda ta, tb: f(1) - ta.astype(f) / tb.astype(f),
        "bare_python_one_minus_quotient": lambda ta, tb: 1.0 - ta.astype(f) / tb.astype(f),
        "bare_sqrt_of_quotient": lambda ta, tb: np.sqrt(ta.astype(f) / tb.astype(f)) + f(2),
        "bare_quotient_over_row_sum": lambda ta, tb: tb.astype(f) / ta.astype(f).sum(axis=1, keepdims=True) * ta,
    }
    rows = {
        "mean": lambda ta, tb: (ta / tb).mean(axis=1),
        "sum": lambda ta, tb: (ta / tb).sum(axis=1),
        "max": lambda ta, tb: (ta / tb).max(axis=1),
        "min": lambda ta, tb: (ta / tb).min(axis=1),
        "var": lambda ta, tb: (ta / tb).var(axis=1),
        "std1": lambda ta, tb: (ta / tb).std(axis=1, ddof=1),
        "plain_mean": lambda ta, tb: ta.mean(axis=1),
        "plain_var": lambda ta, tb: ta.var(axis=1),
        "plain_std": lambda ta, tb: ta.std(axis=1),
        "sqrt_sum": lambda ta, tb: np.sqrt(tb.sum(axis=1)),
        "sum_ratio": lambda ta, tb: ta.sum(axis=1) / tb.sum(axis=1),
        "one_plus_ratio": lambda ta, tb: f(1) + ta.sum(axis=1) / tb.sum(axis=1),
        "ratio_times_two": lambda ta, tb: ta.sum(axis=1) / tb.sum(axis=1) * f(2),
        "python_one_plus_ratio": lambda ta, tb: 1.0 + ta.sum(axis=1) / tb.sum(axis=1),
        "two_ratios": lambda ta, tb: (ta.sum(axis=1) / tb.sum(axis=1) + f(1)) * (tb.max(axis=1) / ta.sum(axis=1) - f(2)),
        "neg_sqrt_ratio": lambda ta, tb: -np.sqrt(ta.sum(axis=1) / tb.sum(axis=1)),
        "max_plus_log": lambda ta, tb: ta.max(axis=1) + np.log(tb.sum(axis=1)),
        "log_plus_max": lambda ta, tb: np.log(tb.sum(axis=1)) + ta.max(axis=1),
        "exp_of_mean": lambda ta, tb: np.exp((ta / tb).mean(axis=1)),
        "masked_mean_of_squares": lambda ta, tb: ((ta / tb) ** 2).mean(axis=1),
    }
    out = {name: (tile_body(fn), False) for name, fn in tiles.items()}
    out.update({name: (row_body(fn), True) for name, fn in rows.items()})
    return out


def _masked_row_case(rows, n, seed=0):
    """a, b: b has zeros here and there, a row of zeros, a row that adds up to
    zero and one with a negative sum; a has a row with an inf and one with a NaN."""
    rng = np.random.default_rng(seed)
    f = np.float32
    a = rng.standard_normal((rows, n)).astype(f)
    b = (rng.standard_normal((rows, n)) + 0.3).astype(f)
    b[rng.random((rows, n)) < 0.08] = 0
    b[1 % rows, :] = 0
    if rows > 4 and n >= 2:
        b[4, :] = 0
        b[4, 0], b[4, 1] = 1.5, -1.5
        b[2, :] = -np.abs(b[2, :]) - f(0.1)
    if rows > 5:
        a[5, n // 2] = np.inf
    if rows > 6:
        a[6, 0] = np.nan
    return a, b


@pytest.mark.parametrize("rows,n", [(8, 5), (37, 200)])
def test_reductions_over_deactivated_elements_follow_numpy_ma(ctx, rows, n):
    """The stages the front-end emits, run in NumPy with the kernel's rules, give
    what the simulator gives: the same values, the same elements left alone."""
    from oracle.hcsim import kernel as sim_kernel
    gpu, sim = _masked_row_bodies(kernel), _masked_row_bodies(sim_kernel)
    a, b = _masked_row_case(rows, n, seed=rows)
    for name, (body, per_row) in gpu.items():
        shape = (rows,) if per_row else (rows, n)
        want = np.full(shape, POISON)
        with np.errstate(all="ignore"):
            sim[name][0](a, b, want, 8)
        fake = [FakeDev(a.shape, "float32"), FakeDev(b.shape, "float32"), FakeDev(shape, "float32")]
        (p,) = body.plan(*fake, 8, ctx=ctx)
        if p.fn is not rt.hcamdLaunchRowProgram:
            # no reduction in the body: the fast map where the values flow plainly, else the
            # general float map, which tracks activity per operand (their parity is a GPU test)
            assert p.fn in (rt.hcamdLaunchFMap, rt.hcamdLaunchMap) and name in (
                "bare_scaled_quotient", "bare_one_minus_quotient", "bare_python_one_minus_quotient",
                "bare_sqrt_of_quotient"), name
            continue
        by_ptr = {fake[0].ptr: a, fake[1].ptr: b}
        operands = [by_ptr[p.args[4][i]] for i in range(p.args[7])]      # in the order of first use
        with np.errstate(all="ignore"):
            got = run_row_stages(row_stages(p), operands, (), np.float32, init=np.full(shape, POISON))
        np.testing.assert_array_equal(got == POISON, want == POISON, err_msg=name)
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want), err_msg=name)
        np.testing.assert_allclose(got, want, rtol=3e-5, atol=1e-6, err_msg=name)


def test_what_a_traced_tile_cannot_give_says_why(ctx):
    N = sym.N

    def body(fn, out_dtype):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, DT]):
            o = gr.work_offset[0]
            gr.store(out[o:], fn(gr.load(a[o:], shape=gr.shape), gr.load(b[o:], shape=gr.shape)))
        return k

    f32, i32 = FakeDev((1000,), "float32"), FakeDev((1000,), "int32")
    with pytest.raises(NoNativeKernel, match="length depends on the data"):
        body(lambda a, b: (a / b).compressed(), "float32").plan(f32, f32, FakeDev((1000,), "float32"), ctx=ctx)
    with pytest.raises(NoNativeKernel, match="float64 in NumPy"):
        body(lambda a, b: a / b, "float32").plan(i32, i32, FakeDev((1000,), "float32"), ctx=ctx)
    with pytest.raises(NoNativeKernel, match="polarity"):
        body(lambda a, b: np.exp(a).mask, "bool").plan(f32, f32, FakeDev((1000,), "bool"), ctx=ctx)
    with pytest.raises(NoNativeKernel, match="inside a larger integer expression"):
        body(lambda a, b: (a % b) + (a // b).mask.astype(np.int32), "int32").plan(
            i32, i32, FakeDev((1000,), "int32"), ctx=ctx)
    # the mask of a whole expression binds: one more instruction, a one-byte output
    (p,) = body(lambda a, b: (a / b).mask, "bool").plan(f32, f32, FakeDev((1000,), "bool"), ctx=ctx)
    assert p.fn is rt.hcamdLaunchFMap and fmap_program(p)[-1][0] == "active"
    (p,) = body(lambda a, b: (a // b).mask, "bool").plan(i32, i32, FakeDev((1000,), "bool"), ctx=ctx)
    assert p.fn is rt.hcamdLaunchIMap and imap_program(p)[-1][0] == "active"


def test_allocated_tiles_bind_as_constants_and_assignment_targets(ctx):
    """CurrentGroup.full / zeros / ones / empty / vec (python/hckernel/kernel_api.py:347-376):
    a constant tile stored as it is is a program that pushes the constant and reads
    nothing; `tile[:] = value` on a fresh tile is the value; a part of a constant
    tile is the constant."""
    N = sym.N

    def body(fn):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, a: Buffer[N, DT], out: Buffer[N, DT]):
            o = gr.work_offset[0]
            gr.store(out[o:], fn(gr, gr.load(a[o:], shape=gr.shape)))
        return k

    f32, f16, i32 = (FakeDev((1000,), t) for t in ("float32", "float16", "int32"))
    (p,) = body(lambda gr, x: gr.full(gr.shape, dtype=np.float32, fill_value=2.5)).plan(f32, f32, ctx=ctx)
    assert p.fn is rt.hcamdLaunchMap and map_program(p) == [("const", 0, 2.5)] and p.args[6] == 0   # no operand
    (p,) = body(lambda gr, x: gr.vones(gr.shape, dtype=np.float16)).plan(f16, f16, ctx=ctx)
    assert map_program(p) == [("const", 0, 1.0)]
    (p,) = body(lambda gr, x: gr.full(gr.shape, dtype=np.int32, fill_value=-7)).plan(i32, i32, ctx=ctx)
    assert p.fn is rt.hcamdLaunchIMap and imap_program(p) == [("const", 0, -7)]
    (p,) = body(lambda gr, x: gr.zeros(gr.shape, dtype=np.bool_)).plan(i32, FakeDev((1000,), "bool"), ctx=ctx)
    assert p.fn is rt.hcamdLaunchIMap and imap_program(p) == [("const", 0, 0)]
    with pytest.raises(NoNativeKernel, match="int32 buffer"):
        body(lambda gr, x: gr.full(gr.shape, dtype=np.int32, fill_value=0.5)).plan(i32, i32, ctx=ctx)

    def filled(gr, x):
        t = gr.empty(gr.shape, dtype=np.float32)
        t[:] = x * np.float32(2)
        return gr.vec(t)
    (p,) = body(filled).plan(f32, f32, ctx=ctx)
    assert map_program(p) == [("in", 0, 0.0), ("muli", 0, 2.0)]
    # stored to a larger window the tile would carry the allocator's fill beyond the loaded part
    M = sym.M

    @kernel(work_shape=M, group_shape=256)
    def wider(gr: CurrentGroup, a: Buffer[N, DT], out: Buffer[M, DT]):
        o = gr.work_offset[0]
        gr.store(out[o:], filled(gr, gr.load(a[o:], shape=gr.shape)))
    with pytest.raises(NoNativeKernel, match=r"allocator's\s+initial value"):
        wider.plan(f32, FakeDev((1200,), "float32"), ctx=ctx)

    def part_of_constant(gr, x):
        return x + gr.vec(gr.full((512,), dtype=np.float32, fill_value=3), shape=gr.shape)
    (p,) = body(part_of_constant).plan(f32, f32, ctx=ctx)
    assert map_program(p) == [("in", 0, 0.0), ("addi", 0, 3.0)]


def test_row_bodies_without_native_code_say_why(ctx):
    M, N, GM = sym.M, sym.N, sym.GM

    def body(fn, out_shape=None):
        @kernel(work_shape=M, group_shape=GM)
        def k(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            gr.store(out[m0:, :], fn(gr.load(x[m0:, :], shape=(mb, N))))
        return k

    x16, x32 = FakeDev((64, 128), "float16"), FakeDev((64, 128), "float32")
    with pytest.raises(NoNativeKernel, match="cast the tile"):
        body(lambda t: t / t.sum(axis=1, keepdims=True)).plan(x16, FakeDev((64, 128), "float16"), 8, ctx=ctx)
    with pytest.raises(NoNativeKernel):                        # reductions down the columns
        body(lambda t: t - t.max(axis=0, keepdims=True)).plan(x32, FakeDev((64, 128), "float32"), 8, ctx=ctx)
    with pytest.raises(NoNativeKernel, match="row scalars"):
        def many(t):
            acc = t
            for k in range(17):
                acc = acc - (t * float(k + 1)).max(axis=1, keepdims=True)
            return acc
        body(many).plan(x32, FakeDev((64, 128), "float32"), 8, ctx=ctx)

    # tiles that hold parts of rows
    @kernel(work_shape=(M, N), group_shape=(8, 32))
    def partial(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT]):
        m0, n0 = gr.work_offset
        t = gr.load(x[m0:, n0:], shape=gr.shape)
        gr.store(out[m0:, n0:], t - t.max(axis=1, keepdims=True))
    with pytest.raises(NoNativeKernel, match="whole rows"):
        partial.plan(x32, FakeDev((64, 128), "float32"), ctx=ctx)


# ---------------------------------------------------------------------------
# Reductions down the columns -> hcamdLaunchMapReduceCols
# ---------------------------------------------------------------------------
def _col_bodies(deco):
    """Kernel bodies that reduce (M, GN) tiles holding whole columns along axis
    0, one group per block of GN columns; `deco` is hc_amd's kernel or the CPU
    simulator's."""
    M, N, GN = sym.M, sym.N, sym.GN

    def body(fn):
        @deco(work_shape=cdiv(N, GN), group_shape=1, literals={GN})
        def k(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], out: Buffer[N, DT],
              gn: GN):
            n0 = gr.id[0] * GN
            tx = gr.load(x[:, n0:], shape=(M, GN))
            ty = gr.load(y[:, n0:], shape=(M, GN))
            gr.store(out[n0:], fn(tx, ty))
        return k

    f32 = np.float32
    return {
        "col_sums": body(lambda a, b: (a * b).sum(axis=0)),
        "col_max_abs": body(lambda a, b: np.abs(a - b).max(axis=0)),
        "col_min": body(lambda a, b: np.minimum(a, b).min(axis=0)),
        "col_means": body(lambda a, b: (a + b).mean(axis=0) * f32(0.5)),
        "col_norms": body(lambda a, b: np.linalg.norm(a - b, axis=0)),
        "col_rms": body(lambda a, b: np.sqrt((a * a).sum(axis=0) / f32(a.shape[0]) + f32(1e-6))),
        "col_var": body(lambda a, b: a.var(axis=0)),
        "col_std": body(lambda a, b: (a - b).std(axis=0, ddof=1)),
    }


def _col_tile_bodies(deco):
    """Bodies that store a (M, GN) tile computed from reductions down its own
    columns (a batch normalisation, a column softmax)."""
    M, N, GN = sym.M, sym.N, sym.GN

    def body(fn):
        @deco(work_shape=cdiv(N, GN), group_shape=1, literals={GN})
        def k(gr: CurrentGroup, x: Buffer[M, N, DT], w: Buffer[M, N, DT], out: Buffer[M, N, DT],
              gn: GN):
            n0 = gr.id[0] * GN
            tx = gr.load(x[:, n0:], shape=(M, GN))
            tw = gr.load(w[:, n0:], shape=(M, GN))
            gr.store(out[:, n0:], fn(tx, tw))
        return k

    f32 = np.float32

    def batch_norm(a, b):
        mean = a.mean(axis=0, keepdims=True)
        return (a - mean) / np.sqrt(a.var(axis=0, keepdims=True) + f32(1e-5)) * b

    def col_softmax(a, b):
        e = np.exp(a - a.max(axis=0, keepdims=True))
        return e / e.sum(axis=0, keepdims=True)

    return {"batch_norm": body(batch_norm), "col_softmax": body(col_softmax),
            "centre": body(lambda a, b: a - (a * b).sum(axis=0, keepdims=True) / f32(a.shape[0]))}


def test_column_reductions_compile_to_a_program_a_fold_and_a_post_program(ctx):
    gpu = _col_bodies(kernel)
    x, y, out = FakeDev((40, 100), "float32"), FakeDev((40, 100), "float32"), FakeDev((100,), "float32")
    want = {
        "col_sums": ("sum", [("in", 0, 0.0), ("mul_in", 1, 0.0)], []),
        "col_max_abs": ("max", [("in", 0, 0.0), ("sub_in", 1, 0.0), ("abs", 0, 0.0)], []),
        "col_means": ("sum", [("in", 0, 0.0), ("add_in", 1, 0.0)],
                      # (numpy.ma's division: a mean that is not finite leaves the sum)
                      [("in", 0, 0.0), ("mdivi", 0, 40.0), ("muli", 0, 0.5)]),
        "col_norms": ("sum", None, [("in", 0, 0.0), ("sqrt", 0, 0.0)]),
    }
    names = {code: op for op, code in rt.MAP_OPS.items()}
    for name, (kind, program, post) in want.items():
        (p,) = gpu[name].plan(x, y, out, 32, ctx=ctx)
        assert p.fn is rt.hcamdLaunchMapReduceCols
        assert p.args[1] == rt.COLS_KINDS[kind] and p.args[12:14] == (40, 100)
        got = [(names[p.args[2][i].op], p.args[2][i].arg, p.args[2][i].imm)
               for i in range(p.args[3])]
        if program is not None:
            assert got == program
        got_post = [(names[p.args[4][i].op], p.args[4][i].arg, p.args[4][i].imm)
                    for i in range(p.args[5])]
        assert got_post == post
    # fp16 sums are refused with the advice to cast, as for rows
    x16 = FakeDev((40, 100), "float16")
    with pytest.raises(NoNativeKernel, match="cast the tile"):
        gpu["col_sums"].plan(x16, x16, FakeDev((100,), "float16"), 32, ctx=ctx)
    # tiles that do not hold whole columns
    M, N = sym.M, sym.N

    @kernel(work_shape=(cdiv(M, 8), cdiv(N, 32)), group_shape=(1, 1))
    def partial(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[N, DT]):
        t = gr.load(x[gr.id[0] * 8:, gr.id[1] * 32:], shape=(8, 32))
        gr.store(out[gr.id[1] * 32:], t.sum(axis=0))
    with pytest.raises(NoNativeKernel, match="whole columns"):
        partial.plan(x, out, ctx=ctx)


def random_row_expression(rng, depth):
    """A function of two (rows, N) tiles T, U and a vector W of N elements that
    mixes elementwise arithmetic with reductions along axis 1, and its source
    text.  Returns (function, text, per_row): per_row says the value has one
    element per row.  Everything is float32 (K = numpy.float32 keeps Python
    scalars from promoting the simulator's masked arithmetic to float64);
    denominators are kept away from zero and exponents bounded."""
    ops = ["+", "-", "*"]

    def elem(d):
        if d == 0 or rng.random() < 0.2:
            return rng.choice(["T", "T", "U", "W"])
        kind = rng.integers(0, 9)
        x = elem(d - 1)
        if kind <= 1:
            return f"({x} {rng.choice(ops)} {elem(d - 1)})"
        if kind <= 3:
            return f"({x} {rng.choice(ops)} {scal(d - 1)})"
        if kind == 4:
            return f"({x} / (np.abs({scal(d - 1)}) + K(1.0)))"
        if kind == 5:
            return f"np.exp(-np.abs({x}))"
        if kind == 6:
            return f"np.sqrt(np.abs({x}))"
        if kind == 7:
            return f"np.maximum({x}, {scal(d - 1)})"
        return f"({x} {rng.choice(ops + ['/'])} K({rng.choice(['0.5', '3.0', '-1.25'])}))"

    def scal(d, keep="True"):
        kind = rng.integers(0, 7) if d > 0 else 0
        if kind <= 2:
            inner = elem(max(d - 1, 0))
            if "T" not in inner and "U" not in inner:
                inner = f"(T + {inner})"                  # a reduction needs a tile under it
            fn = rng.choice(["sum", "max", "min", "mean"])
            return f"({inner}).{fn}(axis=1, keepdims={keep})"
        x = scal(d - 1, keep)
        if kind == 3:
            return f"({x} {rng.choice(ops)} {scal(d - 1, keep)})"
        if kind == 4:
            return f"np.sqrt(np.abs({x}))"
        if kind == 5:
            return f"({x} / (np.abs({scal(d - 1, keep)}) + K(1.0)))"
        return f"({x} {rng.choice(ops)} K({rng.choice(['0.25', '2.0'])}))"

    per_row = rng.random() < 0.3
    if per_row:
        text = scal(depth, keep="False")
    else:
        text = f"({elem(depth)} {rng.choice(ops)} {scal(depth - 1)})"
    return eval(f"lambda T, U, W: {text}", {"np": np, "K": np.float32}), text, per_row


def random_row_body(deco, expr, per_row):
    M, N, GM = sym.M, sym.N, sym.GM
    if per_row:
        @deco(work_shape=M, group_shape=GM)
        def body(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], v: Buffer[N, DT],
                 out: Buffer[M, DT], gshape: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            gr.store(out[m0:], expr(gr.load(x[m0:, :], shape=(mb, N)),
                                    gr.load(y[m0:, :], shape=(mb, N)), gr.load(v[:], shape=(N,))))
    else:
        @deco(work_shape=M, group_shape=GM)
        def body(gr: CurrentGroup, x: Buffer[M, N, DT], y: Buffer[M, N, DT], v: Buffer[N, DT],
                 out: Buffer[M, N, DT], gshape: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            gr.store(out[m0:, :], expr(gr.load(x[m0:, :], shape=(mb, N)),
                                       gr.load(y[m0:, :], shape=(mb, N)), gr.load(v[:], shape=(N,))))
    return body


def random_row_operands(rng, rows, n, per_row):
    f = np.float32
    return [(rng.uniform(0.5, 2.0, (rows, n)) * rng.choice([-1.0, 1.0], (rows, n))).astype(f),
            rng.standard_normal((rows, n)).astype(f), rng.uniform(-1.0, 1.0, n).astype(f),
            np.zeros(rows if per_row else (rows, n), f)]


def test_random_row_expressions_compile_to_stages_that_mean_the_same(ctx):
    """Random bodies with reductions along rows: the stages the front-end emits,
    run in NumPy, against the simulator running the body itself."""
    from oracle.hcsim import kernel as sim_kernel
    rng = np.random.default_rng(2024)
    rows, n = 21, 96
    bound = tried = 0
    while bound < 40:
        expr, text, per_row = random_row_expression(rng, 3)
        tried += 1
        host = random_row_operands(rng, rows, n, per_row)
        fake = [FakeDev(a.shape, a.dtype.name) for a in host]
        try:
            (p,) = random_row_body(kernel, expr, per_row).plan(*fake, 8, ctx=ctx)
        except NoNativeKernel as exc:
            assert any(w in str(exc) for w in ("stack", "row scalars", "operations", "passes", "numpy.ma leaves",
                                               "arrays")), (text, str(exc))
            continue
        assert p.fn is rt.hcamdLaunchRowProgram, text
        bound += 1
        stages = row_stages(p)
        by_ptr = {f.ptr: a for f, a in zip(fake, host)}
        inputs = [by_ptr[p.args[4][i]] for i in range(p.args[7])]
        assert p.args[10] == 0, text
        got = run_row_stages(stages, inputs, (), np.float32)
        want = host[-1].copy()
        with np.errstate(all="ignore"):
            random_row_body(sim_kernel, expr, per_row)(*host[:-1], want, 8)
        scale = 1.0 + float(np.abs(want).max())
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5 * scale, err_msg=text)
    assert tried < 120


# ---------------------------------------------------------------------------
# Control flow on group ids, subgroup and work-item scopes
# ---------------------------------------------------------------------------
def test_control_flow_on_the_group_id_is_refused_not_miscompiled(ctx):
    N = sym.N
    a, b = FakeDev((1024,), "float32"), FakeDev((1024,), "float32")
    for test in (lambda gr: gr.work_offset[0] == 0, lambda gr: gr.id[0] != 0,
                 lambda gr: bool(gr.id[0]), lambda gr: (gr.id[0] // 2) == 0,
                 lambda gr: bool(gr.id[0] % 2)):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, src: Buffer[N, DT], dst: Buffer[N, DT]):
            o = gr.work_offset[0]
            if test(gr):
                gr.store(dst[o:], gr.load(src[o:], shape=gr.shape[0]))

        with pytest.raises(NoNativeKernel, match="traced once for all groups"):
            k.plan(a, b, ctx=ctx)

    # the same tests on numbers that do not depend on the group are fine
    @kernel(work_shape=N, group_shape=256)
    def k2(gr: CurrentGroup, src: Buffer[N, DT], dst: Buffer[N, DT]):
        o = gr.work_offset[0]
        if (o - o) == 0 and gr.shape[0] == 256:
            gr.store(dst[o:], gr.load(src[o:], shape=gr.shape[0]))

    (p,) = k2.plan(a, b, ctx=ctx)
    assert p.fn is rt.hcamdLaunchCopy2D


def _softmax_with_subgroup_partials(rows_per_group, lanes, sg):
    from hc_amd.kernel import CurrentSubGroup
    ROWS, N = sym.ROWS, sym.N

    @kernel(work_shape=(ROWS, lanes), group_shape=(rows_per_group, lanes), subgroup_size=sg)
    def softmax(gr: CurrentGroup, x: Buffer[ROWS, N, DT], y: Buffer[ROWS, N, DT]):
        r0 = gr.work_offset[0]
        n = x.shape[1]
        nsub = gr.shape[1] // sg
        seg = n // nsub
        t = gr.load(x[r0:], shape=(gr.shape[0], n))
        pmax = gr.zeros((gr.shape[0], nsub), np.float32)

        @gr.subgroups
        def part_max(s: CurrentSubGroup):
            i, k = s.subgroup_id()
            pmax[i, k] = t[i, k * seg:(k + 1) * seg].max()

        part_max()
        gr.barrier()
        e = np.exp(t - pmax.max(axis=1, keepdims=True))
        psum = gr.zeros((gr.shape[0], nsub), np.float32)

        @gr.subgroups
        def part_sum(s: CurrentSubGroup):
            i, k = s.subgroup_id()
            psum[i, k] = e[i, k * seg:(k + 1) * seg].sum()

        part_sum()
        gr.barrier()
        gr.store(y[r0:], e / psum.sum(axis=1, keepdims=True))

    return softmax


def test_subgroup_partials_fold_back_into_the_row_softmax(ctx):
    x, y = FakeDev((64, 8192), "float32"), FakeDev((64, 8192), "float32")
    for rows, lanes, sg in ((1, 256, 64), (2, 256, 64), (1, 1024, 64), (1, 256, 16)):
        (p,) = _softmax_with_subgroup_partials(rows, lanes, sg).plan(x, y, ctx=ctx)
        assert p.fn is rt.hcamdLaunchSoftmaxF32
        assert p.args[1] == x.ptr and p.args[3] == y.ptr and p.args[5:7] == (64, 8192)


def test_subgroup_partials_that_do_not_cover_the_row_are_not_folded(ctx):
    from hc_amd.kernel import CurrentSubGroup
    ROWS, N = sym.ROWS, sym.N

    @kernel(work_shape=(ROWS, 256), group_shape=(1, 256), subgroup_size=64)
    def k(gr: CurrentGroup, x: Buffer[ROWS, N, DT], y: Buffer[ROWS, N, DT]):
        r0 = gr.work_offset[0]
        t = gr.load(x[r0:], shape=(1, x.shape[1]))
        pmax = gr.zeros((1, 4), np.float32)

        @gr.subgroups
        def part(s: CurrentSubGroup):
            i, k = s.subgroup_id()
            pmax[i, k] = t[i, k * 100:(k + 1) * 100].max()      # 400 of 1024 columns

        part()
        gr.store(y[r0:], t - pmax.max(axis=1, keepdims=True))

    with pytest.raises(NoNativeKernel):
        k.plan(FakeDev((8, 1024), "float32"), FakeDev((8, 1024), "float32"), ctx=ctx)


def test_subgroup_scope_runs_like_the_simulator(ctx):
    """Ids, sizes and barrier phases of python/hckernel/tests/test_kernel_sim.py:229-320,
    observed while the body is traced: one pass per subgroup id, in order."""
    from hc_amd.kernel import CurrentSubGroup
    G1, G2, G3, L1, L2, L3 = sym.G1, sym.G2, sym.G3, sym.L1, sym.L2, sym.L3
    seen = []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=4)
    def k(gr: CurrentGroup, g: tuple[G1, G2, G3], l: tuple[L1, L2, L3], out):
        @gr.subgroups
        def inner(s: CurrentSubGroup):
            seen.append((1, s.subgroup_id(), s.size()))
            gr.barrier()
            seen.append((2, s.subgroup_id(), s.size()))

        inner()
        out[gr.id[2]] = gr.id[2]

    (p,) = k.plan((1, 1, 16), (1, 1, 8), FakeDev((2,), "int32"), ctx=ctx)
    assert seen == [(1, (0, 0, 0), 4), (1, (0, 0, 1), 4), (2, (0, 0, 0), 4), (2, (0, 0, 1), 4)]
    assert p.fn is rt.hcamdLaunchIdScatter


def test_workitem_scope_binds_ids_and_elementwise_statements(ctx):
    from hc_amd.kernel import CurrentWorkitem
    N = sym.N

    @kernel(work_shape=N, group_shape=64)
    def ids(gr: CurrentGroup, lid: Buffer[N, DT], gid: Buffer[N, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            (g,) = wi.global_id()
            lid[g] = wi.local_id()[0]
            gr.barrier()
            gid[g] = 2 * g + 1

        inner()

    a, b = FakeDev((256,), "int32"), FakeDev((256,), "int32")
    p1, p2 = ids.plan(a, b, ctx=ctx)
    assert p1.fn is rt.hcamdLaunchIdScatter and p2.fn is rt.hcamdLaunchIdScatter
    idx, val = p1.args[6][0], p1.args[7]._obj
    assert (idx.c, idx.g[0], idx.l[0]) == (0, 64, 1) and (val.c, val.g[0], val.l[0]) == (0, 0, 1)
    val2 = p2.args[7]._obj
    assert (val2.c, val2.g[0], val2.l[0]) == (1, 128, 2)
    assert tuple(p1.args[9]) == (4,) and tuple(p1.args[10]) == (64,) and p1.args[11] == 1

    @kernel(work_shape=N, group_shape=256)
    def vadd(gr: CurrentGroup, x: Buffer[N, DT], y: Buffer[N, DT], z: Buffer[N, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            i = wi.global_id()
            z[i] = x[i] + y[i]

        inner()

    x, y, z = (FakeDev((4096,), "float32") for _ in range(3))
    (p,) = vadd.plan(x, y, z, ctx=ctx)
    assert p.fn is rt.hcamdLaunchAddF32 and p.args[1:4] == (x.ptr, y.ptr, z.ptr)

    @kernel(work_shape=N, group_shape=256)
    def shifted(gr: CurrentGroup, x: Buffer[N, DT], z: Buffer[N, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            (i,) = wi.global_id()
            z[i] = x[i + 1]

        inner()

    with pytest.raises(NoNativeKernel, match="wi.global_id"):
        shifted.plan(x, z, ctx=ctx)

    # stores of ids whose outcome would depend on the order of the work-items, or
    # on NumPy's wrap-around of negative indices, are refused
    def id_body(index, value, group=64):
        @kernel(work_shape=N, group_shape=group)
        def k(gr: CurrentGroup, out: Buffer[N, DT]):
            @gr.workitems
            def inner(wi: CurrentWorkitem):
                out[index(gr, wi)] = value(gr, wi)

            inner()
        return k

    o = FakeDev((256,), "int32")
    with pytest.raises(NoNativeKernel, match="different values to one element"):
        id_body(lambda gr, wi: gr.id[0], lambda gr, wi: wi.local_id()[0]).plan(o, ctx=ctx)
    with pytest.raises(NoNativeKernel, match="goes below 0"):
        id_body(lambda gr, wi: wi.global_id()[0] - 1, lambda gr, wi: wi.local_id()[0]).plan(o, ctx=ctx)
    # the same element from every work-item of a group, but the same value: fine
    (p,) = id_body(lambda gr, wi: gr.id[0], lambda gr, wi: gr.id[0] * 3).plan(o, ctx=ctx)
    assert p.fn is rt.hcamdLaunchIdScatter
    # more stores than can be enumerated: a global id is still known to be one-to-one
    big = FakeDev((1 << 24,), "int32")
    (p,) = id_body(lambda gr, wi: wi.global_id()[0], lambda gr, wi: wi.local_id()[0], group=256).plan(big, ctx=ctx)
    assert p.fn is rt.hcamdLaunchIdScatter
    with pytest.raises(NoNativeKernel, match="too many to check"):
        id_body(lambda gr, wi: wi.global_id()[0] - gr.id[0], lambda gr, wi: wi.local_id()[0], group=256).plan(big, ctx=ctx)

    @kernel(work_shape=(N, 8), group_shape=(1, 8))
    def tall(gr: CurrentGroup, out: Buffer[N, 8, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            out[wi.global_id()] = wi.local_id()[1]

        inner()

    with pytest.raises(NoNativeKernel, match="at most 65535"):
        tall.plan(FakeDev((70_000, 8), "int32"), ctx=ctx)


def test_vload_needs_a_static_shape(ctx):
    """docs/langref.md:226-243 of the reference: a vector's shape must be known at
    compile time.  Numbers, group.shape, literal symbols and tunables are;
    buffer dimensions and ordinary scalar arguments are not."""
    W, H, V, T, S = sym.W, sym.H, sym.V, sym.T, sym.S
    a, b = FakeDev((64, 1024), "int32"), FakeDev((64, 1024), "int32")

    @kernel(work_shape=(W, sympy.ceiling(H / V)), literals=[V])
    def literal(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT], v: V):
        x, y = gr.work_offset
        gr.store(dst[x:, y * V:], gr.vload(src[x:, y * V:], shape=(gr.shape[0], gr.shape[1] * V)))

    (p,) = literal.plan(a, b, 4, ctx=ctx)
    assert p.fn is rt.hcamdLaunchCopy2D

    @kernel(work_shape=W, group_shape=1, tunables=TunableParam(T, 1024, [512, 1024]))
    def tunable(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x = gr.work_offset[0]
        gr.store(dst[x:, :], gr.vload(src[x:, :], shape=(1, T)))

    (p,) = tunable.plan(a, b, ctx=ctx)
    assert p.fn is rt.hcamdLaunchCopy2D

    @kernel(work_shape=W, group_shape=1)
    def from_buffer_dim(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x = gr.work_offset[0]
        gr.store(dst[x:, :], gr.vload(src[x:, :], shape=(1, H)))

    @kernel(work_shape=W, group_shape=1)
    def from_shape_attr(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x = gr.work_offset[0]
        gr.store(dst[x:, :], gr.vload(src[x:, :], shape=(1, src.shape[1] // 2 * 2)))

    @kernel(work_shape=W, group_shape=1)
    def from_scalar(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT], n: S):
        x = gr.work_offset[0]
        gr.store(dst[x:, :], gr.vload(src[x:, :], shape=(1, n)))

    for k, extra in ((from_buffer_dim, ()), (from_shape_attr, ()), (from_scalar, (1024,))):
        with pytest.raises(NoNativeKernel, match="static shape"):
            k.plan(a, b, *extra, ctx=ctx)

    # the same bodies with load are fine
    @kernel(work_shape=W, group_shape=1)
    def with_load(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
        x = gr.work_offset[0]
        gr.store(dst[x:, :], gr.load(src[x:, :], shape=(1, H)))

    (p,) = with_load.plan(a, b, ctx=ctx)
    assert p.fn is rt.hcamdLaunchCopy2D


def test_traced_arrays_are_not_kept_alive_by_the_cache(ctx):
    import gc
    import weakref
    N = sym.N

    @kernel(work_shape=N, group_shape=256)
    def k(gr: CurrentGroup, src: Buffer[N, DT], dst: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(dst[o:], gr.load(src[o:], shape=gr.shape[0]))

    a, b = FakeDev((1024,), "float32"), FakeDev((1024,), "float32")
    k.plan(a, b, ctx=ctx)
    ra = weakref.ref(a)
    del a, b
    gc.collect()
    assert ra() is None, "the kernel's plan cache holds the arrays of the call that was traced"


def test_thread_variants_are_private_to_the_thread():
    import threading
    with pytest.raises(rt.HcRuntimeError):
        rt.set_thread_variant("no_such_family", 1)
    rt.set_thread_variant("gemm", 14)
    seen = {}

    def other():
        # another thread neither sees the override nor disturbs it
        rt.set_thread_variant("gemm", 7)
        rt.set_thread_variant("gemm", -1)
        seen["ok"] = True

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["ok"]
    rt.set_thread_variant("gemm", -1)


def fmap_program(plan):
    """(opname, arg, imm) triples of a hcamdLaunchFMap plan."""
    names = {v: k for k, v in rt.FMAP_OPS.items()}
    prog, n = plan.args[1], plan.args[2]
    return [(names[prog[i].op], prog[i].arg, prog[i].imm) for i in range(n)]


def test_float_operators_follow_numpy_ma_and_pick_the_kernel_that_can(ctx):
    """The tile operators / // % ** go through numpy.ma in the reference
    (python/hckernel/kernel_api.py:157-180): failed divisions deactivate their
    elements.  The fast map kernel keeps one flag per element, which is exact
    when the result is a tile (deactivated elements are not stored) or when only
    NumPy functions without a domain sit above the divisions; everything else,
    // % and comparisons go to the general float map."""
    N = sym.N
    f = np.float32

    def plan(expr, out_dt="float32", in_dt="float32"):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, DT]):
            o, g = gr.work_offset[0], gr.shape[0]
            gr.store(out[o:], expr(gr.load(a[o:], shape=g), gr.load(b[o:], shape=g)))
        (p,) = k.plan(FakeDev((1000,), in_dt), FakeDev((1000,), in_dt), FakeDev((1000,), out_dt), ctx=ctx)
        return p

    # the operator: numpy.ma's division; the function: domain fill, general map
    p = plan(lambda a, b: a / b)
    assert p.fn is rt.hcamdLaunchMap and map_program(p) == [("in", 0, 0.0), ("mdiv_in", 1, 0.0)]
    p = plan(lambda a, b: np.divide(a, b))
    assert p.fn is rt.hcamdLaunchFMap and fmap_program(p) == [("in", 0, 0.0), ("in", 1, 0.0), ("udiv", 0, 0.0)]
    assert p.args[-1] == 1                                  # a bare numpy.ma array: stored in full
    # fp16 tiles: the quotient is tested after rounding to fp16 (bit 8 of the operand form's arg)
    p = plan(lambda a, b: a / b + np.float16(1), "float16", "float16")
    assert map_program(p) == [("in", 0, 0.0), ("mdiv_in", 0x101, 0.0), ("addi", 0, 1.0), ("r16", 0, 0.0)]
    # a function without a domain above the division: plain arithmetic on what numpy.ma
    # leaves (the dividend), everything stored
    p = plan(lambda a, b: np.exp(a / b))
    assert p.fn is rt.hcamdLaunchMap
    assert [i[0] for i in map_program(p)] == ["in", "mdiv_in", "exp", "clear"]
    # numpy.sqrt / numpy.log have domains
    p = plan(lambda a, b: a * np.sqrt(b) + b * np.log(a))
    assert p.fn is rt.hcamdLaunchMap
    assert [i[0] for i in map_program(p)] == ["in", "msqrt", "mul_in", "in", "mlog", "mul_in", "add"]
    p = plan(lambda a, b: np.sqrt(a) + np.log(b))           # a bare array on the left: stored in full
    assert p.fn is rt.hcamdLaunchFMap and p.args[-1] == 1
    # ** : numpy.ma.power's check for results that are not finite
    p = plan(lambda a, b: a ** f(2) / b)
    assert [i[0] for i in map_program(p)] == ["in", "mul_in", "powchk", "mdiv_in"]
    # an operator above a division in a result that is stored in full needs numpy.ma's values
    p = plan(lambda a, b: np.abs(a / b) - b / a)
    assert p.fn is rt.hcamdLaunchFMap and p.args[-1] == 1
    assert [i[0] for i in fmap_program(p)] == ["in", "in", "div", "abs", "in", "in", "div", "sub"]
    # the same shape as a tile (left operand a tile): deactivated elements are not stored
    p = plan(lambda a, b: a / b + np.abs(b / a))
    assert p.fn is rt.hcamdLaunchMap
    # // % and comparisons
    p = plan(lambda a, b: (a // b) % f(3))
    assert p.fn is rt.hcamdLaunchFMap and p.args[-1] == 0
    assert fmap_program(p) == [("in", 0, 0.0), ("in", 1, 0.0), ("floordiv", 0, 0.0), ("const", 0, 3.0),
                               ("mod", 0, 0.0)]
    p = plan(lambda a, b: a < b, out_dt="bool")
    assert p.fn is rt.hcamdLaunchFMap and p.args[8] == rt.U8
    assert [i[0] for i in fmap_program(p)] == ["in", "in", "lt"]
    p = plan(lambda a, b: np.add(a, b) * (a - b))            # + as a function: arg bit 1
    assert p.fn is rt.hcamdLaunchMap                         # nothing can deactivate anything
    p = plan(lambda a, b: np.add(a // b, b))
    assert fmap_program(p)[-1] == ("add", 2, 0.0)
    with pytest.raises(NoNativeKernel, match="floor_divide"):
        plan(lambda a, b: np.floor_divide(a, b))


def test_results_of_numpy_where_are_plain_arrays_with_numpys_own_arithmetic(ctx):
    """numpy.where (and tile.mask) return plain NumPy arrays in the reference:
    operators and functions of those alone are NumPy's own (IEEE quotients,
    NaN for a root of a negative number, nothing deactivated: `arg` bit 2),
    next to a tile the tile's reflected operator runs and the result is a tile
    again (stored where active), and a NumPy scalar on the left of a tile is a
    TypeError as it is there."""
    N = sym.N
    f = np.float32

    def plan(expr):
        @kernel(work_shape=N, group_shape=256)
        def k(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, DT]):
            o, g = gr.work_offset[0], gr.shape[0]
            gr.store(out[o:], expr(gr.load(a[o:], shape=g), gr.load(b[o:], shape=g)))
        (p,) = k.plan(FakeDev((1000,), "float32"), FakeDev((1000,), "float32"), FakeDev((1000,), "float32"),
                      ctx=ctx)
        return p

    p = plan(lambda a, b: np.where(a < b, a, b) / f(-0.125))
    assert fmap_program(p)[-2:] == [("const", 0, -0.125), ("div", 4, 0.0)] and p.args[-1] == 1
    p = plan(lambda a, b: np.sqrt(np.where(a < b, a, b)) % f(2))
    assert fmap_program(p)[-3:] == [("sqrt", 4, 0.0), ("const", 0, 2.0), ("mod", 4, 0.0)] and p.args[-1] == 1
    p = plan(lambda a, b: np.where(a < b, a, b) ** f(0.5) // np.where(a < b, b, a))
    assert [i[:2] for i in fmap_program(p) if i[0] in ("sqrt", "psqrt", "floordiv", "powchk")] == \
        [("sqrt", 4), ("floordiv", 4)]
    # next to a tile: on the right numpy.ma's operator, and a tile again; on the left NumPy
    # defers to the tile, which has no reflected operators
    with pytest.raises(TypeError):
        plan(lambda a, b: np.where(a < b, a, b) // a)
    p = plan(lambda a, b: a / np.where(a < b, a, b))
    assert fmap_program(p)[-1] == ("div", 0, 0.0) and p.args[-1] == 0
    # next to what a NumPy function of a tile returned: numpy.ma's operator, stored in full
    p = plan(lambda a, b: np.where(a < b, a, b) / np.exp(a))
    assert fmap_program(p)[-1] == ("div", 0, 0.0) and p.args[-1] == 1
    for op in ("+", "-", "*", "/", "//", "%", "**"):
        with pytest.raises(TypeError):
            plan(eval(f"lambda a, b: f(2) {op} a", {"f": f}))
