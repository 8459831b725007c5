"""Pins the host executor (oracle/hcsim) to the known answers the reference's
own simulator tests hold: python/hckernel/tests/test_kernel_sim.py (group
iteration, masked load/store tails, allocators, subgroup / work-item iteration,
barrier interleaving, Buffer symbol binding, symbol resolution, tunables) and
python/hckernel/tests/test_examples.py (reductions, dot, softmax, pairwise
distance, implicit GEMM)."""

from itertools import product

import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_equal

from oracle.hcsim import (Buffer, CurrentGroup, CurrentSubGroup, CurrentWorkitem,
                          TunableParam, atomic_ref, create_mapping, kernel, sym,
                          typename)

DT = typename.DT
G1, G2, G3 = sym.G1, sym.G2, sym.G3
L1, L2, L3 = sym.L1, sym.L2, sym.L3


def cdiv(a, b):
    return (a + b - 1) // b


# --- geometry (test_kernel_sim.py:26-54) ------------------------------------
@pytest.mark.parametrize("work", [(512, 1, 1), (511, 1, 1), (1, 16, 1), (1, 1, 16), (1, 1, 1)])
@pytest.mark.parametrize("group", [(64, 1, 1), (1, 1, 1)])
def test_groups_visit_row_major(work, group):
    seen = []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3))
    def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
        seen.append((gr.id, gr.work_offset))

    k(work, group)
    ids = list(product(*(range(cdiv(w, g)) for w, g in zip(work, group))))
    assert [s[0] for s in seen] == ids
    assert [s[1] for s in seen] == [tuple(i * g for i, g in zip(t, group)) for t in ids]
    # tiles are disjoint and cover the work shape
    covered = np.zeros(work, int)
    for _, off in seen:
        covered[tuple(slice(o, o + g) for o, g in zip(off, group))] += 1
    assert (covered == 1).all()


# --- masked load / store tails (test_kernel_sim.py:57-104) --------------------
@pytest.mark.parametrize("work,expected", [
    (8, [list(range(8))]),
    (16, [list(range(8)), [8, 9, 10, 11]]),
])
def test_load_masks_past_the_end(work, expected):
    got = []

    @kernel(work_shape=sym.G, group_shape=sym.L)
    def k(gr: CurrentGroup, g: sym.G, l: sym.L, arr):
        got.append(gr.load(arr[gr.work_offset[0]:], shape=gr.shape[0]).compressed())

    k(work, 8, np.arange(12))
    assert_equal(got, [np.array(e) for e in expected])


def test_store_leaves_out_of_window_untouched():
    @kernel(work_shape=sym.G, group_shape=sym.L)
    def k(gr, g: sym.G, l: sym.L, src, dst):
        o = gr.work_offset[0]
        gr.store(dst[o:], gr.load(src[o:], shape=gr.shape[0]))

    dst = np.full(16, -1)
    k(16, 8, np.arange(12), dst)
    assert_equal(dst, list(range(12)) + [-1] * 4)


def test_store_2d_ragged_poisoned_destination():
    # e2e copy shapes of test_e2e.py:46-54 on the host executor
    W, H = sym.W, sym.H
    for shape in [(1, 27), (1, 72), (10, 20), (111, 813), (256, 64)]:
        @kernel(work_shape=(W, H), group_shape=(4, 32))
        def k(gr: CurrentGroup, src: Buffer[W, H, DT], dst: Buffer[W, H, DT]):
            x, y = gr.work_offset
            gr.store(dst[x:, y:], gr.load(src[x:, y:], shape=gr.shape))

        a = np.arange(shape[0] * shape[1], dtype=np.int32).reshape(shape)
        b = np.full_like(a, -7)
        k(a, b)
        assert_equal(b, a)


# --- allocators (test_kernel_sim.py:107-226) ----------------------------------
@pytest.mark.parametrize("name,args,value", [
    ("empty", {}, None), ("vempty", {}, None),
    ("zeros", {}, 0), ("vzeros", {}, 0), ("ones", {}, 1), ("vones", {}, 1),
    ("full", {"fill_value": 42}, 42), ("vfull", {"fill_value": 42}, 42),
])
def test_allocators(name, args, value):
    @kernel(work_shape=sym.G, group_shape=sym.L)
    def k(gr, g: sym.G, l: sym.L):
        t = getattr(gr, name)((2, 3), dtype=np.int32, **args)
        assert_equal(t.shape, (2, 3))
        assert t.mask.all()          # every allocator yields active elements
        if value is not None:
            assert_equal(t, np.full((2, 3), value))

    k(8, 8)


def test_vec_copies_and_slices():
    @kernel(work_shape=sym.G, group_shape=sym.L)
    def k(gr, g: sym.G, l: sym.L):
        a = gr.full((2, 3), dtype=np.int32, fill_value=42)
        assert_equal(gr.vec(a), [[42] * 3] * 2)
        assert_equal(gr.vec(a, shape=(1, 2)), [[42, 42]])

    k(8, 8)


# --- scopes (test_kernel_sim.py:229-379) ---------------------------------------
@pytest.mark.parametrize("literal", [False, True])
def test_subgroup_ids_and_sizes(literal):
    ids, sizes = [], []
    SG = sym.SG

    def body(gr):
        @gr.subgroups
        def inner(s: CurrentSubGroup):
            ids.append(s.subgroup_id())
            sizes.append(s.size())

        inner()

    if literal:
        @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=SG,
                literals={SG})
        def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3], sg: SG):
            body(gr)

        k((1, 1, 16), (1, 1, 8), 4)
    else:
        @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=4)
        def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
            body(gr)

        k((1, 1, 16), (1, 1, 8))
    assert ids == [(0, 0, 0), (0, 0, 1)] * 2
    assert sizes == [4] * 4


def test_subgroup_barrier_order():
    log = []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=4)
    def k(gr, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
        @gr.subgroups
        def inner(s):
            log.append((1, s.subgroup_id()))
            gr.barrier()
            log.append((2, s.subgroup_id()))

        inner()

    k((1, 1, 16), (1, 1, 8))
    one_group = [(1, (0, 0, 0)), (1, (0, 0, 1)), (2, (0, 0, 0)), (2, (0, 0, 1))]
    assert log == one_group * 2


def test_workitem_ids():
    lids, gids = [], []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3))
    def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            lids.append(wi.local_id())
            gids.append(wi.global_id())

        inner()

    k((1, 1, 4), (1, 1, 2))
    assert lids == [(0, 0, 0), (0, 0, 1)] * 2
    assert gids == [(0, 0, i) for i in range(4)]


def test_workitem_barrier_order():
    log = []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3))
    def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            log.append((1, wi.global_id()))
            gr.barrier()
            log.append((2, wi.global_id()))

        inner()

    k((1, 1, 4), (1, 1, 2))
    assert log == [(1, (0, 0, 0)), (1, (0, 0, 1)), (2, (0, 0, 0)), (2, (0, 0, 1)),
                   (1, (0, 0, 2)), (1, (0, 0, 3)), (2, (0, 0, 2)), (2, (0, 0, 3))]


def test_three_phase_barrier_keeps_phases_together():
    # invariant beyond the reference's two cases: with two barriers and three
    # tasks, no task enters phase k+1 before all have finished phase k
    log = []

    @kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3))
    def k(gr: CurrentGroup, w: tuple[G1, G2, G3], g: tuple[L1, L2, L3]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            for phase in range(3):
                log.append(phase)
                if phase < 2:
                    gr.barrier()

        inner()

    k((1, 1, 3), (1, 1, 3))
    assert log == sorted(log)


# --- symbol binding (test_kernel_sim.py:382-470) ---------------------------------
def test_buffer_binds_dims_1d_and_2d():
    G = sym.G

    @kernel(work_shape=G)
    def k1(gr: CurrentGroup, arr: Buffer[G, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            i = wi.global_id()[0]
            if i < arr.shape[0]:
                arr[i] = i

        inner()

    a = np.zeros(12)
    k1(a)
    assert_equal(a, np.arange(12))

    @kernel(work_shape=(G1, G2))
    def k2(gr: CurrentGroup, arr: Buffer[G1, G2, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            i, j = wi.global_id()[:2]
            if i < arr.shape[0] and j < arr.shape[1]:
                arr[i, j] = i * arr.shape[1] + j

        inner()

    b = np.zeros((12, 5))
    k2(b)
    assert_equal(b, np.arange(60).reshape(12, 5))


def test_conflicting_symbol_values_assert():
    G = sym.G

    @kernel(work_shape=G)
    def k(gr: CurrentGroup, a: Buffer[G, DT], b: Buffer[G, DT]):
        pass

    with pytest.raises(AssertionError, match="Symbol value conflict"):
        k(np.zeros(3), np.zeros(4))


GG = sym.GG


def test_symbols_in_closure_and_globals_become_ints():
    G = sym.G

    @kernel(work_shape=G)
    def free(gr: CurrentGroup, arr: Buffer[G, DT]):
        arr[:] = G

    @kernel(work_shape=GG)
    def glob(gr: CurrentGroup, arr: Buffer[GG, DT]):
        arr[:] = GG

    for k in (free, glob):
        a = np.zeros(12)
        k(a)
        assert_equal(a, np.full(12, 12))


@pytest.mark.parametrize("symbol", ["free", "global"])
def test_tunable_default_and_parametrize(symbol):
    S = sym.G if symbol == "free" else GG
    T = TunableParam(S, 5, range(0, 10))

    if symbol == "free":
        @kernel(work_shape=10, tunables=T)
        def k(gr: CurrentGroup, arr: Buffer[10, DT]):
            arr[:] = S
    else:
        @kernel(work_shape=10, tunables=T)
        def k(gr: CurrentGroup, arr: Buffer[10, DT]):
            arr[:] = GG

    a = np.zeros(10)
    k(a)
    assert_equal(a, np.full(10, 5))
    k.parametrize({S: 10})(a)
    assert_equal(a, np.full(10, 10))


def test_decorator_argument_checks():
    with pytest.raises(AssertionError):
        kernel(work_shape=(1, 2, 3, 4))
    with pytest.raises(AssertionError):
        kernel(work_shape=(4, 4), group_shape=(2,))
    with pytest.raises(AssertionError, match="Subgroup size"):
        kernel(work_shape=4, subgroup_size=sym.SG)


# --- example kernels (test_examples.py) -------------------------------------------
def test_reductions_with_atomic_ref():
    WS, GS, N = sym.WS, sym.GS, sym.N
    TN = TunableParam(N, 2, range(1, 64))

    @kernel(work_shape=cdiv(WS, N), group_shape=GS, tunables=TN)
    def whole_tile(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], g: GS):
        view = gr.load(a[gr.work_offset[0] * N:], shape=gr.size * N)
        atomic_ref(result)[0] += view.sum()

    @kernel(work_shape=cdiv(WS, N), group_shape=GS, tunables=TN)
    def strided(gr: CurrentGroup, a: Buffer[WS, DT], result: Buffer[1, DT], g: GS):
        acc = gr.zeros(gr.size, dtype=a.dtype)
        for i in range(N):
            acc += gr.load(a[gr.work_offset[0] * N + i * gr.size:], shape=gr.size)
        atomic_ref(result)[0] += acc.sum()

    a = np.arange(0, 20)
    for k in (whole_tile, strided):
        r = np.zeros(1)
        k(a, r, 8)
        assert_equal(r[0], a.sum())


@pytest.mark.parametrize("blocked", [True, False])
def test_dot_matches_numpy(blocked):
    M, N, K = sym.M, sym.N, sym.K
    GM, GN, MI, NI, KB = sym.GM, sym.GN, sym.MI, sym.NI, sym.KB
    tun = (TunableParam(MI, 1, range(1, 8)), TunableParam(NI, 1, range(1, 8)),
           TunableParam(KB, 16, range(8, 128)))
    KI = cdiv(K, KB)

    @kernel(work_shape=(cdiv(M, MI), cdiv(N, NI)), group_shape=(GM, GN), tunables=tun)
    def dot(gr: CurrentGroup, a: Buffer[M, K, DT], b: Buffer[K, N, DT],
            out: Buffer[M, N, DT], g: (GM, GN)):
        m0, n0 = gr.work_offset[0] * MI, gr.work_offset[1] * NI
        mb, nb = gr.shape[0] * MI, gr.shape[1] * NI
        r = gr.zeros(shape=(mb, nb), dtype=out.dtype)
        if blocked:
            for k in range(KI):
                k0 = k * KB
                r += np.dot(gr.load(a[m0:, k0:], shape=(mb, KB)),
                            gr.load(b[k0:, n0:], shape=(KB, nb)))
        else:
            r += np.dot(gr.load(a[m0:, :], shape=(mb, K)),
                        gr.load(b[:, n0:], shape=(K, nb)))
        gr.store(out[m0:, n0:], r)

    m, n, k = 16, 32, 64
    a = 2 * np.arange(m * k).reshape(m, k) / (m * k)
    b = np.arange(n * k).reshape(k, n) / (n * k)
    out = np.zeros((m, n))
    dot(a, b, out, (8, 8))
    if blocked:
        # K-blocked accumulation rounds in a different order than one np.dot
        assert_allclose(out, np.dot(a, b), rtol=1e-13)
        ref = sum(np.dot(a[:, s:s + 16], b[s:s + 16, :]) for s in range(0, k, 16))
        assert_equal(out, ref)
    else:
        assert_equal(out, np.dot(a, b))


def test_softmax_rows_ragged_groups():
    M, N, GM, MI = sym.M, sym.N, sym.GM, sym.MI

    @kernel(work_shape=cdiv(M, MI), group_shape=GM, tunables=TunableParam(MI, 1, range(1, 8)))
    def softmax(gr: CurrentGroup, a: Buffer[M, N, DT], out: Buffer[M, N, DT], g: GM):
        m0, mb = gr.work_offset[0] * MI, gr.shape[0] * MI
        v = gr.load(a[m0:, :], shape=(mb, N))
        e = np.exp(v - v.max(axis=1, keepdims=True))
        gr.store(out[m0:, :], e / e.sum(axis=1, keepdims=True))

    m, n = 30, 25
    a = 2 * np.arange(m * n).reshape(m, n) / (m * n)
    out = np.zeros((m, n))
    softmax(a, out, 8)
    e = np.exp(a - a.max(axis=1, keepdims=True))
    assert_equal(out, e / e.sum(axis=1, keepdims=True))


def test_pairwise_distance():
    M, N, D, GM, GN, MI, NI = (sym.M, sym.N, sym.D, sym.GM, sym.GN, sym.MI, sym.NI)
    tun = (TunableParam(MI, 1, range(1, 8)), TunableParam(NI, 1, range(1, 8)))

    @kernel(work_shape=(cdiv(M, MI), cdiv(N, NI)), group_shape=(GM, GN), tunables=tun)
    def pw(gr: CurrentGroup, a: Buffer[M, D, DT], b: Buffer[N, D, DT],
           out: Buffer[M, N, DT], g: (GM, GN)):
        m0, n0 = gr.work_offset[0] * MI, gr.work_offset[1] * NI
        av = gr.load(a[m0:, :], shape=(gr.shape[0] * MI, D))
        bv = gr.load(b[n0:, :], shape=(gr.shape[1] * NI, D))
        gr.store(out[m0:, n0:], np.linalg.norm(av[:, None, :] - bv[None, :, :], axis=2))

    m, n, d = 16, 32, 8
    a = 2 * np.arange(m * d).reshape(m, d) / (m * d)
    b = np.arange(n * d).reshape(n, d) / (n * d)
    out = np.zeros((m, n))
    pw(a, b, out, (8, 8))
    assert_equal(out, np.linalg.norm(a[:, None, :] - b[None, :, :], axis=2))


@pytest.mark.parametrize("n,c,nf,stride", [(1, 1, 1, 1), (2, 3, 2, 2), (4, 3, 8, 3), (2, 1, 8, 1)])
def test_implicit_gemm_convolution(n, c, nf, stride):
    rng = np.random.default_rng(11)
    h = w = 4
    hf = wf = 2
    x = rng.standard_normal((n, c, h, w))
    f = rng.standard_normal((nf, c, hf, wf))
    ho = (h - hf) // stride + 1
    wo = (w - wf) // stride + 1
    ref = np.zeros((n, nf, ho, wo))
    for i, o, p, q in product(range(n), range(nf), range(ho), range(wo)):
        ref[i, o, p, q] = np.sum(x[i, :, p * stride:p * stride + hf,
                                   q * stride:q * stride + wf] * f[o])

    N, C, H, W, NF, HF, WF, KB = (sym.N, sym.C, sym.H, sym.W, sym.NF, sym.HF,
                                  sym.WF, sym.KB)
    TN, TNF = sym.TN, sym.TNF
    HO = (H - HF) / stride + 1
    WO = (W - WF) / stride + 1
    SZ = HF * WF * C
    KI = cdiv(SZ, KB)
    tun = (TunableParam(TN, 8, range(1, 64)), TunableParam(TNF, 8, range(1, 64)),
           TunableParam(KB, 16, range(8, 128)))
    x_map = create_mapping(lambda i, j: (i, j // (HF * WF), (j % (HF * WF)) % WF,
                                         (j % (HF * WF)) // WF))
    f_map = create_mapping(lambda i, j: (j, i // (HF * WF), i % WF, (i % (HF * WF)) // WF))
    o_map = create_mapping(lambda i, j: (i, j, 0, 0))

    @kernel(work_shape=(N, NF, HO * WO), group_shape=(TN, TNF, 1), tunables=tun)
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

    out = np.zeros_like(ref)
    conv(x, f, out)
    assert_allclose(out, ref)
