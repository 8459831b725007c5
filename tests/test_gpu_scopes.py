"""Subgroup and work-item scopes on the GPU against the host executor
(oracle.hcsim) running the same body: the id / size / barrier cases of
python/hckernel/tests/test_kernel_sim.py:229-379 expressed as stores of ids into
buffers, per-work-item elementwise statements, and row reductions written with
explicit per-subgroup partial results and barriers."""
import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_array_equal

from hckernel.kernel import *          # noqa: F401,F403
from hc_amd import runtime as rt
from oracle import closed_forms as cf
from oracle.hcsim import kernel as sim_kernel

pytestmark = pytest.mark.gpu
DT = typename.DT
POISON = -7


def both(decorate_args, body, gpu_args, host_args):
    """Runs `body` through the GPU front-end and through the host executor."""
    kernel(**decorate_args)(body)(*gpu_args)
    sim_kernel(**decorate_args)(body)(*host_args)


@pytest.mark.parametrize("work,group", [((1, 1, 16), (1, 1, 8)), ((1, 1, 4), (1, 1, 2)),
                                        ((2, 3, 32), (1, 3, 16)), ((4, 1, 64), (2, 1, 64))])
def test_workitem_ids_stored_to_buffers(work, group):
    G1, G2, G3, L1, L2, L3 = sym.G1, sym.G2, sym.G3, sym.L1, sym.L2, sym.L3

    def body(gr: CurrentGroup, g: tuple[G1, G2, G3], l: tuple[L1, L2, L3], lid0, lid2, gid2, mix):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            i, j, k = wi.global_id()
            a, b, c = wi.local_id()
            lid0[i, j, k] = a
            lid2[i, j, k] = c
            gr.barrier()
            gid2[i, j, k] = k
            mix[i, j, k] = 1000 * i + 100 * j + k - c      # ids combined affinely

        inner()

    host = [np.full(work, POISON, np.int32) for _ in range(3)] + [np.full(work, POISON, np.int64)]
    devs = [rt.to_device(h) for h in host]
    both(dict(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3)), body,
         (work, group, *devs), (work, group, *host))
    for d, h in zip(devs, host):
        assert (h != POISON).all()
        assert_array_equal(d.to_host(), h)
    if work == (1, 1, 4):          # test_kernel_sim.py:343-344
        assert host[1].ravel().tolist() == [0, 1, 0, 1] and host[2].ravel().tolist() == [0, 1, 2, 3]


@pytest.mark.parametrize("sgsize", [4, 2])
def test_subgroup_ids_sizes_and_barrier_phases(sgsize):
    """test_kernel_sim.py:229-320: 16 work-items in groups of 8, subgroups of 4:
    ids (0,0,0), (0,0,1) per group, size 4; phase 2 of every subgroup follows
    phase 1 of all subgroups of the group."""
    G1, G2, G3, L1, L2, L3 = sym.G1, sym.G2, sym.G3, sym.L1, sym.L2, sym.L3
    work, group = (1, 1, 16), (1, 1, 8)
    nsub = group[2] // sgsize
    phases = []

    def body(gr: CurrentGroup, g: tuple[G1, G2, G3], l: tuple[L1, L2, L3], ids, sizes, order):
        @gr.subgroups
        def inner(sg: CurrentSubGroup):
            k = sg.subgroup_id()[2]
            slot = gr.id[2] * nsub + k
            ids[slot] = k
            sizes[slot] = sg.size()
            phases.append((1, sg.subgroup_id()))
            gr.barrier()
            phases.append((2, sg.subgroup_id()))
            order[slot] = 10 * gr.id[2] + k              # written in phase 2

        inner()

    n = (work[2] // group[2]) * nsub
    host = [np.full(n, POISON, np.int32) for _ in range(3)]
    devs = [rt.to_device(h) for h in host]
    kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=sgsize)(body)(
        work, group, *devs)
    traced = list(phases)
    phases.clear()
    sim_kernel(work_shape=(G1, G2, G3), group_shape=(L1, L2, L3), subgroup_size=sgsize)(body)(
        work, group, *host)
    for d, h in zip(devs, host):
        assert_array_equal(d.to_host(), h)
    assert host[0].tolist() == list(range(nsub)) * 2 and (host[1] == sgsize).all()
    # one traced pass sees the phase order the simulator sees in every group
    one_group = [(p, (0, 0, k)) for p in (1, 2) for k in range(nsub)]
    assert traced == one_group and phases == one_group * 2


def test_workitem_elementwise_statements_same_body_both_sides():
    N = sym.N

    def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT]):
        @gr.workitems
        def inner(wi: CurrentWorkitem):
            i = wi.global_id()
            c[i] = a[i] * b[i] + a[i]

        inner()

    n = 64 * 300
    a, b = cf.inputs_c1(n)
    dc = rt.DeviceArray((n,), np.float32)
    hc = np.zeros(n, np.float32)
    both(dict(work_shape=N, group_shape=64), body, (rt.to_device(a), rt.to_device(b), dc), (a, b, hc))
    assert_array_equal(dc.to_host().view(np.uint32), hc.view(np.uint32))


def _softmax_sg(rows_per_group, lanes, sg):
    ROWS, N = sym.ROWS, sym.N

    def body(gr: CurrentGroup, x: Buffer[ROWS, N, DT], y: Buffer[ROWS, N, DT]):
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

    return dict(work_shape=(ROWS, lanes), group_shape=(rows_per_group, lanes), subgroup_size=sg), body


@pytest.mark.parametrize("rows,cols,rpg,lanes,sg", [(64, 8192, 1, 256, 64), (30, 1024, 2, 256, 64),
                                                     (16, 4096, 1, 128, 16)])
def test_softmax_with_subgroup_partials_and_barriers(rows, cols, rpg, lanes, sg):
    deco, body = _softmax_sg(rpg, lanes, sg)
    (x,) = cf.inputs_c3((rows, cols))
    dy = rt.DeviceArray(x.shape, np.float32)
    hy = np.zeros_like(x)
    both(deco, body, (rt.to_device(x), dy), (x, hy))
    assert rt.last_kernel_name().startswith("hcamd_softmax_f32")
    assert_allclose(dy.to_host(), hy, rtol=1e-5, atol=1e-9)
    assert_allclose(hy, cf.np_softmax(x), rtol=1e-5, atol=1e-9)


def test_row_absmax_quantize_with_subgroup_partials_bit_exact():
    ROWS, N = sym.ROWS, sym.N
    f = np.float32

    def body(gr: CurrentGroup, x: Buffer[ROWS, N, DT], q: Buffer[ROWS, N, DT], scale: Buffer[ROWS, DT]):
        r0 = gr.work_offset[0]
        n = x.shape[1]
        nsub = gr.shape[1] // 64
        seg = n // nsub
        xf = gr.load(x[r0:], shape=(1, n)).astype(f)
        mag = np.abs(xf)
        part = gr.zeros((1, nsub), f)

        @gr.subgroups
        def absmax(s: CurrentSubGroup):
            i, k = s.subgroup_id()
            part[i, k] = mag[i, k * seg:(k + 1) * seg].max()

        absmax()
        gr.barrier()
        sc = part.max(axis=1, keepdims=True) / f(127)
        gr.store(q[r0:], np.clip(np.rint(xf / sc), -127, 127).astype(np.int8))
        gr.store(scale[r0:], sc[:, 0])

    (x,) = cf.inputs_c4((96, 4096))
    dq, ds = rt.DeviceArray(x.shape, np.int8), rt.DeviceArray((96,), np.float32)
    hq, hs = np.zeros(x.shape, np.int8), np.zeros(96, np.float32)
    both(dict(work_shape=(ROWS, 256), group_shape=(1, 256), subgroup_size=64), body,
         (rt.to_device(x), dq, ds), (x, hq, hs))
    assert rt.last_kernel_name().startswith("hcamd_quant_f16_i8")
    q_np, s_np = cf.np_quantize(x)
    assert_array_equal(hq, q_np)
    assert_array_equal(dq.to_host(), hq)
    assert_array_equal(ds.to_host().view(np.uint32), hs.view(np.uint32))
