"""The programs the binder emits for the general float map and for row programs,
run on the CPU by NumPy restatements of the kernels' rules (tests/fmap_emulator.py,
run_row_stages of tests/test_kernel_frontend.py), against the host executor, on
random bodies (tests/random_bodies.py).  This checks the
front-end and the binder (which arithmetic a node means, which flags an
instruction carries, operand order) without a GPU; that the kernel follows the
same rules is checked on the GPU, by the same bodies among others."""

import warnings

import numpy as np
import pytest

from hckernel.kernel import *          # noqa: F401,F403
from hc_amd import runtime as rt
from hc_amd.binding import NoNativeKernel
from oracle.hcsim import kernel as sim_kernel

import random_bodies
from fmap_emulator import run_fmap
from test_kernel_frontend import (FakeDev, MapTablesOnly, POISON, ctx, fmap_program,   # noqa: F401  (ctx: a fixture)
                                  row_stages, run_row_stages)
from hc_amd.kernel_api import TraceError

DT = typename.DT
N, M = sym.N, sym.M
SEEDS = 2500


def bodies(fn):
    def one_d(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], c: Buffer[N, DT], out: Buffer[N, DT]):
        o = gr.work_offset[0]
        gr.store(out[o:], fn(*(gr.load(v[o:], shape=gr.shape) for v in (a, b, c))))

    def two_d(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], c: Buffer[M, N, DT],
              out: Buffer[M, N, DT]):
        i, j = gr.work_offset
        gr.store(out[i:, j:], fn(*(gr.load(v[i:, j:], shape=gr.shape) for v in (a, b, c))))
    return (one_d, dict(work_shape=N, group_shape=256)), (two_d, dict(work_shape=(M, N), group_shape=(4, 64)))


def test_random_bodies_mean_what_the_simulator_computes(ctx, monkeypatch):
    monkeypatch.setattr(rt, "GatherMap", MapTablesOnly)
    tally = {"ok": 0, "refused": 0, "both raise": 0, "another kernel": 0}
    for seed in range(SEEDS):
        fn, text, dtype, vals, shape = random_bodies.case(seed)
        body, deco = bodies(fn)[len(shape) - 1]
        want = np.full(shape, 7.5, dtype)
        sim_raises = False
        try:
            with np.errstate(all="ignore"), warnings.catch_warnings():
                warnings.simplefilter("ignore")
                sim_kernel(**deco)(body)(*vals, want)
        except TypeError:                      # a NumPy scalar or plain array on the left of a tile
            sim_raises = True
        devs = [FakeDev(shape, np.dtype(dtype).name) for _ in range(4)]
        try:
            (p,) = kernel(**deco)(body).plan(*devs, ctx=ctx)
        except NoNativeKernel:
            tally["refused"] += 1
            continue
        except TypeError:
            assert sim_raises, f"seed {seed}: {text}: only the front-end raises TypeError"
            tally["both raise"] += 1
            continue
        assert not sim_raises, f"seed {seed}: {text}: only the simulator raises TypeError"
        if p.fn is not rt.hcamdLaunchFMap:
            tally["another kernel"] += 1
            continue
        by_ptr = {d.ptr: v for d, v in zip(devs, vals)}
        got = np.full(shape, 7.5, dtype)
        run_fmap(fmap_program(p), [by_ptr[p.args[3][i]] for i in range(p.args[6])], p.args[-1], got)
        diff = random_bodies.difference(got, want, text)
        assert diff is None, f"seed {seed}: {text} ({np.dtype(dtype).name}): {diff}\n{fmap_program(p)}"
        tally["ok"] += 1
    assert tally["ok"] > SEEDS // 3, tally


ROW_SEEDS = 800


def row_body(deco, fn, per_row):
    GM = sym.GM
    if per_row:
        @deco(work_shape=M, group_shape=GM)
        def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, DT], g: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            gr.store(out[m0:], fn(gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N))))
    else:
        @deco(work_shape=M, group_shape=GM)
        def k(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, N, DT], g: GM):
            m0, mb = gr.work_offset[0], gr.shape[0]
            gr.store(out[m0:, :], fn(gr.load(a[m0:, :], shape=(mb, N)), gr.load(b[m0:, :], shape=(mb, N))))
    return k


def test_random_row_bodies_mean_what_the_simulator_computes(ctx, monkeypatch):
    """Elementwise expressions of two tiles and of sums, maxima, minima, means,
    variances and standard deviations along their rows: the stages the binder
    emits, run in NumPy with the row kernel's rules, store the elements the
    simulator stores, NaN where it has NaN, and the same values to 1e-4 (sums
    are added up in another order)."""
    monkeypatch.setattr(rt, "GatherMap", MapTablesOnly)
    tally = {"ok": 0, "refused": 0, "another kernel": 0}
    for seed in range(ROW_SEEDS):
        fn, text, per_row, (a, b) = random_bodies.row_case(seed)
        shape = (a.shape[0],) if per_row else a.shape
        want = np.full(shape, POISON)
        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            row_body(sim_kernel, fn, per_row)(a, b, want, 4)
        fake = [FakeDev(a.shape, "float32"), FakeDev(b.shape, "float32"), FakeDev(shape, "float32")]
        try:
            plans = row_body(kernel, fn, per_row).plan(*fake, 4, ctx=ctx)
        except (NoNativeKernel, TraceError):
            tally["refused"] += 1
            continue
        if len(plans) != 1 or plans[0].fn is not rt.hcamdLaunchRowProgram:
            tally["another kernel"] += 1
            continue
        (p,) = plans
        by_ptr = {fake[0].ptr: a, fake[1].ptr: b}
        operands = [by_ptr[p.args[4][i]] for i in range(p.args[7])]
        with np.errstate(all="ignore"):
            got = run_row_stages(row_stages(p), operands, (), np.float32, init=np.full(shape, POISON))
        if got.shape != want.shape and got.ndim == 1 and (want[:, 1:] == POISON).all():
            want = want[:, 0]                  # a (rows, 1) value stored to the window: its first column
        where = f"seed {seed}: {text}\n{row_stages(p)}"
        np.testing.assert_array_equal(got == POISON, want == POISON, err_msg=where)
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want), err_msg=where)
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4, err_msg=where)
        tally["ok"] += 1
    assert tally["ok"] > ROW_SEEDS // 2, tally
