"""The programs the binder emits for the general float map, run on the CPU by a
NumPy restatement of the kernel's rules (tests/fmap_emulator.py), against the
host executor, on random bodies (tests/random_bodies.py).  This checks the
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
from test_kernel_frontend import FakeDev, MapTablesOnly, ctx, fmap_program   # noqa: F401  (ctx: a fixture)

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
