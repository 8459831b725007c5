"""hcamdLaunchMapReduceColsNoAlloc (the entry point that allocates no device
memory) against hcamdLaunchMapReduceCols with a caller-owned workspace: same
kernels, same fixed order of additions, so the results are equal bit for bit.
Two calls in a row share the library's static scratch array; the second is
smaller, so stale band results of the first lie behind the ones it uses."""
import sys

import numpy as np
import pytest

from hc_amd import runtime as rt

pytestmark = pytest.mark.gpu


def I(name, arg=0, imm=0.0):
    return (name, arg, imm)


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _both(kind, program, post, x_host):
    """Runs the plan with a workspace and the same arguments through the
    entry point without one; returns (with workspace, without) as bit patterns."""
    rows, cols = x_host.shape
    x = rt.to_device(x_host)
    want = rt.DeviceArray((cols,), np.float32).fill_bytes32(0xA5A5A5A5)
    got = rt.DeviceArray((cols,), np.float32).fill_bytes32(0x5A5A5A5A)
    plan = rt.plan_map_reduce_cols(kind, program, [x], want, post=post)
    plan.launch(sync=True)
    a = list(plan.args)
    out_at = a.index(want.ptr)
    a[out_at] = got.ptr
    noalloc = rt.Plan(plan.ctx, rt.hcamdLaunchMapReduceColsNoAlloc, tuple(a[:-2]),
                      "hcamdLaunchMapReduceColsNoAlloc", plan.keep + (got,))
    noalloc.launch(sync=True)
    return want.to_host().view(np.uint32), got.to_host().view(np.uint32), a[-1]


def test_two_calls_in_a_row_equal_the_workspace_entry_point():
    rng = np.random.default_rng(23)
    # tall and narrow: cut into bands, so the scratch array is really used
    big = rng.standard_normal((200_000, 24)).astype(np.float32)
    small = rng.standard_normal((70_001, 9)).astype(np.float32)
    for tag, x, kind, prog, post in [
            ("first, 200000 x 24 mean of squares", big, "sum",
             [I("in", 0), I("mul_in", 0)], [I("in", 0), I("divi", 0, float(big.shape[0]))]),
            ("second, 70001 x 9 maximum", small, "max", [I("in", 0)], [])]:
        say("no-alloc column reduction:", tag)
        want, got, need = _both(kind, prog, post, x)
        assert 0 < need <= rt.NOALLOC_SCRATCH_BYTES, need
        assert np.array_equal(want, got), tag
        ref = (x.astype(np.float64) ** 2).mean(axis=0) if kind == "sum" else x.max(axis=0)
        assert np.allclose(got.view(np.float32), ref, rtol=1e-5)


def test_launches_leave_the_free_device_memory_as_it_is():
    """The entry point allocates nothing: the free device memory the HIP runtime
    reports is the same before and after its launches, under every variant of the
    column-reduction kernels (their kernels are all resolved when the device is
    created, so no code object is loaded on the way either)."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    rng = np.random.default_rng(25)
    x_host = rng.standard_normal((150_000, 256)).astype(np.float32)
    x = rt.to_device(x_host)
    out = rt.DeviceArray((256,), np.float32)
    plan = rt.plan_map_reduce_cols("sum", [I("in", 0), I("mul_in", 0)], [x], out)
    noalloc = rt.Plan(plan.ctx, rt.hcamdLaunchMapReduceColsNoAlloc, tuple(plan.args[:-2]),
                      "hcamdLaunchMapReduceColsNoAlloc", plan.keep)
    plan.ctx.synchronize()
    try:
        for variant in (0, 1, 2):
            rt.set_variant("cols", variant)
            say("no-alloc column reduction: free memory around launches, cols variant", variant)
            before = free_bytes()
            for _ in range(3):
                noalloc.launch(sync=True)
            assert free_bytes() == before, variant
            ref = (x_host.astype(np.float64) ** 2).sum(axis=0)
            assert np.allclose(out.to_host(), ref, rtol=1e-5)
    finally:
        rt.set_variant("cols", 0)


def test_one_launch_windows_and_refusals():
    rng = np.random.default_rng(24)
    x = rng.standard_normal((64, 1000)).astype(np.float32)      # no bands: scratch unused
    say("no-alloc column reduction: 64 x 1000 sum, one launch")
    want, got, need = _both("sum", [I("in", 0)], [], x)
    assert need == 0 and np.array_equal(want, got)
    # errors come back as codes and messages, as from the other entry point
    out = rt.DeviceArray((8,), np.float32)
    xs = rt.to_device(np.ones((8, 8), np.float32))
    plan = rt.plan_map_reduce_cols("sum", [I("in", 0), I("in", 0)], [xs], out)
    bad = rt.Plan(plan.ctx, rt.hcamdLaunchMapReduceColsNoAlloc, tuple(plan.args[:-2]),
                  "hcamdLaunchMapReduceColsNoAlloc", plan.keep)
    with pytest.raises(rt.HcRuntimeError, match="leaves 2 values"):
        bad.launch(sync=True)
