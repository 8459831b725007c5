"""The committed vectors of tests/golden/workloads_small.npz (written by
tests/golden/make_golden.py): the CPU oracle must still reproduce them
(no GPU needed), and the GPU kernels must match them to each workload's bar."""

import os

import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_array_equal

from oracle import c_oracle as co
from oracle import closed_forms as cf

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "workloads_small.npz")


@pytest.fixture(scope="module")
def g():
    return np.load(GOLDEN)          # plain arrays only, no pickles


def test_oracle_reproduces_the_committed_vectors(g):
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "make_golden", os.path.join(os.path.dirname(GOLDEN), "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    assert set(fresh) == set(g.files)
    for name in g.files:
        a, b = fresh[name], g[name]
        assert a.dtype == b.dtype and a.shape == b.shape, name
        if name in ("c3_out", "c5_out_f32acc"):         # libm exp / BLAS summation order
            assert_allclose(a, b, rtol=1e-6, atol=1e-9, err_msg=name)
        else:
            assert_array_equal(a.view(np.uint8), b.view(np.uint8), err_msg=name)


def test_c_statement_against_the_committed_vectors(g):
    assert_array_equal(co.add_f32(g["c1_a"], g["c1_b"]).view(np.uint32), g["c1_out"].view(np.uint32))
    assert_array_equal(co.fma_f16(g["c2_a"], g["c2_b"], g["c2_c"]).view(np.uint16),
                       g["c2_out"].view(np.uint16))
    assert_allclose(co.softmax(g["c3_x"]), g["c3_out"], rtol=1e-5, atol=1e-9)
    q, s = co.quantize(g["c4_x"])
    assert_array_equal(q, g["c4_q"])
    assert_array_equal(s.view(np.uint32), g["c4_scale"].view(np.uint32))
    _, c32 = co.gemm_bf16(g["c5_a"], g["c5_bt"])
    assert_allclose(c32, g["c5_out_f32acc"], rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_gpu_kernels_against_the_committed_vectors(g):
    from hc_amd import runtime as rt
    d = rt.to_device
    out = rt.DeviceArray(g["c1_out"].shape, np.float32)
    rt.plan_add_f32(d(g["c1_a"]), d(g["c1_b"]), out).launch(sync=True)
    assert_array_equal(out.to_host().view(np.uint32), g["c1_out"].view(np.uint32))
    out = rt.DeviceArray(g["c2_out"].shape, np.float16)
    rt.plan_fma_f16(d(g["c2_a"]), d(g["c2_b"]), d(g["c2_c"]), out).launch(sync=True)
    assert_array_equal(out.to_host().view(np.uint16), g["c2_out"].view(np.uint16))
    out = rt.DeviceArray(g["c3_out"].shape, np.float32)
    rt.plan_softmax_f32(d(g["c3_x"]), out).launch(sync=True)
    assert_allclose(out.to_host(), g["c3_out"], rtol=1e-5, atol=1e-9)
    q = rt.DeviceArray(g["c4_q"].shape, np.int8)
    s = rt.DeviceArray(g["c4_scale"].shape, np.float32)
    rt.plan_quantize_f16_i8(d(g["c4_x"]), q, s).launch(sync=True)
    assert_array_equal(q.to_host(), g["c4_q"])
    assert_array_equal(s.to_host().view(np.uint32), g["c4_scale"].view(np.uint32))
    c = rt.DeviceArray(g["c5_out_f32acc"].shape, np.uint16, bf16=True)
    rt.plan_gemm_bf16(d(g["c5_a"], bf16=True), d(g["c5_bt"], bf16=True), c).launch(sync=True)
    sigma = 0.02 * 0.02 * np.sqrt(128)
    assert_allclose(cf.bf16_bits_to_f32(c.to_host()), g["c5_out_f32acc"], rtol=1e-2, atol=1e-2 * sigma)
