"""Host-only checks of the C ABI: the libraries load, export every symbol the
headers declare, embed gfx950 code objects that hold every kernel the launchers
name, and follow the reference's error behaviour for everything that can be
forced without a GPU (bad device descriptions, bad ranks, bad launch dims)."""

import ctypes as C
import os
import re

import numpy as np
import pytest

from hc_amd import py_runtime
from hc_amd import runtime as rt
from oracle import closed_forms as cf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:ol|hcgpu|hcamd|setGPU|enableFunc)\w*)\s*\(", text)))


def test_runtime_exports_every_declared_symbol():
    names = declared_functions("hc_amd_runtime.h")
    assert len(names) >= 40
    for n in ["olCreateDevice", "olReleaseDevice", "olCreateModule", "olReleaseModule",
              "olGetKernel", "olReleaseKernel", "olSuggestBlockSize", "olCreateQueue",
              "olReleaseQueue", "olSyncQueue", "olAllocDevice", "olDeallocDevice",
              "olLaunchKernel"]:          # the 13 functions a loader dlsym()s
        assert n in names
    for n in names:
        assert hasattr(py_runtime.runtime_lib, n), n


def test_measurement_entry_points_have_a_header_of_their_own_and_probes_stay_out_of_a_default_build():
    names = declared_functions("hc_amd_bench.h")
    assert set(names) == {"hcamdLaunchStream", "hcamdProbesBuilt"}
    assert not set(names) & set(declared_functions("hc_amd_runtime.h"))
    for n in names:
        assert hasattr(py_runtime.runtime_lib, n), n
    blob = C.string_at(*rt.builtin_modules()["gemm"])
    if rt.probes_built():
        assert b"hcamd_gemm_bf16_probe_mfma_only\x00" in blob
        return
    # a default build holds no kernel whose output is not the product, and
    # refuses the numbers that would select one
    assert b"hcamd_gemm_bf16_probe" not in blob
    for v in (17, 18, 19, 20, 21, 22, 26, 28, 29, 30, 31, 32, 33, 34):
        assert rt.hcamdSetVariant(b"gemm", v) == 1 and rt.hcamdSetThreadVariant(b"gemm", v) == 1
        with pytest.raises(rt.HcRuntimeError, match="--probes"):
            rt.set_variant("gemm", v)
    for v in (0, 7, 16, 23, 25, 27):
        assert rt.hcamdSetVariant(b"gemm", v) == 0
    rt.set_variant("gemm", 0)


def test_pyabi_exports_every_declared_symbol():
    names = declared_functions("hc_amd_pyabi.h")
    assert {"hcgpuConvertPyArray", "hcgpuConvertPyInt64", "hcgpuSetRuntimeSearchPaths"} <= set(names)
    for n in names:
        assert hasattr(py_runtime.pyabi_lib, n), n


def test_jit_symbol_table_has_the_reference_names():
    assert {"hcgpuConvertPyArray", "hcgpuGetKernel", "hcgpuSuggestBlockSize",
            "hcgpuLaunchKernel"} <= set(py_runtime.JIT_SYMBOLS)
    assert all(v > 0 for v in py_runtime.JIT_SYMBOLS.values())


def test_builtin_code_objects_are_gfx950_elf_and_hold_the_kernels():
    mods = rt.builtin_modules()
    assert set(mods) == {"copy", "elementwise", "map", "imap", "fmap", "distance", "gather", "softmax", "quantize", "gemm"}
    src = open(os.path.join(ROOT, "hc_amd", "csrc", "runtime.cpp")).read()
    wanted = set(re.findall(r'"(hcamd_[a-z0-9_]+)"', src))
    wanted = {w for w in wanted if not w.endswith("_")}       # prefixes built at run time
    if not rt.probes_built():                                 # measurement builds: only with --probes
        wanted = {w for w in wanted if not w.startswith("hcamd_gemm_bf16_probe_")}
    found = set()
    for name, (addr, n) in mods.items():
        blob = C.string_at(addr, n)
        assert blob[:4] == b"\x7fELF", name
        assert addr % 4096 == 0
        assert b"gfx950" in blob, name
        found |= {w for w in wanted if w.encode() + b"\x00" in blob}
    assert wanted - found == set(), wanted - found
    for suffix in ("b1", "b2", "b4", "b8", "b16"):
        blob = C.string_at(*mods["copy"])
        assert f"hcamd_copy2d_{suffix}".encode() in blob
        assert f"hcamd_copy2d_tiled_{suffix}".encode() in blob


@pytest.mark.parametrize("desc,message", [
    ("xyz:0", "Runtime not found: xyz"),
    ("cuda:0", "Runtime not found: cuda"),
    ("hip", "Invalid device desc: hip"),
    ("hip:abc", "Invalid device id"),
    ("hip:", "Invalid device id"),
    ("hip:-1", "Invalid device id"),
])
def test_bad_device_descriptions(desc, message):
    seen = []
    cb = rt.ERROR_CALLBACK(lambda ctx, sev, text: seen.append((sev, text.decode())))
    assert rt.olCreateDevice(desc.encode(), cb, None) is None
    assert seen == [(0, message)]
    with pytest.raises(rt.HcRuntimeError, match=re.escape(message)):
        rt.Context(desc)


def test_null_callback_is_allowed():
    assert rt.olCreateDevice(b"xyz:0", rt.ERROR_CALLBACK(0), None) is None


@pytest.mark.parametrize("global_sizes,block", [
    ((16_777_259,), (1024,)), ((8193, 8191), (1024, 1)), ((27, 1), (27, 1)),
    ((64, 256), (64, 16)), ((813, 111), (813, 1)), ((100, 100, 100), (100, 8, 1)),
    ((1, 4096, 2), (1, 1024, 1)), ((1, 1, 1), (1, 1, 1)),
])
def test_suggest_block_size_matches_the_oracle(global_sizes, block):
    n = len(global_sizes)
    g = (C.c_size_t * n)(*global_sizes)
    b = (C.c_size_t * n)()
    assert rt.olSuggestBlockSize(None, g, b, n) == 0
    assert tuple(b) == block == cf.suggest_block_size(global_sizes)
    b2 = (C.c_size_t * n)()
    rt.hcgpuSuggestBlockSize(None, g, b2, n)
    assert tuple(b2) == block


def test_suggest_block_size_random_against_oracle():
    rng = np.random.default_rng(3)
    for _ in range(500):
        n = int(rng.integers(1, 4))
        sizes = tuple(int(v) for v in rng.choice([1, 2, 3, 7, 16, 27, 64, 100, 813, 1024, 1025, 10 ** 6], n))
        g = (C.c_size_t * n)(*sizes)
        b = (C.c_size_t * n)()
        assert rt.olSuggestBlockSize(None, g, b, n) == 0
        assert tuple(b) == cf.suggest_block_size(sizes)


def test_suggest_block_size_bad_rank_returns_one():
    g = (C.c_size_t * 4)(1, 2, 3, 4)
    b = (C.c_size_t * 4)()
    assert rt.olSuggestBlockSize(None, g, b, 0) == 1
    assert rt.olSuggestBlockSize(None, g, b, 4) == 1


def test_convert_numpy_array_to_memref():
    a = np.arange(24, dtype=np.int32).reshape(4, 6)
    m = rt.as_memref(a)
    assert (m.ptr, m.shape, m.strides, m.itemsize) == (a.ctypes.data, (4, 6), (6, 1), 4)
    v = a[1:, ::2]                       # offset + non-unit stride, in elements
    m = rt.as_memref(v)
    assert (m.ptr, m.shape, m.strides) == (v.ctypes.data, (3, 3), (6, 2))
    assert not m.is_contiguous()
    h = np.zeros((3, 5), np.float16)
    assert rt.as_memref(h).itemsize == 2
    m1 = rt.as_memref(np.zeros(7, np.float64))
    assert (m1.shape, m1.strides, m1.itemsize) == ((7,), (1,), 8)


def test_convert_rank_mismatch_reports_invalid_rank():
    with pytest.raises(rt.HcRuntimeError, match="Invalid rank"):
        rt.as_memref(np.zeros((2, 3)), rank=1)
    with pytest.raises(rt.HcRuntimeError, match="not an array"):
        rt.as_memref(object(), rank=1)


def test_convert_cuda_array_interface_objects():
    class Fake:
        def __init__(self, strides):
            self.shape = (3, 4)
            self.__cuda_array_interface__ = {
                "shape": (3, 4), "typestr": "<f2", "data": (0x7F0000001000, False),
                "strides": strides, "version": 2}

    m = rt.as_memref(Fake(None))
    assert (m.ptr, m.shape, m.strides, m.itemsize) == (0x7F0000001000, (3, 4), (4, 1), 2)
    m = rt.as_memref(Fake((16, 2)))
    assert m.strides == (8, 1)
    with pytest.raises(rt.HcRuntimeError, match="multiple of the element size"):
        rt.as_memref(Fake((15, 2)))


def test_strided_1d_operands_are_not_taken_for_dense():
    # a view like x[::2], or a column passed as a vector: the dense kernels would
    # read and write the wrong elements
    class Fake:
        def __init__(self, n, stride_bytes):
            self.shape = (n,)
            self.__cuda_array_interface__ = {
                "shape": (n,), "typestr": "<f4", "data": (0x7F0000001000, False),
                "strides": (stride_bytes,), "version": 2}

    assert rt._rows_cols(rt.as_memref(Fake(8, 4))) == (1, 8, 8)
    assert rt._rows_cols(rt.Memref(0x1000, (1,), (7,), 4)) == (1, 1, 1)
    for m in (rt.as_memref(Fake(8, 8)), rt.Memref(0x1000, (8,), (2,), 4)):
        with pytest.raises(rt.HcRuntimeError, match="contiguous"):
            rt._rows_cols(m)


def test_convert_torch_cpu_tensor_via_dlpack():
    torch = pytest.importorskip("torch")
    t = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    m = rt.as_memref(t)
    assert (m.ptr, m.shape, m.strides, m.itemsize) == (t.data_ptr(), (3, 4), (4, 1), 4)
    tt = t.t()
    assert rt.as_memref(tt).strides == (1, 4)
    b = torch.zeros(5, dtype=torch.bfloat16)
    assert rt.as_memref(b).itemsize == 2


def test_convert_int64():
    out = C.c_int64()
    err = C.create_string_buffer(128)
    assert rt.hcamdConvertPyInt64(-(2 ** 40), C.byref(out), err, 128) == 0
    assert out.value == -(2 ** 40)
    assert rt.hcamdConvertPyInt64(np.int32(7), C.byref(out), err, 128) == 0 and out.value == 7
    assert rt.hcamdConvertPyInt64("x", C.byref(out), err, 128) == 1 and err.value
    assert rt.hcamdConvertPyInt64(2 ** 70, C.byref(out), err, 128) == 1


def test_reference_layout_convert_entry_points():
    # hcgpuConvertPyArray writes its message into a C++ std::string; exercise it
    # through a tiny descriptor of the right size and a matching rank only
    desc = (C.c_int64 * 7)()
    fn = py_runtime.pyabi_lib.hcgpuConvertPyArray
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.py_object, C.c_int, C.c_void_p]
    a = np.zeros((2, 5), np.int32)
    assert fn(None, a, 2, C.cast(desc, C.c_void_p)) == 0
    assert list(desc) == [a.ctypes.data, a.ctypes.data, 0, 2, 5, 5, 1]
    assert fn(None, a, 3, C.cast(desc, C.c_void_p)) == 1     # null desc: code only


def test_variant_selection_rejects_unknown_family():
    rt.set_variant("gemm", 0)
    with pytest.raises(rt.HcRuntimeError):
        rt.set_variant("nosuch", 1)


def test_tracing_prints_enter_exit(capfd):
    py_runtime.enable_func_tracing(1, loader=True)
    try:
        g = (C.c_size_t * 1)(27)
        b = (C.c_size_t * 1)()
        rt.hcgpuSuggestBlockSize(None, g, b, 1)
    finally:
        py_runtime.enable_func_tracing(0, loader=True)
    out = capfd.readouterr().out.splitlines()
    assert out == ["hcgpuSuggestBlockSize enter", "olSuggestBlockSize enter",
                   "olSuggestBlockSize exit", "hcgpuSuggestBlockSize exit"]
    rt.hcgpuSuggestBlockSize(None, g, b, 1)
    assert capfd.readouterr().out == ""


def test_no_gpu_means_loud_failure_not_fallback():
    """Without a device the context cannot be created and nothing computes."""
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    with pytest.raises(rt.HcRuntimeError, match="failed with"):
        rt.Context("hip:0")


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "hc_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", ".S")):
                text = open(os.path.join(base, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), f
                assert "liboracle" not in text, f


def test_package_face_leaves_the_simulator_to_the_next_hckernel_on_the_path(tmp_path):
    """`hckernel/` defines the GPU decorator and the runtime face only; a module it
    does not define (the reference's kernel_sim, and the kernel_api that module
    imports relatively) comes from the next `hckernel` directory on the path.
    (A stand-in directory plays the reference's package here.)"""
    import subprocess
    import sys
    other = tmp_path / "elsewhere" / "hckernel"
    other.mkdir(parents=True)
    (other / "__init__.py").write_text("")
    (other / "kernel_api.py").write_text("WHOSE = 'the other package'\n")
    (other / "kernel_sim.py").write_text("from .kernel_api import WHOSE\n")
    (other / "kernel.py").write_text("WHOSE = 'shadowed'\n")
    code = ("import hckernel.kernel as k, hckernel.kernel_sim as s, hckernel.py_runtime as p\n"
            "import hc_amd.kernel, hc_amd.py_runtime\n"
            "assert k.kernel is hc_amd.kernel.kernel and p.runtime_lib is hc_amd.py_runtime.runtime_lib\n"
            "assert s.WHOSE == 'the other package', s.__file__\n"
            "import sys; assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules)\n")
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([ROOT, str(other.parent)]))
    done = subprocess.run([sys.executable, "-B", "-c", code], env=env, cwd=str(tmp_path),
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
