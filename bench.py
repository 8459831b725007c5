#!/usr/bin/env python3
"""Benchmark of the five hc_amd kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1..c5|all]

A "step" is one launch of a workload's kernel over its full synthetic input,
already resident in HBM.  Each workload cycles through ROTATE distinct buffer
sets so that consecutive launches never find their inputs in the 256 MiB
memory-side cache.  Timing: W warm-up launches, then exactly K launches between
two HIP events recorded on the stream the kernels run on, with a host
synchronisation and a wall clock around the same region.  Before the warm-up
steps each workload runs untimed for a fraction of a second so that the GPU's
clocks have settled.

Prints ONE JSON line.  The top-level metric is the fused fp16 elementwise
workload (d = a*b + c, 8191 x 8193); the `configs` object carries the same
fields for all five workloads, each with its roofline and its NumPy CPU
baseline timed on this machine's host cores in the same run.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published
# MI355X fp32 vector peak, published.  It counts packed fused multiply-adds; the
# pairwise kernel issues one subtract and one unpacked multiply-add per term
# (3 flop per 2 lane-instructions), so its own ceiling is well under this figure.
FP32_VECTOR_PEAK_TFLOPS = 157.3
ROTATE = 4
PREWARM_SECONDS = 0.4        # untimed, per workload, before the W warm-up steps

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE),
# scaled by a copy kernel of known size; filled in from profiles/*.txt.
# FETCH_SIZE reads half the true value on this device (a 256 MiB copy reads
# 131,082 KiB), WRITE_SIZE reads true (262,215 KiB), so fetches are scaled by
# 2.0 and writes by 1.0.  Source: profiles/hbm_traffic_pmc.txt.
_KIB = 1024
MEASURED_TRAFFIC = {
    "c0": int((131085.1 * 2.0 + 262156.5) * _KIB),
    "c1": int((65556.6 * 2.0 + 65536.2) * _KIB),     # algorithmic 201,327,108
    "c2": int((196637.6 * 2.0 + 131072.0) * _KIB),   # algorithmic 536,870,904
    "c3": int((65566.9 * 2.0 + 131125.1) * _KIB),    # algorithmic 268,435,456
    "c4": int((65869.6 * 2.0 + 66048.0) * _KIB),     # algorithmic 201,392,128
    "c5": int((98362.2 * 2.0 + 32768.0) * _KIB),     # 2.3 x the algorithmic 100,663,296 (L2 refetch)
    # both launches of the step: the bands (67,221.4 / 2,048.0) and their fold (1,177.5 / 32.0)
    "x6": int(((67221.4 + 1177.5) * 2.0 + 2048.0 + 32.0) * _KIB),   # algorithmic 134,250,496
}


# Stream calibrations: (key, read streams, what is written, MiB per read stream).
# The first four have the read:write mix and size of c1..c4 and are timed next
# to them in the default run.
STREAMS = [
    ("s1", 2, "full", 64),     # c1: two reads, one write of 64 MiB
    ("s2", 3, "full", 128),    # c2: three reads, one write of 128 MiB
    ("s3", 1, "full", 128),    # c3: 128 MiB each way
    ("s4", 1, "half", 128),    # c4: 128 MiB in, 64 MiB out
    ("s5", 1, "none", 256), ("s6", 0, "full", 256), ("s7", 1, "full", 256),
    ("s8", 2, "full", 128), ("s9", 2, "full", 256), ("s10", 3, "full", 256),
    ("s11", 1, "half", 256), ("s12", 1, "none", 128), ("s13", 0, "full", 128),
]
STREAM_OF = {"c1": "s1", "c2": "s2", "c3": "s3", "c4": "s4"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Workload:
    """name, algorithmic work, how to build device buffers, launch and check."""

    def __init__(self, key, title, kernel_dtype, bound, work, unit):
        self.key, self.title, self.dtype = key, title, kernel_dtype
        self.bound, self.work, self.unit = bound, work, unit

    def setup(self, rt):            # -> list of ROTATE argument tuples
        raise NotImplementedError

    def plan(self, rt, args):       # -> hc_amd.runtime.Plan (one foreign call per launch)
        raise NotImplementedError

    def check(self, rt, args):      # -> dict(parity=..., detail=...)
        raise NotImplementedError

    def cpu(self):                  # -> (seconds best-of-n, sample description, cores)
        raise NotImplementedError


def _best_of(fn, repeats=5):
    fn()
    best = float("inf")
    for _ in range(repeats):
        t = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t)
    return best


def _blas_threads():
    try:
        from threadpoolctl import threadpool_info
        return max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        return int(os.environ.get("OPENBLAS_NUM_THREADS", os.cpu_count() or 1))


def make_workloads(rt, wl):
    from hc_amd import workloads as W

    class C1(Workload):
        def setup(self, rt):
            self.a, self.b = W.inputs_c1()
            return [(rt.to_device(self.a), rt.to_device(self.b),
                     rt.DeviceArray(self.a.shape, np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_add_f32(s[0], s[1], s[2])

        def check(self, rt, s):
            from oracle import closed_forms as cf
            ok = np.array_equal(s[2].to_host().view(np.uint32),
                                cf.np_add(self.a, self.b).view(np.uint32))
            return {"parity": "bit-exact" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            from oracle import closed_forms as cf
            return _best_of(lambda: cf.np_add(self.a, self.b)), "full size, a + b", 1

    class C2(Workload):
        def setup(self, rt):
            self.a, self.b, self.c = W.inputs_c2()
            return [(rt.to_device(self.a), rt.to_device(self.b), rt.to_device(self.c),
                     rt.DeviceArray(self.a.shape, np.float16)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_fma_f16(s[0], s[1], s[2], s[3])

        def check(self, rt, s):
            from oracle import closed_forms as cf
            ok = np.array_equal(s[3].to_host().view(np.uint16),
                                cf.np_fma_f16(self.a, self.b, self.c).view(np.uint16))
            return {"parity": "bit-exact" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            from oracle import closed_forms as cf
            return (_best_of(lambda: cf.np_fma_f16(self.a, self.b, self.c), 3),
                    "full size, (a32*b32+c32).astype(f16)", 1)

    class C3(Workload):
        def setup(self, rt):
            (self.x,) = W.inputs_c3()
            return [(rt.to_device(self.x), rt.DeviceArray(self.x.shape, np.float32))
                    for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_softmax_f32(s[0], s[1])

        def check(self, rt, s):
            from oracle import closed_forms as cf
            y, want = s[1].to_host(), cf.np_softmax(self.x)
            ok = np.allclose(y, want, rtol=1e-5, atol=1e-9)
            rel = float(np.max(np.abs(y - want) / np.maximum(np.abs(want), 1e-30)))
            return {"parity": "rtol 1e-5" if ok else "MISMATCH", "ok": bool(ok),
                    "max_rel_err": rel}

        def cpu(self):
            from oracle import closed_forms as cf
            return _best_of(lambda: cf.np_softmax(self.x), 3), "full size, np_softmax", 1

    class C4(Workload):
        def setup(self, rt):
            (self.x,) = W.inputs_c4()
            return [(rt.to_device(self.x), rt.DeviceArray(self.x.shape, np.int8),
                     rt.DeviceArray((self.x.shape[0],), np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_quantize_f16_i8(s[0], s[1], s[2])

        def check(self, rt, s):
            from oracle import closed_forms as cf
            q, sc = cf.np_quantize(self.x)
            ok = (np.array_equal(s[1].to_host(), q) and
                  np.array_equal(s[2].to_host().view(np.uint32), sc.view(np.uint32)))
            return {"parity": "bit-exact" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            from oracle import closed_forms as cf
            return _best_of(lambda: cf.np_quantize(self.x), 3), "full size, np_quantize", 1

    class C5(Workload):
        def setup(self, rt):
            self.a, self.bt = W.inputs_c5()
            m, n = self.a.shape[0], self.bt.shape[0]
            return [(rt.to_device(self.a, bf16=True), rt.to_device(self.bt, bf16=True),
                     rt.DeviceArray((m, n), np.uint16, bf16=True)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_gemm_bf16(s[0], s[1], s[2])

        def check(self, rt, s):
            from oracle import closed_forms as cf
            got = W.bf16_bits_to_f32(s[2].to_host())
            want = cf.np_gemm_bf16(self.a, self.bt, np.float32)
            ok = np.allclose(got, want, rtol=1e-2, atol=2.6e-4)
            return {"parity": "rtol 1e-2 vs fp32 accumulation" if ok else "MISMATCH",
                    "ok": bool(ok), "max_abs_err": float(np.max(np.abs(got - want)))}

        def cpu(self):
            from oracle import closed_forms as cf
            t = _best_of(lambda: cf.np_gemm_bf16(self.a, self.bt, np.float32), 2)
            return t, "full size, OpenBLAS sgemm on bf16-rounded inputs", _blas_threads()

    class C0(Workload):
        """Plain copy of 256 MiB: the yardstick the hardware counters are scaled
        by, and the practical ceiling of a read-once / write-once stream."""

        def setup(self, rt):
            self.n = 64 * 1024 * 1024
            self.src = np.arange(self.n, dtype=np.int32)[None, :]
            return [(rt.to_device(self.src), rt.DeviceArray((1, self.n), np.int32))
                    for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_copy2d(s[0], s[1])

        def check(self, rt, s):
            ok = np.array_equal(s[1].to_host(), self.src)
            return {"parity": "bit-exact" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            dst = np.empty_like(self.src)
            return _best_of(lambda: np.copyto(dst, self.src)), "full size, numpy.copyto", 1


    class Stream(Workload):
        """Stream calibration: n_reads vectors of `mib` MiB added word by word and
        written whole ("full"), folded to half the bytes ("half") or only summed
        ("none"): what HBM delivers for that mix of reads and writes."""

        def __init__(self, key, n_reads, write, mib):
            self.n_reads, self.write, self.nbytes = n_reads, write, mib << 20
            out = {"full": self.nbytes, "half": self.nbytes // 2, "none": self.nbytes // 4096}[write]
            self.out_bytes = out
            mix = f"r{n_reads}w{0 if write == 'none' else 1}{'h' if write == 'half' else ''}"
            moved = n_reads * self.nbytes + (0 if write == "none" else out)
            super().__init__(key, f"stream {mix}: {n_reads} read stream(s) of {mib} MiB, "
                             f"{out >> 20} MiB written (calibration)", "u32", "hbm", moved, "GB/s")
            self.mix = mix

        def setup(self, rt):
            rng = np.random.default_rng(9)
            self.ins = [rng.integers(0, 2 ** 32, self.nbytes // 4, dtype=np.uint32)
                        for _ in range(self.n_reads)]
            return [tuple(rt.to_device(x) for x in self.ins) +
                    (rt.DeviceArray((self.out_bytes // 4,), np.uint32),) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_stream(s[:-1], s[-1], self.write)

        def _numpy(self):
            if not self.ins:
                return np.repeat(np.arange(self.nbytes // 16, dtype=np.uint32), 4)
            total = self.ins[0].copy()
            for x in self.ins[1:]:
                total += x
            if self.write == "full":
                return total
            if self.write == "half":
                return total[0::2] ^ total[1::2]
            return total.reshape(-1, 4096).sum(axis=1, dtype=np.uint32)

        def check(self, rt, s):
            ok = np.array_equal(s[-1].to_host(), self._numpy())
            return {"parity": "bit-exact" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(self._numpy, 1), "full size, NumPy uint32 arithmetic", 1

    # ---- beyond the five configurations: the generic paths, on request only ------
    I = lambda name, arg=0, imm=0.0: (name, arg, imm)      # noqa: E731

    class X1(C2):
        """a*b+c on the C2 arrays through the fused map kernel (3 instructions)."""

        def plan(self, rt, s):
            return rt.plan_map([I("in", 0), I("mul_in", 1), I("add_in", 2)], s[:3], s[3])

    class X2(Workload):
        """fp32 dot product of the C1 vectors through the map-sum kernel."""

        def setup(self, rt):
            self.a, self.b = W.inputs_c1()
            return [(rt.to_device(self.a), rt.to_device(self.b),
                     rt.to_device(np.zeros(1, np.float32))) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_map_sum([I("in", 0), I("mul_in", 1)], s[:2], s[2])

        def check(self, rt, s):
            cell = rt.to_device(np.zeros(1, np.float32))
            rt.plan_map_sum([I("in", 0), I("mul_in", 1)], s[:2], cell).launch(sync=True)
            prod = (self.a * self.b).astype(np.float64)
            err = abs(float(cell.to_host()[0]) - prod.sum())
            ok = err <= 64 * 2.0 ** -24 * np.abs(prod).sum()
            return {"parity": "|err| <= 64 * 2^-24 * sum|x|" if ok else "MISMATCH", "ok": bool(ok),
                    "abs_err": err}

        def cpu(self):
            return _best_of(lambda: np.dot(self.a, self.b)), "full size, numpy.dot", _blas_threads()

    class X3(Workload):
        """Pairwise distances of 8192 x 8192 points in 128 dimensions."""
        M = N = 8192
        D = 128

        def setup(self, rt):
            rng = np.random.default_rng(6)
            self.a = rng.standard_normal((self.M, self.D)).astype(np.float32)
            self.b = rng.standard_normal((self.N, self.D)).astype(np.float32)
            return [(rt.to_device(self.a), rt.to_device(self.b),
                     rt.DeviceArray((self.M, self.N), np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            return rt.plan_pairwise_dist_f32(s[0], s[1], s[2])

        def check(self, rt, s):
            got = s[2].to_host()[:256, :512]
            want = np.sqrt(((self.a[:256, None, :].astype(np.float64) - self.b[None, :512, :]) ** 2
                            ).sum(axis=2))
            ok = np.allclose(got, want, rtol=(self.D + 2) * 2.0 ** -24)
            return {"parity": "rtol (d+2) * 2^-24 vs fp64 (256 x 512 block)" if ok else "MISMATCH",
                    "ok": bool(ok)}

        def cpu(self):
            a, b = self.a[:512], self.b[:512]
            t = _best_of(lambda: np.linalg.norm(a[:, None, :] - b[None, :, :], axis=2), 2)
            return t * (self.M / 512) * (self.N / 512), "512 x 512 block scaled to full size", 1

    class X4(Workload):
        """3 x 3 convolution, NCHW fp32, written as the implicit-GEMM body of the
        reference's examples (one group = 64 images x 64 filters at one output
        position, operands gathered through index mappings) and launched
        through the @kernel front-end."""
        N, C, HW, NF, F = 64, 64, 58, 64, 3

        def setup(self, rt):
            from hc_amd.examples import convolution
            self.kernel = convolution(stride=1, tile=64, k_block=64)
            rng = np.random.default_rng(7)
            self.x = rng.standard_normal((self.N, self.C, self.HW, self.HW)).astype(np.float32)
            self.f = rng.standard_normal((self.NF, self.C, self.F, self.F)).astype(np.float32)
            ho = self.HW - self.F + 1
            return [(rt.to_device(self.x), rt.to_device(self.f),
                     rt.DeviceArray((self.N, self.NF, ho, ho), np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            (p,) = self.kernel.plan(*s)
            return p

        def _direct(self, x, f):
            ho = self.HW - self.F + 1
            out = np.zeros((x.shape[0], f.shape[0], ho, ho), np.float64)
            for p in range(ho):
                for q in range(ho):
                    out[:, :, p, q] = np.einsum("nchw,fchw->nf", x[:, :, p:p + self.F, q:q + self.F],
                                                f, optimize=True)
            return out

        def check(self, rt, s):
            got = s[2].to_host()[:2, :8]
            want = self._direct(self.x[:2].astype(np.float64), self.f[:8].astype(np.float64))
            k = self.C * self.F * self.F
            ok = np.allclose(got, want, rtol=1e-4, atol=(k + 2) * 2.0 ** -22)
            return {"parity": "rtol 1e-4, atol (k+2) * 2^-22 vs fp64 (2 images x 8 filters)"
                    if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            x, f = self.x[:4], self.f
            t = _best_of(lambda: self._direct(x, f), 1)
            return t * (self.N / 4), "4 of 64 images (einsum per output position), scaled", 1

    class X5(Workload):
        """Layer normalisation with weight and bias over the rows of the C3 matrix,
        written as a kernel body with mean and var along axis 1 and launched
        through the @kernel front-end (a five-stage row program)."""

        def setup(self, rt):
            from hc_amd.examples import layer_norm
            self.kernel = layer_norm()
            (self.x,) = W.inputs_c3()
            rng = np.random.default_rng(8)
            self.g = rng.standard_normal(self.x.shape[1]).astype(np.float32)
            self.b = rng.standard_normal(self.x.shape[1]).astype(np.float32)
            return [(rt.to_device(self.x), rt.to_device(self.g), rt.to_device(self.b),
                     rt.DeviceArray(self.x.shape, np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            (p,) = self.kernel.plan_rows(*s)
            return p

        def _numpy(self, x):
            m = x.mean(axis=1, keepdims=True)
            return (x - m) / np.sqrt(x.var(axis=1, keepdims=True) + x.dtype.type(1e-5)) * self.g + self.b

        def check(self, rt, s):
            got, want = s[3].to_host(), self._numpy(self.x.astype(np.float64))
            ok = np.allclose(got, want, rtol=2e-5, atol=2e-5)
            return {"parity": "rtol 2e-5, atol 2e-5 vs fp64" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(lambda: self._numpy(self.x), 2), "full size, NumPy fp32", 1

    class X6(Workload):
        """Root mean square down the columns of the C3 matrix, written as a kernel
        body with a mean along axis 0 of whole-column tiles and launched through
        the @kernel front-end (the column-reduction kernel, three levels)."""

        def setup(self, rt):
            from hc_amd.examples import column_rms
            self.kernel = column_rms()
            (self.x,) = W.inputs_c3()
            return [(rt.to_device(self.x), rt.DeviceArray((self.x.shape[1],), np.float32))
                    for _ in range(ROTATE)]

        def plan(self, rt, s):
            (p,) = self.kernel.plan_cols(*s)
            return p

        def _numpy(self, x):
            return np.sqrt((x * x).mean(axis=0) + x.dtype.type(1e-6))

        def check(self, rt, s):
            got, want = s[1].to_host(), self._numpy(self.x.astype(np.float64))
            ok = np.allclose(got, want, rtol=1e-5)
            return {"parity": "rtol 1e-5 vs fp64" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(lambda: self._numpy(self.x), 2), "full size, NumPy fp32", 1

    table = {
        "c0": C0("c0", "copy 256 MiB int32 (calibration)", "u32", "hbm", 2 * 4 * 64 * 1024 * 1024,
                 "GB/s"),
        "c1": C1("c1", "vadd fp32 N=16777259", "f32", "hbm", W.work_c1(), "GB/s"),
        "c2": C2("c2", "fma fp16 8191x8193 (fp32 math)", "f16", "hbm", W.work_c2(), "GB/s"),
        "c3": C3("c3", "row softmax fp32 4096x8192", "f32", "hbm", W.work_c3(), "GB/s"),
        "c4": C4("c4", "row absmax int8 quantize fp16 16384x4096", "f16->i8", "hbm",
                 W.work_c4(), "GB/s"),
        "c5": C5("c5", "GEMM bf16 4096^3 (fp32 acc)", "bf16", "mfma", W.work_c5(), "TFLOP/s"),
        "x1": X1("x1", "map kernel: fma fp16 8191x8193 as a 3-instruction program", "f16", "hbm",
                 W.work_c2(), "GB/s"),
        "x2": X2("x2", "map-sum kernel: dot fp32 N=16777259", "f32", "hbm", 8 * W.C1_N, "GB/s"),
        "x3": X3("x3", "pairwise distance fp32 8192x8192x128 (sub + fma per term)", "f32", "valu",
                 3 * 8192 * 8192 * 128, "TFLOP/s"),
        "x4": X4("x4", "implicit-GEMM convolution fp32 64x64x58x58 * 64x64x3x3 (gathered tiles)",
                 "f32", "valu", 2 * 64 * 64 * 64 * 9 * 56 * 56, "TFLOP/s"),
        "x5": X5("x5", "row program: layer norm fp32 4096x8192 with weight and bias", "f32", "hbm",
                 W.work_c3(), "GB/s"),
        "x6": X6("x6", "column reduction: root mean square down the columns, fp32 4096x8192", "f32",
                 "hbm", W.work_c3() // 2 + 4 * 8192, "GB/s"),
    }
    # the mix and size of each memory-bound configuration, then the plain streams
    for key, n_reads, write, mib in STREAMS:
        table[key] = Stream(key, n_reads, write, mib)
    if wl == "all":
        keys = ["c1", "c2", "c3", "c4", "c5"]
    elif wl == "streams":
        keys = [k for k, *_ in STREAMS]
    elif wl == "extra":
        keys = ["x1", "x2", "x3", "x4", "x5", "x6"]
    else:
        keys = [wl]
    return [table[k] for k in keys]


def run_one(rt, ctx, w, steps, warmup, want_cpu, prewarm):
    log(f"[bench] {w.key}: {w.title}: building inputs")
    sets = w.setup(rt)
    plans = [w.plan(rt, s) for s in sets]
    launches = [p.launch for p in plans]
    ctx.synchronize()
    # Untimed device warm-up: the GPU raises its clocks only under sustained
    # load, so a short burst would time the ramp instead of the kernel.
    t_end = time.perf_counter() + prewarm
    while time.perf_counter() < t_end:
        for i in range(50):
            launches[i % ROTATE]()
        ctx.synchronize()
    for i in range(warmup):
        launches[i % ROTATE]()
    ctx.synchronize()
    kernel = rt.last_kernel_name()
    start, stop = rt.Event(ctx), rt.Event(ctx)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        launches[i % ROTATE]()
    stop.record()
    ctx.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = start.elapsed_ms(stop)
    ms_step = wall * 1e3 / steps
    kern_ms = ev_ms / steps
    scale = 1e-9 if w.unit == "GB/s" else 1e-12
    value = w.work * scale / (wall / steps)
    achieved = w.work * scale / (kern_ms * 1e-3)
    peak = {"hbm": HBM_PEAK_GBS, "mfma": BF16_PEAK_TFLOPS, "valu": FP32_VECTOR_PEAK_TFLOPS}[w.bound]
    res = {
        "workload": w.title, "kernel": kernel, "dtype": w.dtype,
        "value": round(value, 2), "unit": w.unit, "ms_per_step": round(ms_step, 5),
        "roofline": {"bound": w.bound, "achieved": round(achieved, 2), "peak": peak,
                     "unit": w.unit, "frac": round(achieved / peak, 4),
                     "traffic": MEASURED_TRAFFIC.get(w.key),
                     "kernel_avg_us": round(kern_ms * 1e3, 3),
                     "algorithmic_work": w.work},
    }
    log(f"[bench] {w.key}: {kernel}: {kern_ms * 1e3:.2f} us/launch, "
        f"{achieved:.1f} {w.unit} = {100 * achieved / peak:.1f}% of peak; checking parity")
    res["parity"] = w.check(rt, sets[(steps - 1) % ROTATE])
    if want_cpu:
        sec, sample, cores = w.cpu()
        res["cpu_baseline"] = {"value": round(w.work * scale / sec, 3), "unit": w.unit,
                               "cores": cores, "kind": "port", "sample": sample,
                               "seconds": round(sec, 5)}
        log(f"[bench] {w.key}: cpu {res['cpu_baseline']['value']} {w.unit} on {cores} core(s)")
    for s in sets:
        for a in s:
            a.free()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all", choices=["all", "streams", "c0", "c1", "c2", "c3", "c4", "c5", "extra", "x1", "x2", "x3",
                             "x4", "x5", "x6"] + [k for k, *_ in STREAMS])
    ap.add_argument("--no-cpu", action="store_true", help="skip the NumPy CPU baseline")
    ap.add_argument("--prewarm", type=float, default=PREWARM_SECONDS,
                    help="seconds of untimed device warm-up per workload")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no "
                 "sharding); run with --gpus 1")
    if args.steps < 1:
        sys.exit("--steps must be at least 1")

    from hc_amd import runtime as rt          # fails loudly without the native library
    ctx = rt.default_context("hip:0")
    info = ctx.info()
    log(f"[bench] device {info}")

    results = {}
    for w in make_workloads(rt, args.workload):
        results[w.key] = run_one(rt, ctx, w, args.steps, args.warmup, not args.no_cpu,
                                 args.prewarm)
        if args.workload == "all" and w.key in STREAM_OF:
            # the plain stream of the same read:write mix and size, timed the same
            # way: the ceiling this kernel is held to
            (sw,) = make_workloads(rt, STREAM_OF[w.key])
            sr = run_one(rt, ctx, sw, args.steps, args.warmup, False, args.prewarm)
            kern = results[w.key]["roofline"]
            results[w.key]["stream_ceiling"] = {
                "workload": sr["workload"], "kernel": sr["kernel"],
                "kernel_avg_us": sr["roofline"]["kernel_avg_us"],
                "achieved": sr["roofline"]["achieved"], "unit": "GB/s",
                "frac_of_peak": sr["roofline"]["frac"], "parity_ok": sr["parity"]["ok"],
                "workload_vs_stream": round(kern["achieved"] / sr["roofline"]["achieved"], 4)}

    head_key = "c2" if "c2" in results else next(iter(results))
    head = results[head_key]
    out = {
        "metric": "HBM GB/s (elementwise/softmax/quant) + bf16 GEMM TFLOP/s, 1 MI355X",
        "value": head["value"], "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": head["workload"], "headline": head_key,
                   "rotating_buffer_sets": ROTATE, "device": info["arch"],
                   "compute_units": info["compute_units"],
                   "host_cpus": os.cpu_count(),
                   "host_cpus_usable": len(os.sched_getaffinity(0)),
                   "numpy": np.__version__},
        "roofline": head["roofline"],
        "parity": head["parity"],
        "configs": results,
    }
    if "cpu_baseline" in head:
        out["cpu_baseline"] = head["cpu_baseline"]
    print(json.dumps(out), flush=True)
    bad = [k for k, r in results.items() if not r["parity"]["ok"]]
    if bad:
        sys.exit(f"bench.py: parity failed for {bad}")


if __name__ == "__main__":
    main()
