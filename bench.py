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

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE in
# KiB per dispatch), scaled by what the same counters read for the plain copy
# of known size (workload c0).  The figures live in profiles/hbm_traffic.json,
# which `bench.py --traffic-from DIR` writes from the counter files of the
# commands listed in profiles/hbm_traffic_pmc.txt; a figure is reported only
# while the kernel that ran is the kernel that was measured.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
TRAFFIC_WORKLOADS = ("c0", "c1", "c2", "c3", "c4", "c5", "x5", "x6", "x8")
C0_KIB = 256 * 1024          # c0 reads and writes 256 MiB


def measured_traffic(key, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)["workloads"].get(key)
    except (OSError, ValueError, KeyError):
        return None
    if not rec or rec["kernel"] != kernel:
        return None
    return rec["bytes"]


def traffic_from(dirname, launches):
    """Reads DIR/<workload>_<counter>_counter_collection.csv (rocprofv3 --pmc, one
    counter and one workload per run, `launches` launches each) and writes
    profiles/hbm_traffic.json."""
    import collections
    import csv

    def per_launch(w, counter):
        # a step of a workload may be several kernels (x6: bands, then their fold):
        # their counters add up, and the record is keyed by the last one, which is
        # the name the bench line carries
        total = collections.defaultdict(float)
        last = None
        with open(os.path.join(dirname, f"{w}_{counter}_counter_collection.csv")) as f:
            rows = sorted(csv.DictReader(f), key=lambda r: int(r.get("Dispatch_Id", 0)))
        for r in rows:
            k = r["Kernel_Name"]
            if k.startswith("hcamd_") and "fill" not in k:
                total[k] += float(r["Counter_Value"])
                last = k
        if last is None:
            raise OSError(f"no kernel of the library in the {counter} file of {w}")
        kernels.setdefault(w, sorted(total))
        return last, sum(total.values()) / launches

    kernels = {}

    _, f0 = per_launch("c0", "FETCH_SIZE")
    _, w0 = per_launch("c0", "WRITE_SIZE")
    scale = {"FETCH_SIZE": C0_KIB / f0, "WRITE_SIZE": C0_KIB / w0}
    out = {"unit": "KiB per launch as the counters report them; bytes = scaled sum",
           "calibration": {"workload": "c0", "true_KiB_each_way": C0_KIB,
                           "FETCH_SIZE_KiB": round(f0, 1), "WRITE_SIZE_KiB": round(w0, 1),
                           "scale": {k: round(v, 4) for k, v in scale.items()}},
           "launches_per_run": launches, "workloads": {}}
    for w in TRAFFIC_WORKLOADS:
        try:
            kernel, fetch = per_launch(w, "FETCH_SIZE")
            _, write = per_launch(w, "WRITE_SIZE")
        except OSError:
            continue
        out["workloads"][w] = {
            "kernel": kernel, "kernels": kernels[w],
            "FETCH_SIZE_KiB": round(fetch, 1), "WRITE_SIZE_KiB": round(write, 1),
            "bytes": int((fetch * scale["FETCH_SIZE"] + write * scale["WRITE_SIZE"]) * 1024)}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(out, indent=1, sort_keys=True))


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


    class V5(C5):
        """The vendor library's GEMM on the same operands (hipBLASLt, reached through
        torch.matmul with B given as the transposed view of Bt): the yardstick for
        c5 that is not this library.  PyTorch launches on its own stream, so this
        workload brings its own events."""

        def setup(self, rt):
            import torch
            self.torch = torch
            self.a, self.bt = W.inputs_c5()
            dev = torch.device("cuda:0")

            def bf16(bits):
                return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)
            return [(bf16(self.a), bf16(self.bt),
                     torch.empty((self.a.shape[0], self.bt.shape[0]), dtype=torch.bfloat16,
                                 device=dev)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            torch = self.torch

            class TorchPlan:
                def launch(self_inner):
                    torch.matmul(s[0], s[1].T, out=s[2])
            return TorchPlan()

        def make_events(self):
            torch = self.torch

            class Ev:
                def __init__(self):
                    self.e = torch.cuda.Event(enable_timing=True)

                def record(self):
                    self.e.record()

                def elapsed_ms(self, other):
                    return self.e.elapsed_time(other.e)
            return Ev(), Ev()

        def synchronize(self):
            self.torch.cuda.synchronize()

        def kernel_name(self):
            return "hipBLASLt via torch.matmul (torch %s)" % self.torch.__version__

        def check(self, rt, s):
            from oracle import closed_forms as cf
            got = W.bf16_bits_to_f32(s[2].view(self.torch.int16).cpu().numpy().view(np.uint16))
            want = cf.np_gemm_bf16(self.a, self.bt, np.float32)
            ok = np.allclose(got, want, rtol=1e-2, atol=2.6e-4)
            return {"parity": "rtol 1e-2 vs fp32 accumulation" if ok else "MISMATCH",
                    "ok": bool(ok), "max_abs_err": float(np.max(np.abs(got - want)))}

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

    class X9(C2):
        """max(sqrt(|a*b+c|) * a - b, 0) * 0.5 on the C2 arrays: a 9-instruction program that never
        holds two values at once, which the map entry point runs on its chain kernel."""
        PROGRAM = [("in", 0), ("mul_in", 1), ("add_in", 2), ("abs", 0), ("sqrt", 0), ("mul_in", 0), ("sub_in", 1),
                   ("maxi", 0, 0.0), ("muli", 0, 0.5)]

        def plan(self, rt, s):
            return rt.plan_map([I(*p) for p in self.PROGRAM], s[:3], s[3])

        def numpy_result(self):
            a, b, c = (v.astype(np.float32) for v in (self.a, self.b, self.c))
            return (np.maximum(np.sqrt(np.abs(a * b + c)) * a - b, np.float32(0)) * np.float32(0.5)).astype(np.float16)

        def check(self, rt, s):
            ok = np.array_equal(s[3].to_host().view(np.uint16), self.numpy_result().view(np.uint16))
            return {"parity": "bit-exact vs NumPy (fp32 steps, one rounding to fp16)" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(self.numpy_result, 2), "full size, NumPy fp32 expression", 1

    class X7(C1):
        """a+b on the C1 vectors through the fused map kernel (2 instructions)."""

        def plan(self, rt, s):
            return rt.plan_map([I("in", 0), I("add_in", 1)], s[:2], s[2])

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
        through the @kernel front-end (a six-stage row program)."""

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

    class X10(Workload):
        """Log-softmax over the rows of the C3 matrix, written as a kernel body and launched through
        the @kernel front-end: a row program with a logarithm of a row scalar, which runs as two
        launches (the chain kernel for every row, the general kernel for rows it left alone)."""

        def setup(self, rt):
            from hc_amd.examples import log_softmax
            self.kernel = log_softmax()
            (self.x,) = W.inputs_c3()
            return [(rt.to_device(self.x), rt.DeviceArray(self.x.shape, np.float32)) for _ in range(ROTATE)]

        def plan(self, rt, s):
            (p,) = self.kernel.plan_rows(*s)
            return p

        def _numpy(self, x):
            c = x - x.max(axis=1, keepdims=True)
            return c - np.log(np.exp(c).sum(axis=1, keepdims=True))

        def check(self, rt, s):
            got, want = s[1].to_host(), self._numpy(self.x.astype(np.float64))
            ok = np.allclose(got, want, rtol=2e-5, atol=2e-5)
            return {"parity": "rtol 2e-5, atol 2e-5 vs fp64" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(lambda: self._numpy(self.x), 2), "full size, NumPy fp32", 1

    class X8(Workload):
        """Root-mean-square normalisation with an fp32 weight over the rows of the C4
        matrix (fp16 in, fp32 math, fp16 out), written as a kernel body and
        launched through the @kernel front-end."""

        def setup(self, rt):
            from hc_amd.examples import rms_norm_f16
            self.kernel = rms_norm_f16()
            (self.x,) = W.inputs_c4()
            self.g = np.random.default_rng(9).standard_normal(self.x.shape[1]).astype(np.float32)
            return [(rt.to_device(self.x), rt.to_device(self.g), rt.DeviceArray(self.x.shape, np.float16))
                    for _ in range(ROTATE)]

        def plan(self, rt, s):
            (p,) = self.kernel.plan_rows(*s)
            return p

        def _numpy(self, x):
            return x / np.sqrt((x * x).mean(axis=1, keepdims=True) + x.dtype.type(1e-6)) * self.g.astype(x.dtype)

        def check(self, rt, s):
            got, want = s[2].to_host().astype(np.float64), self._numpy(self.x.astype(np.float64))
            ok = np.allclose(got, want, rtol=1.1e-3, atol=1e-6)
            return {"parity": "one fp16 ulp (rtol 1.1e-3) vs fp64" if ok else "MISMATCH", "ok": bool(ok)}

        def cpu(self):
            return _best_of(lambda: self._numpy(self.x.astype(np.float32)).astype(np.float16), 2), \
                "full size, NumPy fp32", 1

    table = {
        "c0": C0("c0", "copy 256 MiB int32 (calibration)", "u32", "hbm", 2 * 4 * 64 * 1024 * 1024,
                 "GB/s"),
        "c1": C1("c1", "vadd fp32 N=16777259", "f32", "hbm", W.work_c1(), "GB/s"),
        "c2": C2("c2", "fma fp16 8191x8193 (fp32 math)", "f16", "hbm", W.work_c2(), "GB/s"),
        "c3": C3("c3", "row softmax fp32 4096x8192", "f32", "hbm", W.work_c3(), "GB/s"),
        "c4": C4("c4", "row absmax int8 quantize fp16 16384x4096", "f16->i8", "hbm",
                 W.work_c4(), "GB/s"),
        "c5": C5("c5", "GEMM bf16 4096^3 (fp32 acc)", "bf16", "mfma", W.work_c5(), "TFLOP/s"),
        "v5": V5("v5", "vendor library GEMM bf16 4096^3 on the c5 operands (yardstick)", "bf16",
                 "mfma", W.work_c5(), "TFLOP/s"),
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
        "x7": X7("x7", "map kernel: vadd fp32 N=16777259 as a 2-instruction program", "f32", "hbm",
                 W.work_c1(), "GB/s"),
        "x8": X8("x8", "row program: rms norm fp16 16384x4096 with an fp32 weight (fp32 math)", "f16", "hbm",
                 2 * 2 * 16384 * 4096 + 4 * 4096, "GB/s"),
        "x10": X10("x10", "row program: log-softmax fp32 4096x8192 (two launches)", "f32", "hbm",
                   W.work_c3(), "GB/s"),
        "x9": X9("x9", "map kernel: a 9-instruction chain on the fp16 8191x8193 arrays", "f16", "hbm",
                 W.work_c2(), "GB/s"),
    }
    # the mix and size of each memory-bound configuration, then the plain streams
    for key, n_reads, write, mib in STREAMS:
        table[key] = Stream(key, n_reads, write, mib)
    if wl == "all":
        keys = ["c1", "c2", "c3", "c4", "c5"]
    elif wl == "streams":
        keys = [k for k, *_ in STREAMS]
    elif wl == "extra":
        keys = ["x1", "x2", "x3", "x4", "x5", "x6", "x7", "x8", "x9", "x10"]
    else:
        keys = [wl]
    return [table[k] for k in keys]


def run_one(rt, ctx, w, steps, warmup, want_cpu, prewarm, check=True):
    log(f"[bench] {w.key}: {w.title}: building inputs")
    sets = w.setup(rt)
    plans = [w.plan(rt, s) for s in sets]
    launches = [p.launch for p in plans]
    # a workload that does not launch on this library's queue brings its own
    # synchronisation and events (the vendor-library yardstick)
    sync = getattr(w, "synchronize", ctx.synchronize)
    sync()
    # Untimed device warm-up: the GPU raises its clocks only under sustained
    # load, so a short burst would time the ramp instead of the kernel.
    t_end = time.perf_counter() + prewarm
    while time.perf_counter() < t_end:
        for i in range(50):
            launches[i % ROTATE]()
        sync()
    for i in range(warmup):
        launches[i % ROTATE]()
    sync()
    kernel = w.kernel_name() if hasattr(w, "kernel_name") else rt.last_kernel_name()
    start, stop = w.make_events() if hasattr(w, "make_events") else (rt.Event(ctx), rt.Event(ctx))
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        launches[i % ROTATE]()
    stop.record()
    sync()
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
                     "traffic": measured_traffic(w.key, kernel),
                     "kernel_avg_us": round(kern_ms * 1e3, 3),
                     "algorithmic_work": w.work},
    }
    if res["roofline"]["traffic"] and w.bound == "hbm":
        res["roofline"]["traffic_vs_algorithmic"] = round(res["roofline"]["traffic"] / w.work, 4)
    log(f"[bench] {w.key}: {kernel}: {kern_ms * 1e3:.2f} us/launch, "
        f"{achieved:.1f} {w.unit} = {100 * achieved / peak:.1f}% of peak; checking parity")
    res["parity"] = (w.check(rt, sets[(steps - 1) % ROTATE]) if check
                     else {"parity": "not checked", "ok": True, "checked": False})
    if want_cpu:
        sec, sample, cores = w.cpu()
        res["cpu_baseline"] = {"value": round(w.work * scale / sec, 3), "unit": w.unit,
                               "cores": cores, "kind": "port", "sample": sample,
                               "seconds": round(sec, 5)}
        log(f"[bench] {w.key}: cpu {res['cpu_baseline']['value']} {w.unit} on {cores} core(s)")
    for s in sets:
        for a in s:
            if hasattr(a, "free"):
                a.free()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all", choices=["all", "streams", "c0", "c1", "c2", "c3", "c4", "c5", "v5", "extra", "x1", "x2", "x3",
                             "x4", "x5", "x6", "x7", "x8", "x9", "x10"] + [k for k, *_ in STREAMS])
    ap.add_argument("--no-cpu", action="store_true", help="skip the NumPy CPU baseline")
    ap.add_argument("--variant", action="append", default=[], metavar="FAMILY=N",
                    help="measure kernel variant N of a family (hcamdSetVariant), e.g. gemm=14; "
                         "for profiling alternatives, never part of the default run")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the parity check (only for measurement probes whose output "
                         "is not the product, such as gemm=17)")
    ap.add_argument("--prewarm", type=float, default=PREWARM_SECONDS,
                    help="seconds of untimed device warm-up per workload")
    ap.add_argument("--traffic-from", metavar="DIR",
                    help="no benchmark: read rocprofv3 --pmc counter files from DIR and write "
                         "profiles/hbm_traffic.json (see profiles/hbm_traffic_pmc.txt)")
    ap.add_argument("--traffic-launches", type=int, default=6,
                    help="launches per counter run (warm-up + steps) for --traffic-from")
    args = ap.parse_args()
    if args.traffic_from:
        traffic_from(args.traffic_from, args.traffic_launches)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no "
                 "sharding); run with --gpus 1")
    if args.steps < 1:
        sys.exit("--steps must be at least 1")

    from hc_amd import runtime as rt          # fails loudly without the native library
    ctx = rt.default_context("hip:0")
    info = ctx.info()
    log(f"[bench] device {info}")

    for spec in args.variant:
        family, _, number = spec.partition("=")
        rt.set_variant(family, int(number))
    results = {}
    for w in make_workloads(rt, args.workload):
        results[w.key] = run_one(rt, ctx, w, args.steps, args.warmup, not args.no_cpu,
                                 args.prewarm, not args.no_check)
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
