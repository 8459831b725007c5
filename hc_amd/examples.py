"""Kernel bodies written against the `@kernel` API that the benchmarks launch.

(No `from __future__ import annotations` here: the decorator reads the
parameter annotations as objects, as the reference's does.)
"""

import numpy as np

from .kernel import (Buffer, CurrentGroup, TunableParam, create_mapping, kernel, sym, typename)

DT = typename.DT


def convolution(stride: int = 1, tile: int = 64, k_block: int = 64):
    """Valid 2-D convolution (cross-correlation), NCHW fp32, as the implicit
    GEMM of python/hckernel/tests/test_examples.py:203-252: a group owns TN
    images x TNF filters at one output position; the im2col row of an image and
    the flattened filter are gathered through index mappings and multiplied in
    K blocks.  (H - HF) and (W - WF) must be multiples of the stride."""
    N, C, H, W, NF, HF, WF, KB, TN, TNF = (sym.N, sym.C, sym.H, sym.W, sym.NF, sym.HF, sym.WF,
                                           sym.KB, sym.TN, sym.TNF)
    HO = (H - HF) / stride + 1
    WO = (W - WF) / stride + 1
    SZ = HF * WF * C
    KI = (SZ + KB - 1) // KB
    tun = (TunableParam(TN, tile, range(1, 65)), TunableParam(TNF, tile, range(1, 65)),
           TunableParam(KB, k_block, range(8, 129)))
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

    return conv


def layer_norm(eps: float = 1e-5, rows_per_group: int = 8):
    """out = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias along the rows of
    a float32 matrix: a body that mixes elementwise arithmetic with reductions
    along axis 1 (the shape of python/hckernel/tests/test_examples.py:304-336,
    the reference's softmax example).  A group owns `rows_per_group` whole rows."""
    M, N, GM = sym.M, sym.N, sym.GM

    @kernel(work_shape=M, group_shape=GM)
    def body(gr: CurrentGroup, x: Buffer[M, N, DT], weight: Buffer[N, DT], bias: Buffer[N, DT],
             out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        w, b = gr.load(weight[:], shape=(N,)), gr.load(bias[:], shape=(N,))
        mean = t.mean(axis=1, keepdims=True)
        var = t.var(axis=1, keepdims=True)
        gr.store(out[m0:, :], (t - mean) / np.sqrt(var + np.float32(eps)) * w + b)

    def plan(x, weight, bias, out, **kw):
        return body.plan(x, weight, bias, out, rows_per_group, **kw)
    body.plan_rows = plan
    return body


def log_softmax(rows_per_group: int = 8):
    """out = (x - max(x)) - log(sum(exp(x - max(x)))) along the rows of a float32
    matrix: a row program in which a NumPy function of a row scalar (the
    logarithm of the sum, which numpy.ma deactivates outside its domain) stands
    between the reductions and the store."""
    M, N, GM = sym.M, sym.N, sym.GM

    @kernel(work_shape=M, group_shape=GM)
    def body(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N))
        c = t - t.max(axis=1, keepdims=True)
        gr.store(out[m0:, :], c - np.log(np.exp(c).sum(axis=1, keepdims=True)))

    def plan(x, out, **kw):
        return body.plan(x, out, rows_per_group, **kw)
    body.plan_rows = plan
    return body


def rms_norm_f16(eps: float = 1e-6, rows_per_group: int = 8):
    """out = x / sqrt(mean(x * x) + eps) * weight along the rows of a float16
    matrix, computed in float32 (the weight is float32) and stored as float16:
    the second normalisation that is common enough to have a kernel of its own
    behind the row-program entry point."""
    M, N, GM = sym.M, sym.N, sym.GM
    f = np.float32

    @kernel(work_shape=M, group_shape=GM)
    def body(gr: CurrentGroup, x: Buffer[M, N, DT], weight: Buffer[N, DT], out: Buffer[M, N, DT], gshape: GM):
        m0, mb = gr.work_offset[0], gr.shape[0]
        t = gr.load(x[m0:, :], shape=(mb, N)).astype(f)
        ms = np.mean(np.square(t), axis=1, keepdims=True)
        gr.store(out[m0:, :], (t / np.sqrt(ms + f(eps)) * gr.load(weight[:], shape=(N,))).astype(np.float16))

    def plan(x, weight, out, **kw):
        return body.plan(x, weight, out, rows_per_group, **kw)
    body.plan_rows = plan
    return body


def column_rms(eps: float = 1e-6, cols_per_group: int = 512):
    """out[c] = sqrt(mean(x[:, c] ** 2) + eps) down the columns of a float32
    matrix: a body that reduces tiles holding whole columns along axis 0 (the
    tile methods the simulator forwards to NumPy,
    python/hckernel/kernel_api.py:150-151).  A group owns `cols_per_group`
    columns."""
    M, N, GN = sym.M, sym.N, sym.GN

    @kernel(work_shape=(N + GN - 1) // GN, group_shape=1, literals={GN})
    def body(gr: CurrentGroup, x: Buffer[M, N, DT], out: Buffer[N, DT], gn: GN):
        n0 = gr.id[0] * GN
        t = gr.load(x[:, n0:], shape=(M, GN))
        gr.store(out[n0:], np.sqrt((t * t).mean(axis=0) + np.float32(eps)))

    def plan(x, out, **kw):
        return body.plan(x, out, cols_per_group, **kw)
    body.plan_cols = plan
    return body
