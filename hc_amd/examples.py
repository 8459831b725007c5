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
