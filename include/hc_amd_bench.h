/*
 * hc_amd_bench.h - measurement entry points of libhc_amd_runtime.so
 *
 * Not part of the drop-in boundary (hc_amd_runtime.h): nothing here computes a
 * result a kernel body asks for, and none of it has a counterpart in the
 * reference.  These entry points exist so that the throughput of the kernels can
 * be held against what the memory system delivers (the stream calibration, which
 * the benchmark's default run uses for its per-workload ceilings) and so that the
 * GEMM's loop can be taken apart on the GPU (the probe builds).
 */
#ifndef HC_AMD_BENCH_H
#define HC_AMD_BENCH_H

#include "hc_amd_runtime.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Stream calibration (no counterpart in the reference): what HBM delivers for
 * a mix of read and write streams with nothing else in the way, the yardstick
 * the memory-bound kernels are held to.  nReads (0..3) vectors of `bytes` bytes
 * are added in 32-bit lanes, word by word; writeMode selects what leaves:
 * HCAMD_STREAM_FULL the sum (bytes out), HCAMD_STREAM_HALF the xor of each sum
 * word's halves (bytes / 2 out: the 2:1 ratio of the int8 quantiser),
 * HCAMD_STREAM_NONE one 32-bit total per 16 KiB of input (bytes / 4096 out: a
 * read-only stream with a checkable result).  nReads == 0 writes the word
 * index (a fill; HCAMD_STREAM_FULL only).  bytes must be a multiple of 16 KiB,
 * pointers 16-byte aligned.  Each mix runs in the form that measured fastest
 * for it: three reads against one write from workgroups held to four waves per
 * SIMD that pause between the arrival of their words and their store, the
 * others from full workgroups that do not ("stream" variants 1..5 force one
 * form on every mix that reads and writes). */
enum HcamdStreamWrite { HCAMD_STREAM_NONE = 0, HCAMD_STREAM_FULL = 1, HCAMD_STREAM_HALF = 2 };
int hcamdLaunchStream(OlQueue q, int nReads, int writeMode, const void *const *inputs,
                      void *out, size_t bytes) HCAMD_NOEXCEPT;

/* 1 if the library holds the measurement builds of the bf16 GEMM ("gemm"
 * variants 17..22, 26, 28 and 29: the default 256 x 256 kernel with its MFMAs
 * only, without its waits on loads, without its barriers, without its LDS
 * reads, without its loads, with its loads to registers, with B read directly,
 * without its stores, with two K tiles only; 30..32, further hand orders of
 * the four-wave kernel of variant 27 that only measurements select; 33 and 34,
 * the MFMAs only in 16 x 16 x 32 and in 32 x 32 x 16 blocks with C stored
 * straight from the accumulators).  What 17..29, 33 and 34 leave in C is NOT
 * the product.  They are compiled only when the
 * library is built with `python -m hc_amd.build --probes` (HCAMD_PROBES); any
 * other build returns 0 here, holds none of them, and hcamdSetVariant /
 * hcamdSetThreadVariant return 1 for their numbers. */
int hcamdProbesBuilt(void) HCAMD_NOEXCEPT;

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* HC_AMD_BENCH_H */
