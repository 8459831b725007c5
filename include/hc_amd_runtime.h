/*
 * hc_amd_runtime.h - C ABI of libhc_amd_runtime.so
 *
 * One shared library for one MI355X (gfx950).  It exports three groups of
 * entry points:
 *
 *   1. ol*     - the 13-function offload ABI of the reference
 *                (gpu-runtime/common/include/offload_api.h:27-63), implemented
 *                directly on the HIP module API.  The library is therefore both
 *                "the loader" and "the hip backend" of the reference
 *                (gpu-runtime/loader/src/Loader.cpp:326-444,
 *                gpu-runtime/hip-runtime/src/Runtime.cpp:100-248).
 *   2. hcgpu*  - the entry points JIT'd host code and ctypes bind in the
 *                reference (python/cpp/py-runtime/src/PyRuntime.cpp:36-94).
 *                The two functions that take a PyObject* live in the companion
 *                library libhc_amd_pyabi.so (hc_amd_pyabi.h) so that this
 *                library has no CPython dependency.
 *   3. hcamd*  - additions that have no counterpart in the reference: access
 *                to the built-in gfx950 code objects, typed launchers for the
 *                hand-written kernels, copies and events.  The reference has
 *                none of these because its device code is compiler generated
 *                and its buffers are torch allocations
 *                (python/hckernel/tests/test_e2e.py:32-33).
 *
 * Conventions: plain pointers and sizes only; every function is noexcept;
 * handle-returning functions return NULL on error and int-returning functions
 * return non-zero on error, after calling the device's error callback with a
 * message of at most 255 characters (offload_api.h:29-31).  No function takes
 * a lock: callers serialise, as the reference's do
 * (python/cpp/py-runtime/src/GpuRuntime.cpp:23-24).
 */
#ifndef HC_AMD_RUNTIME_H
#define HC_AMD_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#define HCAMD_NOEXCEPT noexcept
#else
#define HCAMD_NOEXCEPT
#endif

/* ---------------------------------------------------------------------------
 * 1. Offload ABI.  offload_api.h:9-20 (handle and callback types).
 * ------------------------------------------------------------------------ */
typedef void *OlDevice;
typedef void *OlModule;
typedef void *OlKernel;
typedef void *OlQueue;

/* offload_api.h:14-18 declares `enum class OlSeverity : int`; an int carries
 * the same values through a C signature. */
typedef int OlSeverity;
#define OL_SEVERITY_ERROR 0
#define OL_SEVERITY_WARNING 1
#define OL_SEVERITY_MESSAGE 2

typedef void (*OlErrorCallback)(void *ctx, OlSeverity sev, const char *desc);

/* offload_api.h:32-35; hip-runtime/src/Runtime.cpp:100-126.  `desc` is
 * "hip:<index>".  A prefix other than "hip" reports "Runtime not found: <p>"
 * (Loader.cpp:357-359), a missing ':' reports "Invalid device desc: <desc>"
 * (Loader.cpp:331-335), an unparsable index reports "Invalid device id"
 * (Runtime.cpp:115-119).  Makes the device current (hipSetDevice). */
OlDevice olCreateDevice(const char *desc, OlErrorCallback errCallback,
                        void *ctx) HCAMD_NOEXCEPT;
/* offload_api.h:35; Runtime.cpp:127-129. */
void olReleaseDevice(OlDevice dev) HCAMD_NOEXCEPT;

/* offload_api.h:38-40; Runtime.cpp:131-145.  `data` is an ELF code object for
 * gfx950 (hipModuleLoadData); `len` is not needed by HIP and is ignored, as in
 * the reference. */
OlModule olCreateModule(OlDevice dev, const void *data,
                        size_t len) HCAMD_NOEXCEPT;
void olReleaseModule(OlModule mod) HCAMD_NOEXCEPT;

/* offload_api.h:42-44; Runtime.cpp:147-159 (hipModuleGetFunction).  The module
 * must outlive the kernel.  olReleaseKernel frees the small handle. */
OlKernel olGetKernel(OlModule mod, const char *name) HCAMD_NOEXCEPT;
void olReleaseKernel(OlKernel k) HCAMD_NOEXCEPT;

/* offload_api.h:46-49; Runtime.cpp:161-191.  globalsSizes is x-first (the last
 * Python dimension first, mlir/lib/Transforms/LowerHKernel.cpp:296-305).
 * Budget 1024 work-items: for each dim with size > 1 take min(size, budget)
 * and divide the budget by that value rounded up to a power of two; other dims
 * get 1.  Returns 1 when nDims is not 1..3.  `k` may be NULL: the heuristic
 * does not look at the kernel. */
int olSuggestBlockSize(OlKernel k, const size_t *globalsSizes,
                       size_t *blockSizesRet, size_t nDims) HCAMD_NOEXCEPT;

/* offload_api.h:51-53; Runtime.cpp:193-212.  One HIP stream at the default
 * priority. */
OlQueue olCreateQueue(OlDevice dev) HCAMD_NOEXCEPT;
void olReleaseQueue(OlQueue q) HCAMD_NOEXCEPT;
int olSyncQueue(OlQueue q) HCAMD_NOEXCEPT;

/* offload_api.h:55-57; Runtime.cpp:214-231 (hipMalloc / hipFree; `align` is
 * satisfied by hipMalloc's 256-byte alignment). */
void *olAllocDevice(OlQueue q, size_t size, size_t align) HCAMD_NOEXCEPT;
void olDeallocDevice(OlQueue q, void *data) HCAMD_NOEXCEPT;

/* offload_api.h:59-63; Runtime.cpp:233-248.  nDims must be 3 ("Invalid launch
 * dims: <n>" otherwise); gridSizes/blockSizes are x,y,z; `args` is an array of
 * nArgs pointers, one to each kernel argument
 * (mlir/lib/Transforms/GpuToGpuRuntime.cpp:279-292).  Asynchronous on the
 * queue's stream (hipModuleLaunchKernel). */
int olLaunchKernel(OlQueue q, OlKernel k, const size_t *gridSizes,
                   const size_t *blockSizes, size_t nDims, void **args,
                   size_t nArgs, size_t sharedMemSize) HCAMD_NOEXCEPT;

/* Loader extras: gpu-runtime/loader/src/Loader.cpp:20-45.  The backend is
 * built in, so the search paths are recorded but never searched.  Tracing
 * prints "<fn> enter" / "<fn> exit" on stdout for every ol* call and the
 * launch geometry for olLaunchKernel (Loader.cpp:433-438). */
void setGPULoaderSearchPaths(const char *paths[], size_t count) HCAMD_NOEXCEPT;
void enableFuncTracing(int val) HCAMD_NOEXCEPT;

/* ---------------------------------------------------------------------------
 * 2. Python-runtime ABI (launch half).  PyRuntime.cpp:36-94.
 * ------------------------------------------------------------------------ */

/* PyRuntime.cpp:36-39.  "<fn> enter/exit" on stdout for every hcgpu* call. */
void hcgpuEnableTraceFunctions(int val) HCAMD_NOEXCEPT;

/* PyRuntime.cpp:73-78; GpuRuntime.cpp:26-51.  Returns *handle when it is set.
 * Otherwise creates the process-wide device and queue from deviceDesc on first
 * use (the first desc wins for the life of the process), loads the code
 * object, looks the kernel up, stores it in *handle and returns it.  Any
 * failure prints "Offload error: <msg>" on stderr and aborts
 * (GpuRuntime.cpp:11-21). */
void *hcgpuGetKernel(void **handle, const char *deviceDesc, const void *data,
                     size_t dataSize, const char *kernelName) HCAMD_NOEXCEPT;

/* PyRuntime.cpp:80-85; GpuRuntime.cpp:53-58.  olSuggestBlockSize, abort on
 * failure. */
void hcgpuSuggestBlockSize(void *kernel, const size_t *globalSizes,
                           size_t *blockSizesRet, size_t nDim) HCAMD_NOEXCEPT;

/* PyRuntime.cpp:87-94; GpuRuntime.cpp:60-69.  olLaunchKernel on the
 * process-wide queue followed by olSyncQueue: synchronous on return.  Abort on
 * failure. */
void hcgpuLaunchKernel(void *kernel, const size_t *gridSizes,
                       const size_t *blockSizes, size_t nDim, void **args,
                       size_t nArgs, size_t sharedMemSize) HCAMD_NOEXCEPT;

/* ---------------------------------------------------------------------------
 * 3. Additions (no counterpart in the reference).
 * ------------------------------------------------------------------------ */

/* The process-wide device and queue hcgpuGetKernel uses, created on first use
 * from deviceDesc.  Unlike hcgpu*, failures return NULL after the
 * "Offload error" line instead of aborting. */
OlQueue hcamdGetDefaultQueue(const char *deviceDesc) HCAMD_NOEXCEPT;
OlDevice hcamdGetDefaultDevice(const char *deviceDesc) HCAMD_NOEXCEPT;
/* The device a queue belongs to. */
OlDevice hcamdQueueDevice(OlQueue q) HCAMD_NOEXCEPT;

/* Built-in gfx950 code objects, embedded in the library the way JIT'd host
 * code embeds its blob (GpuToGpuRuntime.cpp:161-169).  Index 0..count-1;
 * returns 0 and fills name/data/len, or 1 when the index is out of range.
 * The blobs can be handed to olCreateModule / hcgpuGetKernel. */
size_t hcamdBuiltinModuleCount(void) HCAMD_NOEXCEPT;
int hcamdGetBuiltinModule(size_t index, const char **name, const void **data,
                          size_t *len) HCAMD_NOEXCEPT;
/* Kernel handle from the built-in modules, loaded once per device and cached.
 * The handle is owned by the device: do not release it. */
OlKernel hcamdGetBuiltinKernel(OlDevice dev, const char *moduleName,
                               const char *kernelName) HCAMD_NOEXCEPT;

/* Copies on the queue's stream.  kind: 0 host-to-device, 1 device-to-host,
 * 2 device-to-device.  Asynchronous for pinned host memory; pageable host
 * memory is staged by HIP.  hcamdFill32 writes `count` 32-bit words with a
 * small kernel (safe under stream capture). */
int hcamdMemcpy(OlQueue q, void *dst, const void *src, size_t bytes,
                int kind) HCAMD_NOEXCEPT;
int hcamdFill32(OlQueue q, void *dst, uint32_t value,
                size_t count) HCAMD_NOEXCEPT;

/* Events on the queue's stream, for timing kernels where they run. */
typedef void *HcamdEvent;
HcamdEvent hcamdEventCreate(OlQueue q) HCAMD_NOEXCEPT;
void hcamdEventDestroy(HcamdEvent e) HCAMD_NOEXCEPT;
int hcamdEventRecord(HcamdEvent e) HCAMD_NOEXCEPT;
int hcamdEventSynchronize(HcamdEvent e) HCAMD_NOEXCEPT;
int hcamdEventElapsedMs(HcamdEvent start, HcamdEvent stop,
                        float *ms) HCAMD_NOEXCEPT;

/* Device facts used for roofline arithmetic: compute units, engine clock in
 * kHz, memory clock in kHz, memory bus width in bits, bytes of device memory,
 * and the gcn arch name (copied into archName, NUL terminated, at most
 * archLen bytes). */
int hcamdDeviceInfo(OlDevice dev, int *computeUnits, int *clockKHz,
                    int *memClockKHz, int *memBusBits, size_t *totalMem,
                    char *archName, size_t archLen) HCAMD_NOEXCEPT;

/* ---- Typed launchers for the hand-written kernels -------------------------
 * All are asynchronous on the queue's stream and return 0 / non-zero.  They
 * validate shapes and alignment on the host and pick the launch geometry;
 * pointers are device pointers.  Leading dimensions (ld*) are in elements.
 * Element types are given by size for copies and are fixed for the rest.
 */

/* Masked 2-D tile copy, the one kernel the reference's compiled path can
 * express (python/hckernel/tests/test_e2e.py:57-136; semantics of
 * CurrentGroup.load/store, python/hckernel/kernel_api.py:297-342): copies the
 * window [0,min(srcRows,dstRows)) x [0,min(srcCols,dstCols)) and leaves every
 * other byte of dst untouched.  elemSize is 1, 2, 4, 8 or 16.  Strides in
 * elements; either may be non-unit.  Dense windows move as one vector; windows
 * with unit inner strides move in aligned 16-byte pieces of the destination
 * rows with byte-wise ends (read with aligned loads where the source rows lie
 * the same way against 16-byte boundaries, with unaligned ones otherwise);
 * other windows element by element; source and destination must not overlap. */
int hcamdLaunchCopy2D(OlQueue q, size_t elemSize, const void *src,
                      size_t srcRows, size_t srcCols, ptrdiff_t srcStride0,
                      ptrdiff_t srcStride1, void *dst, size_t dstRows,
                      size_t dstCols, ptrdiff_t dstStride0,
                      ptrdiff_t dstStride1) HCAMD_NOEXCEPT;

/* dst[c][r] = src[r][c] for r < rows, c < cols: what a body stores that
 * writes a loaded tile's `.T` to the transposed window (an attribute the
 * reference's tile wrapper forwards to numpy.ma,
 * python/hckernel/kernel_api.py:150-151).  elemSize is 1, 2, 4 or 8; leading
 * dimensions in elements, unit inner strides; 64 x 64 elements per workgroup
 * through LDS; every other byte of dst stays as it was; source and destination
 * must not overlap. */
int hcamdLaunchTranspose2D(OlQueue q, size_t elemSize, const void *src, size_t srcLd, void *dst,
                           size_t dstLd, size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* Ids as data: out[index] = value for every work-item (perItem != 0) or once per
 * group, with index (one per dimension of out) and value affine in the group id
 * and the local id: x = c + sum_k g[k] * group_id[k] + sum_k l[k] * local_id[k],
 * k over the `rank` dimensions of the work shape in the Python order.  This is
 * what a body computes that stores `wi.local_id()`, `wi.global_id()`, group ids
 * or subgroup ids into a buffer (python/hckernel/kernel_api.py:231-252,397-403;
 * python/hckernel/kernel.py:97-131), and the launch uses the reference's own
 * geometry: block = groupShape, grid = groupCount, last dimension on x
 * (mlir/lib/Transforms/LowerHKernel.cpp:284-367), so hardware ids are the
 * model's ids.  outType: HCAMD_I32, HCAMD_I64 or HCAMD_F32; strides in
 * elements.  An index outside out stores nothing.  prod(groupShape) <= 1024. */
typedef struct HcamdAffineId {
  int64_t c, g[3], l[3];
} HcamdAffineId;
int hcamdLaunchIdScatter(OlQueue q, void *out, int outType, size_t outRank,
                         const size_t *outShape, const ptrdiff_t *outStrides,
                         const HcamdAffineId *index, const HcamdAffineId *value, size_t rank,
                         const size_t *groupCount, const size_t *groupShape,
                         int perItem) HCAMD_NOEXCEPT;

/* The same copy launched with the reference's own geometry and kernel argument
 * list (tests/Transforms/gpu-to-gpu-runtime.mlir:34-37): grid =
 * (ceil(cols/(bx*unroll)), ceil(rows/by), 1), block = (bx, by, 1), one element
 * per work-item per load, `unroll` loads per work-item along the row
 * (test_e2e.py:80-136).  Present so that the reference's tile decomposition
 * can be checked on the GPU; hcamdLaunchCopy2D is the fast path. */
int hcamdLaunchCopy2DTiled(OlQueue q, size_t elemSize, const void *src,
                           void *dst, size_t rows, size_t cols,
                           ptrdiff_t srcStride0, ptrdiff_t dstStride0,
                           size_t blockX, size_t blockY,
                           size_t unroll) HCAMD_NOEXCEPT;

/* c[i] = a[i] + b[i], fp32, i < n.  One IEEE add per element. */
int hcamdLaunchAddF32(OlQueue q, const float *a, const float *b, float *c,
                      size_t n) HCAMD_NOEXCEPT;

/* d = (half)((float)a * (float)b + (float)c) over a rows x cols window of
 * row-major fp16 arrays; round to nearest even on the final conversion, fp16
 * denormals kept.  When all four arrays are contiguous (ld == cols) the window
 * is processed as one flat vector of rows*cols elements. */
int hcamdLaunchFmaF16(OlQueue q, const void *a, size_t lda, const void *b,
                      size_t ldb, const void *c, size_t ldc, void *d,
                      size_t ldd, size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* Fused elementwise map: out = f(in_0 .. in_{n-1}) element by element over a
 * rows x cols window, f given as a postfix program on a stack of fp32 values
 * (at most HCAMD_MAP_STACK_DEPTH deep, HCAMD_MAP_MAX_INSTRS long, leaving one
 * value).  This is what a kernel body made of loads, arithmetic and one store
 * lowers to (python/hckernel/kernel_api.py:106-211 gives the tile operators
 * their NumPy meaning): IEEE fp32 arithmetic without contraction; R16 rounds
 * the top of the stack to fp16 and back (arithmetic on fp16 tiles); MAX / MIN
 * propagate NaN like numpy.maximum / numpy.minimum; the store rounds to
 * nearest even.  Operands are fp32 or fp16, each with its own leading
 * dimension in elements.  The program is validated on the host; a malformed
 * one is an error, not a launch.  On dense arrays a program of five
 * instructions or more that never holds two values at once (IN or CONST first,
 * then no further push and no two-value operation) runs on a kernel that
 * interprets sixteen elements of a lane per dispatch; the results are the same
 * bit for bit (variant 4 of the "map" family: every such program, 5: none). */
enum HcamdElemType { HCAMD_F32 = 0, HCAMD_F16 = 1, HCAMD_BF16 = 2, HCAMD_I32 = 3, HCAMD_I64 = 4,
                     HCAMD_U8 = 5 };
enum HcamdMapOp {
  HCAMD_MAP_END = 0,
  HCAMD_MAP_IN = 1,    /* push operand `arg` */
  HCAMD_MAP_CONST = 2, /* push imm */
  HCAMD_MAP_ADD = 3,   /* pop b, pop a, push a op b */
  HCAMD_MAP_SUB = 4,
  HCAMD_MAP_MUL = 5,
  HCAMD_MAP_DIV = 6,
  HCAMD_MAP_MAX = 7,
  HCAMD_MAP_MIN = 8,
  HCAMD_MAP_RSUB = 9,  /* b - a */
  HCAMD_MAP_RDIV = 10, /* b / a */
  HCAMD_MAP_ADDI = 11, /* top = top op imm */
  HCAMD_MAP_SUBI = 12,
  HCAMD_MAP_MULI = 13,
  HCAMD_MAP_DIVI = 14,
  HCAMD_MAP_MAXI = 15,
  HCAMD_MAP_MINI = 16,
  HCAMD_MAP_RSUBI = 17, /* imm - top */
  HCAMD_MAP_RDIVI = 18, /* imm / top */
  HCAMD_MAP_NEG = 19,   /* top = f(top) */
  HCAMD_MAP_ABS = 20,
  HCAMD_MAP_SQRT = 21,
  HCAMD_MAP_RINT = 22,
  HCAMD_MAP_EXP = 23,
  HCAMD_MAP_LOG = 24,
  HCAMD_MAP_TANH = 25,
  HCAMD_MAP_R16 = 26,
  HCAMD_MAP_ADD_IN = 27, /* top = top op operand `arg` */
  HCAMD_MAP_SUB_IN = 28,
  HCAMD_MAP_MUL_IN = 29,
  HCAMD_MAP_DIV_IN = 30,
  HCAMD_MAP_MAX_IN = 31,
  HCAMD_MAP_MIN_IN = 32,
  HCAMD_MAP_RSUB_IN = 33, /* operand - top */
  HCAMD_MAP_RDIV_IN = 34, /* operand / top */
  /* The tile OPERATOR `/`, as numpy.ma computes it
   * (python/hckernel/kernel_api.py:157-180 forwards it to numpy.ma): a quotient
   * that is not finite (a zero divisor gives one) makes its element inactive,
   * nothing is stored or summed for it, and its value becomes 0 + dividend.
   * The forms mirror DIV / RDIV; for an fp16 tile the quotient is rounded to
   * fp16 before the test: bit 8 of `arg` says so (MDIV / RMDIV: any `arg`; the
   * low bits of the *_IN forms are the operand index).  HCAMD_MAP_DIV and its
   * forms stay the plain quotient.  hcamdLaunchMap, hcamdLaunchMapSum and the
   * element-wise stages of hcamdLaunchRowProgram (whose sums, maxima and
   * minima leave inactive elements out, as numpy.ma's reductions do). */
  HCAMD_MAP_MDIV = 35,
  HCAMD_MAP_RMDIV = 36,
  HCAMD_MAP_MDIVI = 37,
  HCAMD_MAP_RMDIVI = 38,
  HCAMD_MAP_MDIV_IN = 39,
  HCAMD_MAP_RMDIV_IN = 40,
  HCAMD_MAP_CLEAR = 41,  /* every element active again (ends a program whose result is stored in full) */
  HCAMD_MAP_POWCHK = 42, /* numpy.ma.power: top not finite -> inactive, value 1e20 */
  HCAMD_MAP_MSQRT = 43,  /* numpy.sqrt of a tile: x < 0 -> inactive, value 0 */
  HCAMD_MAP_MLOG = 44    /* numpy.log of a tile: x <= 0 -> inactive, value 1 */
  /* 45 .. 55: the row programs' scalar forms (enum below) */
};
#define HCAMD_MAP_MAX_INPUTS 4
#define HCAMD_MAP_MAX_INSTRS 32
#define HCAMD_MAP_STACK_DEPTH 4
typedef struct HcamdMapInstr {
  uint16_t op;  /* HcamdMapOp */
  uint16_t arg; /* operand index for HCAMD_MAP_IN and the *_IN forms */
  float imm;    /* HCAMD_MAP_CONST and the *I forms */
} HcamdMapInstr;
int hcamdLaunchMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                   const void *const *inputs, const int *inputTypes,
                   const size_t *inputLd, size_t nInputs, void *out,
                   int outType, size_t ldo, size_t rows,
                   size_t cols) HCAMD_NOEXCEPT;

/* The integer sibling of hcamdLaunchMap: out = f(in_0 .. in_{n-1}) over a
 * rows x cols window of int32 operands, f a postfix program of HCAMD_IMAP_*
 * instructions on a four-entry stack (HcamdMapInstr with `imm` carrying the bit
 * pattern of an int32 constant).  These are the integer operators the
 * reference's tile wrapper forwards to NumPy
 * (python/hckernel/kernel_api.py:157-211) with NumPy's int32 semantics: + - *
 * wrap around, // and % are floor division and its remainder, << and >> with a
 * count outside 0..31 give 0 (-1 for >> of a negative value), comparisons give
 * 0 / 1.  An element that was divided by zero is inactive, as numpy.ma makes
 * it: nothing is stored for it.  outType is HCAMD_I32, or HCAMD_U8 for a
 * result of 0 / 1 stored as one byte (a bool buffer). */
enum HcamdIMapOp {
  HCAMD_IMAP_END = 0, HCAMD_IMAP_IN = 1, HCAMD_IMAP_CONST = 2,
  HCAMD_IMAP_ADD = 3, HCAMD_IMAP_SUB = 4, HCAMD_IMAP_MUL = 5, HCAMD_IMAP_FLOORDIV = 6,
  HCAMD_IMAP_MOD = 7, HCAMD_IMAP_MIN = 8, HCAMD_IMAP_MAX = 9, HCAMD_IMAP_AND = 10,
  HCAMD_IMAP_OR = 11, HCAMD_IMAP_XOR = 12, HCAMD_IMAP_SHL = 13, HCAMD_IMAP_SHR = 14,
  HCAMD_IMAP_LT = 15, HCAMD_IMAP_LE = 16, HCAMD_IMAP_EQ = 17, HCAMD_IMAP_NE = 18,
  HCAMD_IMAP_GE = 19, HCAMD_IMAP_GT = 20,
  HCAMD_IMAP_NEG = 21, HCAMD_IMAP_ABS = 22, HCAMD_IMAP_NOT = 23, HCAMD_IMAP_LNOT = 24,
  HCAMD_IMAP_ACTIVE = 25, /* top = 1 where the element is still active, else 0; the element is active again
                             (`tile.mask`, python/hckernel/kernel_api.py:117-119) */
  /* numpy.where(c, a, b) with c, a, b the three top entries (b on top): picked from
   * the values (the dividend under a failed //, 1 under a failed %); the element
   * is active again, as NumPy returns a plain array */
  HCAMD_IMAP_SELECT = 26,
  HCAMD_IMAP_COUNT = 27
};
int hcamdLaunchIMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                    const void *const *inputs, const size_t *inputLd, size_t nInputs,
                    void *out, int outType, size_t ldo, size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* The general float map: out = f(in_0 .. in_{n-1}) over a rows x cols window of
 * fp32 / fp16 operands with numpy.ma's activity rules, for what hcamdLaunchMap
 * leaves out of the operators the reference's tile wrapper forwards
 * (python/hckernel/kernel_api.py:157-211): // and %, the six comparisons, and
 * expressions in which the value numpy.ma leaves under a deactivated element
 * is seen again.  Activity is tracked per stack entry:
 *   ADD SUB MUL  tile operators: the first operand's value where an operand is
 *                inactive; `arg` bit 1: called as a NumPy function (computed
 *                from the values whatever their activity)
 *   DIV FLOORDIV tile operators / and //: inactive if the divisor is zero or the
 *                result is not finite (`arg` bit 0: tested as fp16), value
 *                0 + dividend; an active quotient has 0 * dividend added
 *   MOD, UDIV    % and numpy.divide as a function: inactive with the value 1
 *                where the divisor is zero or the dividend infinite (neither
 *                NaN), otherwise the remainder / the plain quotient
 *   SQRT LOG     numpy.sqrt / numpy.log: inactive with the value 0 / 1 where the
 *                operand is inactive or outside the domain
 *   PSQRT POWCHK x ** 0.5 (the operand's value where it is inactive), and
 *                numpy.ma.power's check: not finite -> inactive, value 1e20
 *   MIN MAX      numpy.minimum / maximum: a NaN wins; of two equal values (+0, -0)
 *                the second (`arg` bit 0, fp16 tiles: the first, as NumPy's half
 *                loops do)
 *   the rest     computed from the values, activity kept; comparisons give 0 / 1
 *   EQ NE        under an inactive result: 1 / 0 where both operands are inactive,
 *                0 / 1 where one is (numpy.ma compares the activity there);
 *                `arg` bit 1: numpy.equal / not_equal as functions, the values
 *   `arg` bit 3  on MIN MAX: the program evaluated the operands in the other
 *                order (which of two equal values wins depends on the order)
 *   `arg` bit 4  on a binary operation: the second operand's activity does not
 *                count (a bare numpy.ma array % tile: ndarray's operator converts
 *                the tile to its values)
 *   `arg` bit 2  on DIV FLOORDIV MOD UDIV SQRT LOG LOG2 LOG10: the operands are
 *                plain NumPy arrays (results of numpy.where, numpy.dot, tile.mask
 *                and arithmetic of those), so the operation is NumPy's own: IEEE
 *                results, nothing deactivated
 * An operand of type HCAMD_I32 is converted to fp32 when it is read (a tile's
 * astype(float32)).  Every rounding to fp16 other than DIV / FLOORDIV's is an explicit
 * HCAMD_FMAP_R16.  outType is HCAMD_F32, HCAMD_F16, or HCAMD_U8 (one byte of
 * 0 / 1, a bool buffer).  Inactive elements are not stored, unless storeAll is
 * set: a NumPy function returns a bare numpy.ma array, which the reference's
 * store writes out in full.  Programs have at most 48 instructions on a
 * four-entry stack. */
enum HcamdFMapOp {
  HCAMD_FMAP_END = 0, HCAMD_FMAP_IN = 1, HCAMD_FMAP_CONST = 2,
  HCAMD_FMAP_ADD = 3, HCAMD_FMAP_SUB = 4, HCAMD_FMAP_MUL = 5, HCAMD_FMAP_DIV = 6,
  HCAMD_FMAP_FLOORDIV = 7, HCAMD_FMAP_MOD = 8, HCAMD_FMAP_MIN = 9, HCAMD_FMAP_MAX = 10,
  HCAMD_FMAP_UDIV = 11,
  HCAMD_FMAP_LT = 12, HCAMD_FMAP_LE = 13, HCAMD_FMAP_EQ = 14, HCAMD_FMAP_NE = 15,
  HCAMD_FMAP_GE = 16, HCAMD_FMAP_GT = 17,
  HCAMD_FMAP_NEG = 18, HCAMD_FMAP_ABS = 19, HCAMD_FMAP_SQRT = 20, HCAMD_FMAP_RINT = 21,
  HCAMD_FMAP_EXP = 22, HCAMD_FMAP_LOG = 23, HCAMD_FMAP_R16 = 24, HCAMD_FMAP_PSQRT = 25,
  HCAMD_FMAP_POWCHK = 26,
  HCAMD_FMAP_ACTIVE = 27, /* top = 1 where the element is active in it, else 0; active again (`tile.mask`) */
  HCAMD_FMAP_TANH = 28,
  /* numpy.where(c, a, b) with c, a, b the three top entries (b on top): the
   * values are taken whatever their activity and the result is active, a plain
   * array as NumPy returns one */
  HCAMD_FMAP_SELECT = 29,
  /* more NumPy functions of one operand, computed from the values with the
   * activity kept; LOG2 and LOG10 have numpy.ma's domain like LOG */
  HCAMD_FMAP_FLOOR = 30, HCAMD_FMAP_CEIL = 31, HCAMD_FMAP_TRUNC = 32, HCAMD_FMAP_SIGN = 33,
  HCAMD_FMAP_EXP2 = 34, HCAMD_FMAP_LOG2 = 35, HCAMD_FMAP_LOG10 = 36, HCAMD_FMAP_LOG1P = 37,
  HCAMD_FMAP_EXPM1 = 38, HCAMD_FMAP_SIN = 39, HCAMD_FMAP_COS = 40, HCAMD_FMAP_RECIP = 41,
  /* `tile[:] = value` and the in-place operators of the reference's tiles
   * (python/hckernel/kernel_api.py:123-145: tile op= x is tile[:] = tile op x): of the
   * two top entries (the tile below, the value on top) the value where it is active, the
   * tile's own element elsewhere; active where either is */
  HCAMD_FMAP_MERGE = 42,
  HCAMD_FMAP_COUNT = 43
};
int hcamdLaunchFMap(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                    const void *const *inputs, const int *inputTypes, const size_t *inputLd,
                    size_t nInputs, void *out, int outType, size_t ldo, size_t rows,
                    size_t cols, int storeAll) HCAMD_NOEXCEPT;

/* Map-reduce: *cell += sum over the window of f(in_0 .. in_{n-1}), fp32, with
 * one hardware atomic add per workgroup.  This is the reference's reduction
 * idiom `atomic_ref(result)[0] += tile.sum()` with the tile an elementwise
 * expression of loads (python/hckernel/tests/test_examples.py:31-71;
 * atomic_ref: kernel_api.py:450-451).  The order of the additions is not
 * fixed, so two runs may differ in the last bits. */
int hcamdLaunchMapSum(OlQueue q, const HcamdMapInstr *prog, size_t nInstr,
                      const void *const *inputs, const int *inputTypes,
                      const size_t *inputLd, size_t nInputs, float *cell,
                      size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* Reductions along columns: out[c] = post(fold over the rows r of
 * f(in_0[r][c] .. in_{n-1}[r][c])) for a rows x cols window, i.e. the tile
 * methods the reference's simulator forwards to NumPy (`tile.sum(axis=0)`,
 * `max`, `min`, `mean`: python/hckernel/kernel_api.py:150-151) applied to an
 * elementwise expression of loads.  `prog` is a map program as for
 * hcamdLaunchMap; `kind` selects the fold (fp32 sum; maximum and minimum
 * propagate NaN like numpy.maximum / numpy.minimum); `post` (nPost may be 0)
 * is a map program with the folded value as its operand 0, e.g. the division
 * of a mean.  An operand with leading dimension 0 is a vector of cols elements
 * that every row uses.  `out` holds cols contiguous elements.  Rows are folded
 * in a fixed order: results do not change from run to run.  Windows with many
 * rows and few columns are cut into bands of rows whose results meet in
 * `workspace` (device memory, 16-byte aligned, at least
 * hcamdMapReduceColsWorkspace(rows, cols) bytes, a function of the shape alone;
 * that is 0 when one launch does it all and workspace may then be null).  The
 * launch allocates nothing.  The sums of x and of x * x down a dense fp32 window
 * of 256 columns or more are the commonest cases and fill their bands with a
 * kernel that interprets nothing, and the bands of any sum whose post program
 * only changes the folded value in place (at most four of ADDI SUBI MULI DIVI
 * RSUBI RDIVI NEG ABS SQRT after IN 0) into a dense fp32 result fold on another
 * (variant 1 of the "cols" family keeps the general one for both). */
enum HcamdColsKind { HCAMD_COLS_SUM = 0, HCAMD_COLS_MAX = 1, HCAMD_COLS_MIN = 2 };
#define HCAMD_COLS_MAX_POST 8
size_t hcamdMapReduceColsWorkspace(size_t rows, size_t cols) HCAMD_NOEXCEPT;
int hcamdLaunchMapReduceCols(OlQueue q, int kind, const HcamdMapInstr *prog, size_t nInstr,
                             const HcamdMapInstr *post, size_t nPost,
                             const void *const *inputs, const int *inputTypes,
                             const size_t *inputLd, size_t nInputs, void *out,
                             int outType, size_t rows, size_t cols, void *workspace,
                             size_t workspaceBytes) HCAMD_NOEXCEPT;

/* hcamdLaunchMapReduceCols for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments and results
 * (bit for bit) without the workspace: the bands meet in a static device array
 * of HCAMD_NOALLOC_SCRATCH_BYTES that each GPU the library runs on holds until
 * the process ends; its address is looked up when the device is created
 * (olCreateDevice), where the kernels are resolved too, so the call itself
 * allocates and loads nothing.  A window whose
 * hcamdMapReduceColsWorkspace(rows, cols) exceeds the limit is refused with a
 * message (the workspace never exceeds about 3.1 MiB for any window the
 * kernel accepts today; the limit is what protects a change of that).  All
 * calls on one GPU share the array: calls that overlap on one GPU (two
 * queues, two threads) race; calls on one queue are ordered and safe. */
#define HCAMD_NOALLOC_SCRATCH_BYTES ((size_t)4 << 20)
int hcamdLaunchMapReduceColsNoAlloc(OlQueue q, int kind, const HcamdMapInstr *prog,
                                    size_t nInstr, const HcamdMapInstr *post, size_t nPost,
                                    const void *const *inputs, const int *inputTypes,
                                    const size_t *inputLd, size_t nInputs, void *out,
                                    int outType, size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* Row programs: bodies that mix elementwise arithmetic with reductions along
 * the rows of a 2-D tile, e.g. the reference's row softmax
 * (python/hckernel/tests/test_examples.py:304-336:
 * exp = np.exp(x - x.max(axis=1, keepdims=True)); exp / exp.sum(axis=1, keepdims=True)),
 * normalisations, row sums.  The expression is a list of stages; each stage is
 * a postfix program in the instruction set of hcamdLaunchMap (its instructions
 * follow the previous stage's in `prog`) and ends in one of:
 *   SUM, MAX, MIN  the value at every element of a row is folded into row
 *                  scalar `dst` of that row (fp32; MAX/MIN propagate NaN)
 *   SCALAR         the program reads row scalars only; its value becomes row
 *                  scalar `dst`
 *   STORE          the value at every element is stored to out[row, col]
 *   STORE_COL      as SCALAR, stored to out[row * ldo]; with dst = 1 a row whose
 *                  result is deactivated is not stored (the value is a tile: a
 *                  per-row operand on the left of the tile operators)
 *   COUNT          the number of active elements of the value (see below) becomes
 *                  row scalar `dst` (fp32)
 * Exactly one stage stores, and it is the last.  Programs read row scalars with
 * HCAMD_MAP_RED (push) and the *_RED forms (top = top op scalar), only scalars
 * that an earlier stage or a column operand has written.
 * Activity follows numpy.ma, to which the reference's tiles forward their
 * operators and reductions (python/hckernel/kernel_api.py:150-180).  Elements
 * that the masked forms (HCAMD_MAP_MDIV .. MLOG) deactivate are neither stored
 * nor folded, and are not counted.  A fold over a row without any active
 * element is a deactivated row scalar (holding 0 for a sum, 1e20 for a maximum
 * or minimum); so is the result of a SCALAR stage in which a masked form fails
 * (a quotient that is not finite, a root of a negative number) or that reads a
 * deactivated row scalar.  Every element of a stage that reads a deactivated
 * row scalar is inactive.  STORE_COL stores every row, a deactivated one with
 * the value numpy.ma leaves in it: in SCALAR / STORE_COL stages + - * leave
 * their first operand's value there, the quotient leaves the dividend, NumPy
 * functions compute regardless (sqrt and log give their fill values 0 and 1).
 * For that, `arg` of the instructions of those stages carries three more flags:
 * 0x200, the operation was called as a NumPy function; 0x400, a commutative
 * operation whose running value (the stack top of an immediate or *_RED form,
 * the deeper entry of a stack form) is its second operand; 0x800, a unary
 * operation that leaves a deactivated value as it is (the square root of
 * x ** 0.5: numpy.ma.power keeps its operand where that is inactive).  HCAMD_MAP_RED0
 * pushes a row scalar's value whether deactivated or not (numpy.ma's variance
 * reads the sum of the centred squares that way: 0 if all of them were
 * inactive); HCAMD_MAP_MASQRT is numpy.ma.sqrt (the standard deviation's: a
 * result that is not finite deactivates and leaves the argument);
 * HCAMD_MAP_LIVEPOS, as the last instruction of a SCALAR stage, replaces the
 * result's activity: active iff row scalar `arg` is positive (a variance is
 * active where count - ddof is).  HCAMD_MAP_FROZEN, as the last instruction of
 * a STORE stage, makes that stage store every element, a deactivated one with
 * the value numpy.ma leaves in it (the stored expression is a bare numpy.ma
 * array and a tile operator follows an operation that can deactivate): the
 * stage's program must push one value and change it in place, and its
 * instructions carry the two form flags like those of SCALAR stages.
 * Operands: `inputs` are rows x cols tiles with a leading dimension in elements,
 * or, with leading dimension 0, one vector of cols elements used for every row;
 * `columns` hold one value per row and fill row scalars 0 .. nColumns-1.
 * A row is handled by one wave (cols <= 4096) or one workgroup; every stage
 * reads the operands it uses again (a row just read is still in L2).  Programs
 * whose stages all change one value in place (an operand, then *I, *_IN, *_RED
 * and unary forms; `x x MUL` with two equal halves counts) over 16-byte aligned
 * rows of whole chunks of 8 elements, at most 32768 elements, run on kernels that
 * take a lane's whole part of the row at once: the operand most instructions
 * read is fetched once per row (into LDS), and an instruction is dispatched
 * once for 8, 16 or 32 elements of a lane; a program in which only operations
 * on row scalars can deactivate anything (a quotient, a root, a logarithm, a
 * power) runs there too, followed by a launch of the general kernel for the
 * rows on which one did, which the first launch leaves untouched and marks in
 * a byte array the device keeps (one byte per row, at least 64 KiB: the first
 * such launch on a device allocates it with hipMalloc and a launch with more
 * rows than any before replaces it, so callers that cannot allocate, a stream
 * under capture among them, select variant 3 of "rows": the general kernel alone
 * for such programs; variant 1 of the "rows" family keeps the general kernel
 * for every program).  One program has a kernel of its own that interprets
 * nothing: the layer normalisation (x - mean) / sqrt(var + eps) * w + b in the
 * six stages the front-end emits for it (sum; RED MDIVI; the sum of the
 * centred squares; RED0 DIVI; RED ADDI MSQRT; IN SUB_RED MDIV_RED MUL_IN
 * ADD_IN) on dense fp32 rows of at most 32768 elements with fp32 vectors w and
 * b: the same operations per element, the row read once, nothing stored to a
 * row whose mean is not finite; and so has the root-mean-square normalisation
 * x / sqrt(mean(x * x) + eps) * w in its three stages (IN MUL_IN summed; RED
 * MDIVI ADDI MSQRT; IN MDIV_RED MUL_IN; with R16 at the end on fp16 rows of
 * whole chunks of 8 with an fp32 w) under the same conditions (variant 2 of
 * "rows" keeps both on the kernels above).  Programs in which a row scalar can
 * be deactivated, or that count, run on the general kernel.  Sums add in an order that
 * depends on the shape and the kernel only: results are reproducible, and agree with a
 * sequential fp32 sum to within the usual n * 2^-24 bound. */
enum HcamdRowStageKind {
  HCAMD_ROW_SUM = 0,
  HCAMD_ROW_MAX = 1,
  HCAMD_ROW_MIN = 2,
  HCAMD_ROW_SCALAR = 3,
  HCAMD_ROW_STORE = 4,
  HCAMD_ROW_STORE_COL = 5,
  HCAMD_ROW_COUNT = 6
};
enum {
  HCAMD_MAP_RED = 45,     /* push row scalar `arg` */
  HCAMD_MAP_ADD_RED = 46, /* top = top + row scalar `arg` */
  HCAMD_MAP_SUB_RED = 47,
  HCAMD_MAP_MUL_RED = 48,
  HCAMD_MAP_DIV_RED = 49,
  HCAMD_MAP_MAX_RED = 50,
  HCAMD_MAP_MIN_RED = 51,
  HCAMD_MAP_RSUB_RED = 52, /* scalar - top */
  HCAMD_MAP_RDIV_RED = 53, /* scalar / top */
  /* the tile operator / with a row scalar under numpy.ma's rule (see
   * HCAMD_MAP_MDIV): `arg` bits 0..3 the scalar, bit 8 the fp16 flag */
  HCAMD_MAP_MDIV_RED = 54, /* top / scalar */
  HCAMD_MAP_RMDIV_RED = 55, /* scalar / top */
  HCAMD_MAP_RED0 = 56,    /* SCALAR / STORE_COL stages: push row scalar `arg`, deactivated or not */
  HCAMD_MAP_MASQRT = 57,  /* SCALAR / STORE_COL stages: numpy.ma.sqrt */
  HCAMD_MAP_LIVEPOS = 58, /* closes a SCALAR stage: active iff row scalar `arg` > 0 */
  HCAMD_MAP_FROZEN = 59   /* closes a STORE stage: every element is stored (see above) */
};
#define HCAMD_ROW_MAX_STAGES 16
#define HCAMD_ROW_MAX_SCALARS 16
#define HCAMD_ROW_MAX_INSTRS 128
typedef struct HcamdRowStage {
  uint32_t kind;   /* HcamdRowStageKind */
  uint32_t nInstr; /* instructions of this stage */
  uint32_t dst;    /* row scalar written by SUM, MAX, MIN, SCALAR */
} HcamdRowStage;
int hcamdLaunchRowProgram(OlQueue q, const HcamdMapInstr *prog,
                          const HcamdRowStage *stages, size_t nStages,
                          const void *const *inputs, const int *inputTypes,
                          const size_t *inputLd, size_t nInputs,
                          const void *const *columns, const int *columnTypes,
                          size_t nColumns, void *out, int outType, size_t ldo,
                          size_t rows, size_t cols) HCAMD_NOEXCEPT;

/* Pairwise Euclidean distances, fp32: out[i, j] = sqrt(sum_k (a[i,k] - b[j,k])^2)
 * for a[m, d], b[n, d] row-major, out[m, n].  The expression of
 * python/hckernel/tests/test_examples.py:270-301
 * (numpy.linalg.norm(a[:, None, :] - b[None, :, :], axis=2)); differences are
 * formed explicitly, sums run over d in ascending order per output. */
int hcamdLaunchPairwiseDistF32(OlQueue q, const float *a, size_t lda,
                               const float *b, size_t ldb, float *out,
                               size_t ldo, size_t m, size_t n,
                               size_t d) HCAMD_NOEXCEPT;

/* Matrix product of gathered tiles, fp32 -- the operation of a kernel body that
 * loads its operands through index mappings and multiplies them
 * (CurrentGroup.load / store with mapping=..., python/hckernel/kernel_api.py:297-345;
 * the implicit-GEMM convolution of python/hckernel/tests/test_examples.py:168-258):
 *
 *     out_g[mo(i, j)] = sum_k a_g[ma(i, k)] * b_g[mb(k, j)]       for every group g
 *
 * x_g is the window of buffer x that starts at starts[g][d] along dimension d
 * (the `x[s0:, s1:, ...]` of the body).  Element (r, c) of a tile sits at index
 * rowIndex[r][d] + colIndex[c][d] of the window; for every dimension one of
 * the two tables must be all zero (the index depends on the tile row or on the
 * tile column, not on both).  An element is active if
 * 0 <= index < shape[d] - starts[g][d] for every d, which is the reference's
 * bounds test; inactive operand elements count as zero, inactive output
 * elements are not written.  The a tile is tm x k, the b tile k x tn, the out
 * tile tm x tn.  Two active out elements of one launch must not share a
 * destination (their order is not defined).
 *
 * hcamdGatherGemmCreate checks the description, builds the device tables and
 * returns a plan (NULL after reporting an error); it allocates device memory
 * (the tables and a scratch array of one packed k x tn tile per distinct b
 * window, about the size of b) and synchronises.  hcamdGatherGemmLaunchF32
 * enqueues one launch of the plan (two kernels: the b tiles are packed, then
 * multiplied) on buffers that have the shapes and strides given at creation;
 * it neither allocates nor synchronises.  Launches of one plan share its
 * scratch array: enqueue them on one queue, or wait between them.  Groups run in
 * an order the plan chooses (by window address).  All pointers in
 * HcamdGatherOperand are host memory and are not kept. */
typedef struct HcamdGatherOperand {
  int ndim;               /* 1..4 */
  size_t shape[4];        /* elements per dimension of the whole buffer */
  size_t strides[4];      /* in elements */
  const int32_t *starts;  /* [nGroups][ndim], >= 0 */
  const int32_t *rowIndex; /* [tile rows][ndim] */
  const int32_t *colIndex; /* [tile cols][ndim] */
} HcamdGatherOperand;
typedef struct HcamdGatherGemm_ *HcamdGatherGemm;
HcamdGatherGemm hcamdGatherGemmCreate(OlQueue q, const HcamdGatherOperand *a,
                                      const HcamdGatherOperand *b,
                                      const HcamdGatherOperand *out,
                                      size_t nGroups, size_t tm, size_t tn,
                                      size_t k) HCAMD_NOEXCEPT;
int hcamdGatherGemmLaunchF32(OlQueue q, HcamdGatherGemm plan, const float *a,
                             const float *b, float *out) HCAMD_NOEXCEPT;
/* The same for buffers of another storage type (HcamdElemType; a, b and out
 * alike): elements are widened to fp32 when read, products and sums are fp32,
 * the result is rounded to nearest even when stored. */
int hcamdGatherGemmLaunch(OlQueue q, HcamdGatherGemm plan, int elemType,
                          const void *a, const void *b,
                          void *out) HCAMD_NOEXCEPT;
void hcamdGatherGemmRelease(HcamdGatherGemm plan) HCAMD_NOEXCEPT;

/* Elementwise expressions of gathered tiles -- what a body computes that loads
 * tiles through index mappings, or stores one through a mapping, outside a
 * matrix product (CurrentGroup.load / store with mapping=...,
 * python/hckernel/kernel_api.py:304-310,319-335):
 *
 *     out_g[mo(e)] = f(in0_g[m0(e)], in1_g[m1(e)], ...)     for every group g, tile element e
 *
 * x_g is the window of buffer x that starts at starts[g][d] along dimension d;
 * element e of a tile (row-major) sits at index[e][d] of the window and is
 * active if 0 <= index[e][d] < shape[d] - starts[g][d] for every d, the
 * reference's bounds test; an operand without a mapping has the identity table.
 * f is a program of hcamdLaunchFMap with its activity rules: an inactive operand
 * element is a zero that deactivates what is computed from it; an inactive
 * output position is not written, and neither is a deactivated result unless
 * storeAll: 1 writes the value the program leaves there, 2 writes NaN (a float
 * out) or 0 (a bool out), which is what NumPy makes of numpy.ma's masked
 * constant when the reference stores a bare numpy.ma array through a mapping
 * (python/hckernel/kernel_api.py:331-334).  With copyBytes != 0 (1, 2, 4 or 8) there is no program: operand 0
 * is copied element by element whatever its type (a gathered / scattered copy).
 * Two active out elements of one launch must not share a destination (their
 * order is not defined).  `operands` holds the nInputs inputs, then the output;
 * all pointers in it are host memory and are not kept.  Create allocates device
 * memory for the tables and synchronises; Launch neither allocates nor
 * synchronises. */
typedef struct HcamdGatherMapOperand {
  int ndim;              /* 1..4 */
  size_t shape[4];       /* elements per dimension of the whole buffer */
  size_t strides[4];     /* in elements */
  const int32_t *starts; /* [nGroups][ndim], >= 0 */
  const int32_t *index;  /* [tileElems][ndim] */
} HcamdGatherMapOperand;
typedef struct HcamdGatherMap_ *HcamdGatherMap;
HcamdGatherMap hcamdGatherMapCreate(OlQueue q, const HcamdGatherMapOperand *operands, size_t nInputs,
                                    size_t nGroups, size_t tileElems) HCAMD_NOEXCEPT;
int hcamdGatherMapLaunch(OlQueue q, HcamdGatherMap plan, const HcamdMapInstr *prog, size_t nInstr,
                         const void *const *inputs, const int *inputTypes, void *out, int outType,
                         int storeAll, size_t copyBytes) HCAMD_NOEXCEPT;
void hcamdGatherMapRelease(HcamdGatherMap plan) HCAMD_NOEXCEPT;

/* Row softmax, fp32: y[r,:] = exp(x[r,:]-max(x[r,:])) / sum(exp(...)).
 * Expression of python/hckernel/tests/test_examples.py:330-335. */
int hcamdLaunchSoftmaxF32(OlQueue q, const float *x, size_t ldx, float *y,
                          size_t ldy, size_t rows,
                          size_t cols) HCAMD_NOEXCEPT;

/* Row-wise symmetric int8 quantisation of fp16 rows:
 * scale[r] = max|x[r,:]| / 127 (fp32), q = clamp(rint((float)x / scale[r]),
 * -127, 127) with IEEE division and round-half-even.  A row whose absmax is
 * zero gets scale 0 and q 0.  A row holding NaN gets scale NaN and q 0; an
 * infinite absmax gives scale inf, q 0 for finite x and 0 for the infinite
 * entries too (inf/inf is NaN). */
int hcamdLaunchQuantizeF16I8(OlQueue q, const void *x, size_t ldx, int8_t *qout,
                             size_t ldq, float *scale, size_t rows,
                             size_t cols) HCAMD_NOEXCEPT;

/* C[M,N] = A[M,K] * B[K,N]; A row-major bf16 (lda), B column-major bf16 given
 * as Bt[N,K] row-major (ldb), fp32 accumulation on MFMA, C row-major bf16
 * (ldc), round to nearest even.  Any M, N, K >= 1.  The matrix-core kernels
 * take every shape whose K-contiguous rows can be fetched in 16-byte pieces
 * (A and Bt 16-byte aligned, lda, ldb and K multiples of 8, K > 64): M and N
 * need not be multiples of the tile, C may have any leading dimension.  Other
 * shapes (odd K or leading dimensions, K <= 64) run a much slower general
 * kernel. */
int hcamdLaunchGemmBF16(OlQueue q, const void *a, size_t lda, const void *bt,
                        size_t ldb, void *c, size_t ldc, size_t m, size_t n,
                        size_t k) HCAMD_NOEXCEPT;

/* The same product with fp16 storage (A, Bt, C) and the fp16 MFMA: the dtype
 * NumPy has natively, so the reference's blocked-dot example
 * (python/hckernel/tests/test_examples.py:124-165, written with Bt) can be run
 * on both sides. */
int hcamdLaunchGemmF16(OlQueue q, const void *a, size_t lda, const void *bt,
                       size_t ldb, void *c, size_t ldc, size_t m, size_t n,
                       size_t k) HCAMD_NOEXCEPT;

/* Chooses between kernel variants of one family by number (0 = default
 * choice by shape).  For tuning and measurement; family names are "add",
 * "fma", "softmax", "quantize", "gemm", "copy", "map", "rows", "cols", "stream", "norm"
 * (lanes to a row in the normalisation kernels: 1 twice, 2 half as many), "gather"
 * (block shape), "gather_fuse" (groups per workgroup; read by
 * hcamdGatherGemmCreate).
 * Process-wide, guarded by a lock.  Returns 1 for an unknown family, and for
 * the numbers of the measurement builds of the "gemm" family (17..22, 26, 28..34:
 * most of them leave something other than the product in C) unless the library was built with them
 * (hc_amd_bench.h).  Every variant a default build accepts computes the same
 * result as variant 0. */
int hcamdSetVariant(const char *family, int variant) HCAMD_NOEXCEPT;
/* The same choice for the calling thread only: it takes precedence over
 * hcamdSetVariant for launches made by this thread and is invisible to others
 * (variant < 0 removes it).  What a tuned kernel object uses around its own
 * launches, so that threads launching differently tuned kernels do not race
 * and a process-wide choice is left as it was. */
int hcamdSetThreadVariant(const char *family, int variant) HCAMD_NOEXCEPT;

/* Name and launch geometry of the kernel the most recent typed launcher
 * enqueued on this thread (for reports and profiles). */
const char *hcamdLastKernelName(void) HCAMD_NOEXCEPT;

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* HC_AMD_RUNTIME_H */
