// Masked tile copy: dst[window] = src[window], every byte of dst outside the
// window untouched.  Three forms:
//   * flat    - both sides contiguous: one vector of 16-byte words plus a byte
//               tail (same structure as the flat elementwise maps);
//   * 2-D     - arbitrary element strides, one element per work-item;
//   * tiled   - the reference's own decomposition: a (by, bx*unroll) tile per
//               workgroup, one element per work-item per load, launched with
//               the grid and block the reference would use.  Its argument list
//               follows the reference's generated kernel (block dim, source
//               row stride, source pointer, rows, cols, destination row stride,
//               destination pointer), with the unroll factor in the first slot.
//   * fill32  - dst[i] = value for 32-bit words.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kThreads = 256;

template <int VPT, bool NT>
__device__ __forceinline__ void copy_flat(const uint8_t *src, uint8_t *dst,
                                          size_t nbytes) {
  const size_t nvec = nbytes / 16;
  const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
  u32x4 *d = reinterpret_cast<u32x4 *>(dst);
  const size_t first = (size_t)blockIdx.x * (kThreads * VPT) + threadIdx.x;
  if (((size_t)blockIdx.x + 1) * (kThreads * VPT) <= nvec) {
    u32x4 v[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      v[j] = ldg<NT>(s + first + (size_t)j * kThreads);
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      stg<NT>(d + first + (size_t)j * kThreads, v[j]);
    return;
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t w = first + (size_t)j * kThreads;
    if (w < nvec)
      d[w] = s[w];
  }
  const size_t e = nvec * 16 + threadIdx.x;
  if (threadIdx.x < 16 && e < nbytes)
    dst[e] = src[e];
}

template <class T>
__device__ __forceinline__ void copy_2d(const T *src, ptrdiff_t ss0,
                                        ptrdiff_t ss1, T *dst, ptrdiff_t ds0,
                                        ptrdiff_t ds1, size_t rows,
                                        size_t cols) {
  const size_t col = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t row = (size_t)blockIdx.y * blockDim.y + threadIdx.y;
  if (col < cols && row < rows)
    dst[(ptrdiff_t)row * ds0 + (ptrdiff_t)col * ds1] =
        src[(ptrdiff_t)row * ss0 + (ptrdiff_t)col * ss1];
}

template <class T>
__device__ __forceinline__ void copy_tiled(int64_t unroll, int64_t ss0,
                                           const T *src, int64_t rows,
                                           int64_t cols, int64_t ds0, T *dst) {
  const int64_t row = (int64_t)blockIdx.y * blockDim.y + threadIdx.y;
  const int64_t tile0 = (int64_t)blockIdx.x * blockDim.x * unroll;
  if (row >= rows)
    return;
  for (int64_t u = 0; u < unroll; ++u) {
    const int64_t col = tile0 + u * blockDim.x + threadIdx.x;
    if (col < cols)
      dst[row * ds0 + col] = src[row * ss0 + col];
  }
}
} // namespace

#define HCAMD_COPY_FLAT(NAME, VPT, NT)                                         \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const uint8_t *src, uint8_t *dst, size_t nbytes) {                       \
    copy_flat<VPT, NT>(src, dst, nbytes);                                      \
  }
HCAMD_COPY_FLAT(hcamd_copy_flat_v1, 1, false)
HCAMD_COPY_FLAT(hcamd_copy_flat_v2, 2, false)
HCAMD_COPY_FLAT(hcamd_copy_flat_v4, 4, false)
HCAMD_COPY_FLAT(hcamd_copy_flat_v8, 8, false)
HCAMD_COPY_FLAT(hcamd_copy_flat_v1_nt, 1, true)
HCAMD_COPY_FLAT(hcamd_copy_flat_v2_nt, 2, true)
HCAMD_COPY_FLAT(hcamd_copy_flat_v4_nt, 4, true)
HCAMD_COPY_FLAT(hcamd_copy_flat_v8_nt, 8, true)

#define HCAMD_COPY_2D(NAME, T)                                                 \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const T *src, ptrdiff_t ss0, ptrdiff_t ss1, T *dst, ptrdiff_t ds0,       \
      ptrdiff_t ds1, size_t rows, size_t cols) {                               \
    copy_2d<T>(src, ss0, ss1, dst, ds0, ds1, rows, cols);                      \
  }
HCAMD_COPY_2D(hcamd_copy2d_b1, uint8_t)
HCAMD_COPY_2D(hcamd_copy2d_b2, uint16_t)
HCAMD_COPY_2D(hcamd_copy2d_b4, uint32_t)
HCAMD_COPY_2D(hcamd_copy2d_b8, uint64_t)
HCAMD_COPY_2D(hcamd_copy2d_b16, u32x4)

// Windows whose rows are contiguous inside and lie the same way against 16-byte
// boundaries in both arrays, whatever the element size and however ragged the
// ends: a lane owns one aligned 16-byte piece of the destination row and moves
// it whole, or, at the two ends of the row, the bytes of it that belong to the
// window.  (An int32 window of odd width or offset otherwise moves 4 bytes per
// lane: 8191 x 8191 of a stride-8200 array 160 us, a uint8 one 1 byte per lane.)
// ANY: the source rows lie differently from the destination rows; the 16 bytes of
// a piece are then read from wherever they are (the compiler is told nothing
// about their alignment and emits what the target allows for that).
template <bool ANY>
__device__ __forceinline__ void copy_rows(
    const uint8_t *src, ptrdiff_t src_row_bytes, uint8_t *dst, ptrdiff_t dst_row_bytes,
    size_t rows, size_t row_bytes) {
  const size_t row = (size_t)blockIdx.y * blockDim.y + threadIdx.y;
  if (row >= rows)
    return;
  const uint8_t *s0 = src + (ptrdiff_t)row * src_row_bytes;
  uint8_t *d0 = dst + (ptrdiff_t)row * dst_row_bytes;
  const ptrdiff_t lead = (ptrdiff_t)(reinterpret_cast<uintptr_t>(d0) & 15);
  const ptrdiff_t piece = (ptrdiff_t)((size_t)blockIdx.x * blockDim.x + threadIdx.x);
  const ptrdiff_t b0 = piece * 16 - lead, b1 = b0 + 16, end = (ptrdiff_t)row_bytes;
  if (b0 >= end)
    return;
  if (b0 >= 0 && b1 <= end) {
    u32x4 v;
    if constexpr (ANY)
      __builtin_memcpy(&v, s0 + b0, 16);
    else
      v = ldg<true>(reinterpret_cast<const u32x4 *>(s0 + b0));
    stg<true>(reinterpret_cast<u32x4 *>(d0 + b0), v);
    return;
  }
  const ptrdiff_t lo = b0 < 0 ? 0 : b0, hi = b1 < end ? b1 : end;
  for (ptrdiff_t b = lo; b < hi; ++b)
    d0[b] = s0[b];
}
extern "C" __global__ __launch_bounds__(256) void hcamd_copy2d_rows(
    const uint8_t *src, ptrdiff_t src_row_bytes, uint8_t *dst, ptrdiff_t dst_row_bytes,
    size_t rows, size_t row_bytes) {
  copy_rows<false>(src, src_row_bytes, dst, dst_row_bytes, rows, row_bytes);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_copy2d_rows_any(
    const uint8_t *src, ptrdiff_t src_row_bytes, uint8_t *dst, ptrdiff_t dst_row_bytes,
    size_t rows, size_t row_bytes) {
  copy_rows<true>(src, src_row_bytes, dst, dst_row_bytes, rows, row_bytes);
}

#define HCAMD_COPY_TILED(NAME, T)                                              \
  extern "C" __global__ __launch_bounds__(1024) void NAME(                     \
      int64_t unroll, int64_t ss0, const T *src, int64_t rows, int64_t cols,   \
      int64_t ds0, T *dst) {                                                   \
    copy_tiled<T>(unroll, ss0, src, rows, cols, ds0, dst);                     \
  }
HCAMD_COPY_TILED(hcamd_copy2d_tiled_b1, uint8_t)
HCAMD_COPY_TILED(hcamd_copy2d_tiled_b2, uint16_t)
HCAMD_COPY_TILED(hcamd_copy2d_tiled_b4, uint32_t)
HCAMD_COPY_TILED(hcamd_copy2d_tiled_b8, uint64_t)
HCAMD_COPY_TILED(hcamd_copy2d_tiled_b16, u32x4)

// ---------------------------------------------------------------------------
// dst[c][r] = src[r][c] over a rows x cols window of src (what a body stores
// that writes a tile's .T to the transposed window): 64 x 64 elements per
// workgroup through LDS, read along the rows of src and written along the rows
// of dst, 64 lanes to a row piece both ways; a pad column keeps the column
// reads of the LDS tile off one bank.  Leading dimensions in elements.
// ---------------------------------------------------------------------------
namespace {
template <class T>
__device__ __forceinline__ void transpose_tile(const T *__restrict__ src, size_t lds, T *__restrict__ dst,
                                               size_t ldd, uint32_t rows, uint32_t cols) {
  __shared__ T tile[64][65];
  const uint32_t tx = threadIdx.x % 64, ty = threadIdx.x / 64;   // 64 x 4 lanes
  const uint32_t r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
#pragma unroll
  for (uint32_t k = 0; k < 64; k += 4) {
    const uint32_t r = r0 + ty + k, c = c0 + tx;
    if (r < rows && c < cols)
      tile[ty + k][tx] = src[(size_t)r * lds + c];
  }
  __syncthreads();
#pragma unroll
  for (uint32_t k = 0; k < 64; k += 4) {
    const uint32_t c = c0 + ty + k, r = r0 + tx;                 // a row of dst is a column of src
    if (c < cols && r < rows)
      dst[(size_t)c * ldd + r] = tile[tx][ty + k];
  }
}
} // namespace
#define HCAMD_TRANSPOSE(NAME, T)                                                            \
  extern "C" __global__ __launch_bounds__(256) void NAME(const T *src, size_t lds, T *dst,   \
                                                         size_t ldd, uint32_t rows, uint32_t cols) { \
    transpose_tile<T>(src, lds, dst, ldd, rows, cols);                                      \
  }
HCAMD_TRANSPOSE(hcamd_transpose2d_b1, uint8_t)
HCAMD_TRANSPOSE(hcamd_transpose2d_b2, uint16_t)
HCAMD_TRANSPOSE(hcamd_transpose2d_b4, uint32_t)
HCAMD_TRANSPOSE(hcamd_transpose2d_b8, uint64_t)

// ---------------------------------------------------------------------------
// Stream calibration: what HBM delivers for a given mix of read and write
// streams when nothing else is in the way.  R input vectors of 16-byte words
// are added lane by lane (32-bit wrap-around) and
//   W = 1: the sum word is written (16 bytes out per 16 bytes of each input),
//   W = 2: its halves are xor-ed and 8 bytes written (the 2:1 byte ratio of the
//          int8 quantiser),
//   W = 0: nothing is written but one 32-bit sum per workgroup (a read-only
//          stream with a checkable result).
// With R = 0 the kernel writes the word index (a fill).  A workgroup of 512
// lanes owns 1024 consecutive words, two per lane, non-temporal both ways: the
// structure that measured fastest for every mix.  The launcher passes whole
// workgroups only (bytes a multiple of 16 KiB).
template <int R, int W, int kT = 512, int kVpt = 2, int DELAY = -1>
__device__ __forceinline__ void stream_mix(const u32x4 *a, const u32x4 *b, const u32x4 *c,
                                           void *out) {
  const u32x4 *in[3] = {a, b, c};
  const size_t first = (size_t)blockIdx.x * (kT * kVpt) + threadIdx.x;
  u32x4 v[kVpt][R > 0 ? R : 1];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < kVpt; ++j)
      v[j][r] = ldg<true>(in[r] + first + (size_t)j * kT);
  if constexpr (DELAY >= 0 && R > 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (DELAY > 0)
      __builtin_amdgcn_s_sleep(DELAY);
  }
  uint32_t total = 0;
#pragma unroll
  for (int j = 0; j < kVpt; ++j) {
    const uint32_t w = (uint32_t)(first + (size_t)j * kT);
    u32x4 s = R ? v[j][0] : u32x4{w, w, w, w};
    // (written out: as a loop over r the compiler drops the non-temporal
    // marking of the store when kVpt is 1)
    if constexpr (R >= 2)
      s += v[j][1];
    if constexpr (R >= 3)
      s += v[j][2];
    if constexpr (W == 1) {
      stg<true>(static_cast<u32x4 *>(out) + first + (size_t)j * kT, s);
    } else if constexpr (W == 2) {
      const u32x2 h = {s[0] ^ s[1], s[2] ^ s[3]};
      stg<true>(static_cast<u32x2 *>(out) + first + (size_t)j * kT, h);
    } else {
      total += s[0] + s[1] + s[2] + s[3];
    }
  }
  if constexpr (W == 0) {
    __shared__ uint32_t slots[kT / kWave];
    struct USum {
      using T = uint32_t;
      static __device__ __forceinline__ uint32_t identity() { return 0u; }
      static __device__ __forceinline__ uint32_t apply(uint32_t x, uint32_t y) { return x + y; }
    };
    total = group_reduce<USum, kT / kWave>(total, slots);
    if (threadIdx.x == 0)
      static_cast<uint32_t *>(out)[blockIdx.x] = total;
  }
}
#define HCAMD_STREAM(NAME, R, W)                                               \
  extern "C" __global__ __launch_bounds__(512) void NAME(                      \
      const u32x4 *a, const u32x4 *b, const u32x4 *c, void *out) {             \
    stream_mix<R, W>(a, b, c, out);                                            \
  }
HCAMD_STREAM(hcamd_stream_r1w0, 1, 0)
HCAMD_STREAM(hcamd_stream_r0w1, 0, 1)
HCAMD_STREAM(hcamd_stream_r1w1, 1, 1)
HCAMD_STREAM(hcamd_stream_r2w1, 2, 1)
HCAMD_STREAM(hcamd_stream_r3w1, 3, 1)
HCAMD_STREAM(hcamd_stream_r1w1h, 1, 2)

// The same mixes paced as the fp16 fma kernel is: 256 lanes, one word each, REG
// the highest register touched (127: four waves per SIMD), DELAY * 64 clocks
// between the arrival of a wave's words and its store (-1: no wait at all).
// Only the mixes that both read and write have such forms.
#define HCAMD_STREAM_PACED(NAME, R, W, REG, DELAY)                             \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const u32x4 *a, const u32x4 *b, const u32x4 *c, void *out) {             \
    asm volatile("v_mov_b32 v" #REG ", 0" ::: "v" #REG);                       \
    stream_mix<R, W, 256, 1, DELAY>(a, b, c, out);                             \
  }
#define HCAMD_STREAM_PACED_ALL(SUFFIX, REG, DELAY)                             \
  HCAMD_STREAM_PACED(hcamd_stream_r1w1##SUFFIX, 1, 1, REG, DELAY)              \
  HCAMD_STREAM_PACED(hcamd_stream_r2w1##SUFFIX, 2, 1, REG, DELAY)              \
  HCAMD_STREAM_PACED(hcamd_stream_r3w1##SUFFIX, 3, 1, REG, DELAY)              \
  HCAMD_STREAM_PACED(hcamd_stream_r1w1h##SUFFIX, 1, 2, REG, DELAY)
HCAMD_STREAM_PACED_ALL(_w4_d6, 127, 6)
HCAMD_STREAM_PACED_ALL(_w4_d0, 127, 0)
HCAMD_STREAM_PACED_ALL(_w4_d12, 127, 12)
HCAMD_STREAM_PACED_ALL(_w8, 63, -1)

// ---------------------------------------------------------------------------
// Ids as data: out[index(g, l)] = value(g, l), both affine in the group id g and
// the local id l, for every work-item (per_item) or once per group.  Launched
// with the reference's own geometry (block = group shape, grid = group counts,
// last Python dimension on x: mlir/lib/Transforms/LowerHKernel.cpp:284-367), so
// the hardware ids ARE the ids of the programming model
// (python/hckernel/kernel.py:97-131: work_offset = group_id * group_shape,
// global id = work_offset + local_id).  An index outside the buffer stores
// nothing.
struct IdScatterArgs {
  void *out;
  int32_t out_type; // 0 int32, 1 int64, 2 float32
  int32_t out_rank;
  int32_t rank;     // of the work shape
  int32_t per_item;
  int64_t out_shape[3], out_stride[3];
  int64_t idx_c[3], idx_g[3][3], idx_l[3][3];
  int64_t val_c, val_g[3], val_l[3];
};
extern "C" __global__ __launch_bounds__(1024) void hcamd_id_scatter(IdScatterArgs a) {
  const int64_t hw_g[3] = {blockIdx.x, blockIdx.y, blockIdx.z};
  const int64_t hw_l[3] = {threadIdx.x, threadIdx.y, threadIdx.z};
  int64_t g[3] = {0, 0, 0}, l[3] = {0, 0, 0};
  for (int d = 0; d < a.rank; ++d) {
    g[d] = hw_g[a.rank - 1 - d];
    l[d] = hw_l[a.rank - 1 - d];
  }
  if (!a.per_item && (l[0] | l[1] | l[2]) != 0)
    return;
  int64_t at = 0;
  for (int d = 0; d < a.out_rank; ++d) {
    int64_t i = a.idx_c[d];
    for (int k = 0; k < 3; ++k)
      i += a.idx_g[d][k] * g[k] + a.idx_l[d][k] * l[k];
    if (i < 0 || i >= a.out_shape[d])
      return;
    at += i * a.out_stride[d];
  }
  int64_t v = a.val_c;
  for (int k = 0; k < 3; ++k)
    v += a.val_g[k] * g[k] + a.val_l[k] * l[k];
  if (a.out_type == 0)
    static_cast<int32_t *>(a.out)[at] = (int32_t)v;
  else if (a.out_type == 1)
    static_cast<int64_t *>(a.out)[at] = v;
  else
    static_cast<float *>(a.out)[at] = (float)v;
}

extern "C" __global__ __launch_bounds__(256) void hcamd_fill32(uint32_t *dst,
                                                               uint32_t value,
                                                               size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count)
    dst[i] = value;
}
