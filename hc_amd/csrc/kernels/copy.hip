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

extern "C" __global__ __launch_bounds__(256) void hcamd_fill32(uint32_t *dst,
                                                               uint32_t value,
                                                               size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count)
    dst[i] = value;
}
