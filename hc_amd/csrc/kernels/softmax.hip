// Row softmax, fp32: y = exp(x - max(x)) / sum(exp(x - max(x))) per row.
//
// Register-resident kernels: TPR threads share one row and each keeps VPT
// 16-byte words of it in VGPRs, so a row is read from HBM exactly once and
// written exactly once.  The two reductions (max, then sum) run on DPP inside
// each wave and cross waves through one LDS slot per wave.  TPR = 256 gives one
// workgroup per row (rows up to 1024*VPT columns); TPR = 64 gives one wave per
// row and four rows per workgroup for short rows, with no barrier at all.
//
// A streaming kernel covers rows that do not fit or are not 16-byte aligned.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kThreads = 256;

// exp(x) for x <= 0 (and NaN), about 1.5 ulp.  exp(x) = 2^(x*log2(e)); the
// product is formed in two pieces so that its rounding error (which would
// otherwise be multiplied by |x| up to ~45 ulp at x = -30) is added back to
// first order: 2^(hi+lo) = 2^hi * (1 + lo*ln2 + O(lo^2)), |lo| < 2^-17.
// Arguments below -200 (including -inf, which masked lanes carry) give 0.
__device__ __forceinline__ float exp_nonpos(float x) {
  constexpr float kLog2eHi = 1.44269502162933349609375f; // fl(log2 e)
  constexpr float kLog2eLo = 1.925963033500011e-08f;     // log2 e - hi
  constexpr float kLn2 = 0.693147182464599609375f;
  x = (x < -200.0f) ? -200.0f : x; // keeps NaN (compare is false)
  const float hi = x * kLog2eHi;
  float lo = __builtin_fmaf(x, kLog2eHi, -hi);
  lo = __builtin_fmaf(x, kLog2eLo, lo);
  const float e = __builtin_amdgcn_exp2f(hi);
  return __builtin_fmaf(e, lo * kLn2, e);
}

template <int TPR, int VPT, bool FULL, bool NT>
__device__ __forceinline__ void softmax_regs(const float *x, size_t ldx,
                                             float *y, size_t ldy, size_t rows,
                                             size_t cols) {
  constexpr int kRowsPerGroup = kThreads / TPR;
  constexpr int kWaves = TPR / kWave;
  __shared__ float smax[kRowsPerGroup * kWaves];
  __shared__ float ssum[kRowsPerGroup * kWaves];

  const int t = threadIdx.x % TPR;
  const int rg = threadIdx.x / TPR;
  const size_t row = (size_t)blockIdx.x * kRowsPerGroup + rg;
  const bool row_ok = row < rows; // uniform per wave
  const float *xr = x + row * ldx;
  float *yr = y + row * ldy;

  f32x4 v[VPT];
  const float ninf = -INFINITY;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t c = ((size_t)j * TPR + t) * 4;
    if (FULL) {
      v[j] = ldg<NT>(reinterpret_cast<const f32x4 *>(xr + c));
    } else {
      v[j] = f32x4{ninf, ninf, ninf, ninf};
      if (row_ok) {
        if (c + 4 <= cols) {
          v[j] = ldg<NT>(reinterpret_cast<const f32x4 *>(xr + c));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (c + i < cols)
              v[j][i] = xr[c + i];
        }
      }
    }
  }

  float m = ninf;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    m = fmaxf(fmaxf(fmaxf(m, v[j][0]), fmaxf(v[j][1], v[j][2])), v[j][3]);
  m = group_reduce<MaxOp, kWaves>(m, smax + rg * kWaves);

  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[j][i] = exp_nonpos(v[j][i] - m);
      s += v[j][i];
    }
  }
  s = group_reduce<SumOp, kWaves>(s, ssum + rg * kWaves);
  const float inv = 1.0f / s;

#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t c = ((size_t)j * TPR + t) * 4;
    const f32x4 o = v[j] * inv;
    if (FULL) {
      stg<NT>(reinterpret_cast<f32x4 *>(yr + c), o);
    } else if (row_ok) {
      if (c + 4 <= cols) {
        stg<NT>(reinterpret_cast<f32x4 *>(yr + c), o);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c + i < cols)
            yr[c + i] = o[i];
      }
    }
  }
}
} // namespace

#define HCAMD_SOFTMAX(NAME, TPR, VPT, FULL, NT)                                \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *x, size_t ldx, float *y, size_t ldy, size_t rows,           \
      size_t cols) {                                                           \
    softmax_regs<TPR, VPT, FULL, NT>(x, ldx, y, ldy, rows, cols);              \
  }

// masked (any cols up to the capacity, rows need 16-byte alignment only)
HCAMD_SOFTMAX(hcamd_softmax_f32_w64_v1, 64, 1, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_w64_v2, 64, 2, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_w64_v4, 64, 4, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v2, 256, 2, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v4, 256, 4, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v8, 256, 8, false, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v16, 256, 16, false, false)
// full rows (cols == 4*TPR*VPT): no predicates at all
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v8_full, 256, 8, true, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v8_full_nt, 256, 8, true, true)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v4_full, 256, 4, true, false)
HCAMD_SOFTMAX(hcamd_softmax_f32_g256_v2_full, 256, 2, true, false)

// Streaming kernel: one workgroup per row, three sweeps over the row (max,
// sum, write) with scalar accesses; the second and third sweeps hit L2.  Any
// alignment, any number of columns.
extern "C" __global__ __launch_bounds__(256) void hcamd_softmax_f32_stream(
    const float *x, size_t ldx, float *y, size_t ldy, size_t rows,
    size_t cols) {
  __shared__ float smax[kThreads / kWave];
  __shared__ float ssum[kThreads / kWave];
  const size_t row = blockIdx.x;
  const float *xr = x + row * ldx;
  float *yr = y + row * ldy;
  float m = -INFINITY;
  for (size_t c = threadIdx.x; c < cols; c += kThreads)
    m = fmaxf(m, xr[c]);
  // fmaxf drops NaN, but exp(NaN - m) below makes the sum, and so the whole
  // row, NaN, which is what the whole-array expression gives.
  m = group_reduce<MaxOp, kThreads / kWave>(m, smax);
  float s = 0.0f;
  for (size_t c = threadIdx.x; c < cols; c += kThreads)
    s += exp_nonpos(xr[c] - m);
  s = group_reduce<SumOp, kThreads / kWave>(s, ssum);
  const float inv = 1.0f / s;
  for (size_t c = threadIdx.x; c < cols; c += kThreads)
    yr[c] = exp_nonpos(xr[c] - m) * inv;
}
