// Row softmax, fp32: y = exp(x - max(x)) / sum(exp(x - max(x))) per row.
//
// Register-resident kernels: TPR threads share one row and each keeps VPT
// 16-byte words of it in VGPRs, so a row is read from HBM exactly once and
// written exactly once.  The two reductions (max, then sum) run on DPP inside
// each wave and cross waves through one LDS slot per wave.  TPR = 256 gives one
// workgroup per row (rows up to 1024*VPT columns); TPR = 64 gives one wave per
// row and four rows per workgroup for short rows, with no barrier at all.
//
// Rows that are not 16-byte aligned stay register-resident with 4-byte
// accesses (256 or 1024 lanes per row, up to 32,768 columns); longer rows take
// two sweeps with an online maximum and sum.  The three-sweep streaming kernel
// is kept as the plainest statement of the operation (variant 1).
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

// exp(x - m) as 2^(x*log2(e) - m*log2(e)): one fma and one v_exp_f32.  The fma
// rounds x*log2(e) - m*log2(e) once; with |x - m| <= 88 that is an absolute
// error of at most 2^-18 in the exponent, i.e. a relative error below 3e-6 in
// the result (1.3e-6 at |x - m| = 30); the rounding of m*log2(e) is common to
// the whole row and cancels in the normalisation.  Results below 2^-126 flush to
// zero.  NaN propagates; -inf (masked lanes) gives 0.
__device__ __forceinline__ float exp_scaled(float x, float m_log2e) {
  constexpr float kLog2e = 1.44269502162933349609375f;
  return __builtin_amdgcn_exp2f(__builtin_fmaf(x, kLog2e, -m_log2e));
}
// The fused form leaves the rounding error of m * log2(e) in every exponent of
// the row.  It cancels in the normalisation as long as 2^error stays in range,
// i.e. for |m| up to about 1e9; rows with a larger maximum take the plain
// exp2((x - m) * log2(e)), one more operation per element.
constexpr float kFusedMaxAbs = 1.0e6f;
__device__ __forceinline__ float exp_shifted(float x, float m) {
  constexpr float kLog2e = 1.44269502162933349609375f;
  return __builtin_amdgcn_exp2f((x - m) * kLog2e);
}

template <int TPR, int VPT, bool FULL, bool NT, bool FAST = true>
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
  // a row of -inf (or a masked-out row) has m = -inf: m*log2(e) - that would
  // make fma(-inf, c, +inf) NaN, which is also what the plain expression gives
  const float m_log2e = m * 1.44269502162933349609375f;
  if (!FAST || __builtin_fabsf(m) < kFusedMaxAbs) { // uniform over the row
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[j][i] = FAST ? exp_scaled(v[j][i], m_log2e) : exp_nonpos(v[j][i] - m);
        s += v[j][i];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[j][i] = exp_shifted(v[j][i], m);
        s += v[j][i];
      }
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
    softmax_regs<TPR, VPT, FULL, NT, true>(x, ldx, y, ldy, rows, cols);        \
  }
#define HCAMD_SOFTMAX_ACC(NAME, TPR, VPT, FULL, NT)                            \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *x, size_t ldx, float *y, size_t ldy, size_t rows,           \
      size_t cols) {                                                           \
    softmax_regs<TPR, VPT, FULL, NT, false>(x, ldx, y, ldy, rows, cols);       \
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
// compensated exponential (about 1.5 ulp) instead of the two-instruction one
HCAMD_SOFTMAX_ACC(hcamd_softmax_f32_g256_v8_full_nt_acc, 256, 8, true, true)
HCAMD_SOFTMAX_ACC(hcamd_softmax_f32_g256_v8_acc, 256, 8, false, false)

// Full rows of 8192 columns on 1024 lanes, two words per lane, one row per
// workgroup.  Same arithmetic as softmax_regs; what differs is how much of the
// matrix is in flight: two workgroups of this size fit a compute unit, so the
// chip holds 512 rows (16 MiB) at a time instead of 2048, and HBM sees a
// narrower window of addresses (measured 44.0 us against 44.9 for the
// persistent kernel and 46.4 for 256 lanes per row at 4096 x 8192).
template <int T, int VPT, bool NT>
__device__ __forceinline__ void softmax_wide(const float *x, size_t ldx, float *y,
                                             size_t ldy) {
  constexpr int kWaves = T / kWave;
  __shared__ float smax[kWaves];
  __shared__ float ssum[kWaves];
  const int t = threadIdx.x;
  const size_t row = blockIdx.x;
  const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * ldx);
  f32x4 *yr = reinterpret_cast<f32x4 *>(y + row * ldy);
  f32x4 v[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    v[j] = ldg<NT>(xr + j * T + t);
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    m = fmaxf(fmaxf(fmaxf(m, v[j][0]), fmaxf(v[j][1], v[j][2])), v[j][3]);
  m = group_reduce<MaxOp, kWaves>(m, smax);
  const float m_log2e = m * 1.44269502162933349609375f;
  float s = 0.0f;
  if (__builtin_fabsf(m) < kFusedMaxAbs) { // uniform over the row
#pragma unroll
    for (int j = 0; j < VPT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[j][i] = exp_scaled(v[j][i], m_log2e);
        s += v[j][i];
      }
  } else {
#pragma unroll
    for (int j = 0; j < VPT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[j][i] = exp_shifted(v[j][i], m);
        s += v[j][i];
      }
  }
  s = group_reduce<SumOp, kWaves>(s, ssum);
  const float inv = 1.0f / s;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    stg<NT>(yr + j * T + t, v[j] * inv);
}
extern "C" __global__ __launch_bounds__(1024) void hcamd_softmax_f32_g1024_v2_full_nt(
    const float *x, size_t ldx, float *y, size_t ldy, size_t rows, size_t cols) {
  softmax_wide<1024, 2, true>(x, ldx, y, ldy);
}

// The same rows with one exchange between the waves instead of two: every wave
// takes the maximum of its own 512 elements, exponentiates against it and sums;
// the waves exchange (maximum, sum) pairs once and each rescales what it holds
// by exp(own maximum - row maximum) / row sum.  A wave of -inf counts its
// maximum as 0 (every exponential is then 0).  Measured next to the kernel
// above at 4096 x 8192: 44.4 us against 43.9 us (512 and 256 lanes to a row: 46.1
// and 45.1 us) -- the kernel waits on HBM, not at its barriers -- so it is kept
// as a variant only.
namespace {
template <int T, int VPT, bool NT>
__device__ __forceinline__ void softmax_one_exchange(const float *x, size_t ldx, float *y,
                                                     size_t ldy) {
  constexpr int kWaves = T / kWave;
  constexpr float kLog2e = 1.44269502162933349609375f;
  __shared__ float wmax[kWaves];
  __shared__ float wsum[kWaves];
  const int t = threadIdx.x;
  const size_t row = blockIdx.x;
  const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * ldx);
  f32x4 *yr = reinterpret_cast<f32x4 *>(y + row * ldy);
  f32x4 v[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    v[j] = ldg<NT>(xr + j * T + t);
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    m = fmaxf(fmaxf(fmaxf(m, v[j][0]), fmaxf(v[j][1], v[j][2])), v[j][3]);
  m = wave_reduce<MaxOp>(m);
  const float mine = m == -INFINITY ? 0.0f : m;
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[j][i] = exp_shifted(v[j][i], mine);
      s += v[j][i];
    }
  s = wave_reduce<SumOp>(s);
  if ((t & (kWave - 1)) == 0) {
    wmax[t / kWave] = mine;
    wsum[t / kWave] = s;
  }
  __syncthreads();
  float top = wmax[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w)
    top = fmaxf(top, wmax[w]);
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w)
    total += wsum[w] * __builtin_amdgcn_exp2f((wmax[w] - top) * kLog2e);
  const float f = __builtin_amdgcn_exp2f((mine - top) * kLog2e) / total;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    stg<NT>(yr + j * T + t, v[j] * f);
}
} // namespace
extern "C" __global__ __launch_bounds__(1024) void hcamd_softmax_f32_g1024_v2_one_exchange_nt(
    const float *x, size_t ldx, float *y, size_t ldy, size_t rows, size_t cols) {
  softmax_one_exchange<1024, 2, true>(x, ldx, y, ldy);
}

// Persistent form of the full-row kernel: a workgroup walks rows blockIdx.x,
// blockIdx.x + gridDim.x, ... and requests the next row before it reduces the
// current one, so that loads stay in flight during the reductions, the
// exponentials and the stores, and reads and writes reach HBM interleaved
// rather than in alternating bursts.
template <int VPT, bool NT>
__device__ __forceinline__ void softmax_persistent(const float *x, size_t ldx,
                                                   float *y, size_t ldy,
                                                   size_t rows) {
  constexpr int kWaves = kThreads / kWave;
  __shared__ float smax[kWaves];
  __shared__ float ssum[kWaves];
  const int t = threadIdx.x;
  size_t row = blockIdx.x;
  if (row >= rows)
    return;
  f32x4 cur[VPT], nxt[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    nxt[j] = ldg<NT>(reinterpret_cast<const f32x4 *>(x + row * ldx) + j * kThreads + t);
  for (; row < rows; row += gridDim.x) {
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      cur[j] = nxt[j];
    const size_t next_row = row + gridDim.x;
    if (next_row < rows) {
#pragma unroll
      for (int j = 0; j < VPT; ++j)
        nxt[j] = ldg<NT>(reinterpret_cast<const f32x4 *>(x + next_row * ldx) + j * kThreads + t);
    }
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      m = fmaxf(fmaxf(fmaxf(m, cur[j][0]), fmaxf(cur[j][1], cur[j][2])), cur[j][3]);
    m = group_reduce<MaxOp, kWaves>(m, smax);
    const float m_log2e = m * 1.44269502162933349609375f;
    float s = 0.0f;
    if (__builtin_fabsf(m) < kFusedMaxAbs) { // uniform over the row
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          cur[j][i] = exp_scaled(cur[j][i], m_log2e);
          s += cur[j][i];
        }
    } else {
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          cur[j][i] = exp_shifted(cur[j][i], m);
          s += cur[j][i];
        }
    }
    s = group_reduce<SumOp, kWaves>(s, ssum);
    const float inv = 1.0f / s;
    f32x4 *yr = reinterpret_cast<f32x4 *>(y + row * ldy);
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      stg<NT>(yr + j * kThreads + t, cur[j] * inv);
  }
}

#define HCAMD_SOFTMAX_PERSIST(NAME, VPT, NT)                                   \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *x, size_t ldx, float *y, size_t ldy, size_t rows,           \
      size_t cols) {                                                           \
    softmax_persistent<VPT, NT>(x, ldx, y, ldy, rows);                         \
  }
HCAMD_SOFTMAX_PERSIST(hcamd_softmax_f32_p256_v8_nt, 8, true)
HCAMD_SOFTMAX_PERSIST(hcamd_softmax_f32_p256_v8, 8, false)
HCAMD_SOFTMAX_PERSIST(hcamd_softmax_f32_p256_v4_nt, 4, true)

// Rows that are not 16-byte aligned (a column count or leading dimension that
// is not a multiple of 4) but still fit in registers: one workgroup per row,
// lane t holds elements t, t + 256, ... (EPL of them), read and written with
// 4-byte accesses that a wave coalesces into 256-byte requests.  The row still
// crosses HBM once each way.  All loads are issued before the first is used;
// elements past the end are read from element 0 and replaced by -inf.
template <int EPL, int kThreads = 256>
__device__ __forceinline__ void softmax_scalar_regs(const float *x, size_t ldx, float *y,
                                                    size_t ldy, size_t cols) {
  __shared__ float smax[kThreads / kWave];
  __shared__ float ssum[kThreads / kWave];
  const size_t row = blockIdx.x;
  const float *xr = x + row * ldx;
  float *yr = y + row * ldy;
  const int t = threadIdx.x;
  float v[EPL];
  // 32-bit element offsets from the row start (rows are shorter than 2^31)
  const uint32_t n = (uint32_t)cols;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const uint32_t c = (uint32_t)j * kThreads + t;
    v[j] = __builtin_nontemporal_load(xr + (c < n ? c : 0u));
    if (j % 16 == 15) // keeps the address arithmetic of later loads from piling up
      __builtin_amdgcn_sched_barrier(0);
  }
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    v[j] = (size_t)j * kThreads + t < cols ? v[j] : -INFINITY;
    m = fmaxf(m, v[j]);
  }
  m = group_reduce<MaxOp, kThreads / kWave>(m, smax);
  float s = 0.0f;
  if (__builtin_fabsf(m) < kFusedMaxAbs) { // uniform over the row
    const float m_log2e = m * 1.44269502162933349609375f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      v[j] = exp_scaled(v[j], m_log2e);
      s += v[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      v[j] = exp_shifted(v[j], m);
      s += v[j];
    }
  }
  s = group_reduce<SumOp, kThreads / kWave>(s, ssum);
  const float inv = 1.0f / s;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const size_t c = (size_t)j * kThreads + t;
    if (c < cols)
      __builtin_nontemporal_store(v[j] * inv, yr + c);
  }
}
#define HCAMD_SOFTMAX_SCALAR(NAME, EPL)                                        \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *x, size_t ldx, float *y, size_t ldy, size_t rows,           \
      size_t cols) {                                                           \
    softmax_scalar_regs<EPL>(x, ldx, y, ldy, cols);                            \
  }
HCAMD_SOFTMAX_SCALAR(hcamd_softmax_f32_s256_e4, 4)
HCAMD_SOFTMAX_SCALAR(hcamd_softmax_f32_s256_e8, 8)
HCAMD_SOFTMAX_SCALAR(hcamd_softmax_f32_s256_e16, 16)
HCAMD_SOFTMAX_SCALAR(hcamd_softmax_f32_s256_e32, 32)
HCAMD_SOFTMAX_SCALAR(hcamd_softmax_f32_s256_e64, 64)
// the same with 1024 lanes per row: rows of up to 32,768 elements stay in
// registers (32 per lane, four waves per SIMD)
#define HCAMD_SOFTMAX_SCALAR_1024(NAME, EPL)                                   \
  extern "C" __global__ __launch_bounds__(1024) void NAME(                     \
      const float *x, size_t ldx, float *y, size_t ldy, size_t rows,           \
      size_t cols) {                                                           \
    softmax_scalar_regs<EPL, 1024>(x, ldx, y, ldy, cols);                      \
  }
HCAMD_SOFTMAX_SCALAR_1024(hcamd_softmax_f32_s1024_e32, 32)

// Rows too long for registers: two sweeps instead of three.  The first keeps a
// running maximum and a sum that is rescaled whenever the maximum grows (the
// online form: s <- s * exp(m_old - m_new) + exp(x - m_new)), per lane, and
// lanes are merged the same way at the end; the second sweep writes.  A
// workgroup of 1024 lanes per row, so that a row of 50,000 elements is ~49
// elements per lane and the second sweep finds the row in L2.
__device__ __forceinline__ void online_merge(float &m, float &s, float m2, float s2) {
  const float mm = fmaxf(m, m2);
  // exp(-inf - -inf) would be NaN: a side that has seen nothing contributes 0
  const float a = m == -INFINITY ? 0.0f : s * exp_nonpos(m - mm);
  const float b = m2 == -INFINITY ? 0.0f : s2 * exp_nonpos(m2 - mm);
  m = mm;
  s = a + b;
}
extern "C" __global__ __launch_bounds__(1024) void hcamd_softmax_f32_online(
    const float *x, size_t ldx, float *y, size_t ldy, size_t rows,
    size_t cols) {
  constexpr int kT = 1024;
  __shared__ float sm[kT / kWave], ss[kT / kWave];
  const size_t row = blockIdx.x;
  const float *xr = x + row * ldx;
  float *yr = y + row * ldy;
  const int t = threadIdx.x;
  float m = -INFINITY, s = 0.0f;
  bool nan = false;
  size_t c = t;
  // four independent loads in flight per lane
  for (; c + 3 * kT < cols; c += 4 * kT) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = xr[c + u * kT];
    const float vm = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
    nan = nan || v[0] != v[0] || v[1] != v[1] || v[2] != v[2] || v[3] != v[3];
    if (vm > m) {
      s = m == -INFINITY ? 0.0f : s * exp_nonpos(m - vm);
      m = vm;
    }
    // while the maximum is still -inf every element so far was -inf (or NaN,
    // which the flag remembers) and adds nothing; -inf - -inf would be NaN
    if (m != -INFINITY) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        s += exp_nonpos(v[u] - m);
    }
  }
  for (; c < cols; c += kT) {
    const float v = xr[c];
    nan = nan || v != v;
    if (v > m) {
      s = m == -INFINITY ? 0.0f : s * exp_nonpos(m - v);
      m = v;
    }
    if (m != -INFINITY)
      s += exp_nonpos(v - m);
  }
  // lanes -> wave (DPP shuffles through readlane-free butterfly) -> workgroup
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off, kWave), s2 = __shfl_xor(s, off, kWave);
    online_merge(m, s, m2, s2);
  }
  if (t % kWave == 0) {
    sm[t / kWave] = m;
    ss[t / kWave] = s;
  }
  const bool any_nan = __syncthreads_or(nan);
  m = sm[0];
  s = ss[0];
#pragma unroll
  for (int w = 1; w < kT / kWave; ++w)
    online_merge(m, s, sm[w], ss[w]);
  // a NaN anywhere makes the whole row NaN, as the whole-array expression does
  const float inv = any_nan ? __builtin_nanf("") : 1.0f / s;
  for (c = t; c < cols; c += kT)
    yr[c] = exp_nonpos(xr[c] - m) * inv;
}

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
