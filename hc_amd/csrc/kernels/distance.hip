// Pairwise Euclidean distances: out[m, n] = sqrt(sum_d (a[m, d] - b[n, d])^2),
// fp32, a[M, D] and b[N, D] row-major.  The differences are formed explicitly
// (no |a|^2 + |b|^2 - 2ab expansion, which cancels for nearby points), so the
// kernel is bound by the vector ALUs: one subtract and one fused multiply-add
// per (m, n, d).
//
// A workgroup of 256 owns a 64 x 64 block of out; lane (ty, tx) of the 16 x 16
// arrangement owns the 4 x 4 sub-block at rows 4*ty, columns 4*tx.  D is walked in
// steps of 32: the 64 x 32 panels of a and b are stored to LDS transposed
// (d-major, rows of 64 + 4 floats), so that the four row values a lane needs
// for one d are a single 16-byte LDS read; the sixteen lanes that share ty
// read the same address (a broadcast), the others fall into different banks.
// Panel elements outside the matrices are loaded as zero for both a and b, so
// they add nothing to any sum; out-of-range outputs are not stored.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kTile = 64;  // outputs per workgroup and dimension
constexpr int kStep = 32;  // d values per panel
constexpr int kPitch = kTile + 4;
} // namespace

extern "C" __global__ __launch_bounds__(256) void hcamd_pairwise_dist_f32(
    const float *a, size_t lda, const float *b, size_t ldb, float *out,
    size_t ldo, size_t M, size_t N, size_t D) {
  __shared__ __attribute__((aligned(16))) float as[kStep][kPitch];
  __shared__ __attribute__((aligned(16))) float bs[kStep][kPitch];
  const int t = threadIdx.x;
  const int tx = t % 16, ty = t / 16;
  const size_t m0 = (size_t)blockIdx.y * kTile, n0 = (size_t)blockIdx.x * kTile;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[i][j] = 0.0f;

  // panel loads: lane t reads d = t % 32 of rows t / 32 + 8 * k, so that a wave
  // reads two runs of 32 consecutive floats
  const int ld_d = t % kStep, ld_r = t / kStep;
  for (size_t d0 = 0; d0 < D; d0 += kStep) {
    const size_t d = d0 + ld_d;
    // all sixteen loads are issued before any is used: an element outside the
    // matrices is read from element 0 instead and replaced by zero afterwards
    // (a load inside a per-lane branch would be waited for on the spot)
    float va[kTile / 8], vb[kTile / 8];
#pragma unroll
    for (int k = 0; k < kTile / 8; ++k) {
      const int r = ld_r + 8 * k;
      const size_t ma = m0 + r, nb = n0 + r;
      va[k] = a[(d < D && ma < M) ? ma * lda + d : 0];
      vb[k] = b[(d < D && nb < N) ? nb * ldb + d : 0];
    }
#pragma unroll
    for (int k = 0; k < kTile / 8; ++k) {
      const int r = ld_r + 8 * k;
      as[ld_d][r] = (d < D && m0 + r < M) ? va[k] : 0.0f;
      bs[ld_d][r] = (d < D && n0 + r < N) ? vb[k] : 0.0f;
    }
    __syncthreads();
#pragma unroll 8
    for (int dd = 0; dd < kStep; ++dd) {
      const f32x4 av = *reinterpret_cast<const f32x4 *>(&as[dd][4 * ty]);
      const f32x4 bv = *reinterpret_cast<const f32x4 *>(&bs[dd][4 * tx]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float diff = av[i] - bv[j];
          acc[i][j] = __builtin_fmaf(diff, diff, acc[i][j]);
        }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const size_t m = m0 + 4 * ty + i;
    if (m >= M)
      continue;
    float *row = out + m * ldo + n0 + 4 * tx;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n0 + 4 * tx + j < N)
        row[j] = __builtin_sqrtf(acc[i][j]);
  }
}
