// Row-wise symmetric int8 quantisation of fp16 rows:
//   scale[r] = max|x[r,:]| / 127            (fp32, IEEE division)
//   q[r,c]   = clamp(rint((float)x[r,c] / scale[r]), -127, 127)   (int8)
// with round-half-even and a correctly rounded fp32 quotient, so that the int8
// output is bit-identical to the whole-array NumPy expression.
//
// Layout: a thread owns chunks of 16 consecutive fp16 values (two 16-byte
// loads) and produces 16 int8 values (one 16-byte store).  TPR threads share a
// row; TPR = 256 is one workgroup per row, TPR = 64 is one wave per row and
// four rows per workgroup.  The row stays in VGPRs between the absmax
// reduction and the quantisation, so HBM sees one read and one write.
//
// absmax is computed on the fp16 bit patterns with the sign cleared: for
// non-negative fp16 the unsigned integer order equals the numeric order, and
// every NaN pattern (0x7c01..0x7fff) sorts above infinity, so a NaN anywhere in
// the row makes the scale NaN, as numpy.max does.  Two values share one
// 32-bit lane operation.
//
// Division: with EXACT_DIV the quotient is the compiler's IEEE fp32 division.
// Otherwise the row's correctly rounded reciprocal y = fl(1/scale) is formed
// once and each element takes q0 = x*y; r = fma(-q0, scale, x); q = fma(r, y,
// q0): the residual r is exact and the corrected q equals the correctly rounded
// quotient.  That equality was checked on the CPU for every one of the
// 1,007,713,278 (x, absmax) pairs of finite fp16 values with |x| <= absmax; the
// only difference is the sign of a zero quotient for x = -0, which the integer
// conversion drops.  The same sweep shows |rint(q)| <= 127 always: for finite
// rows the clamp never acts.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kThreads = 256;

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t absmax_bits(uint32_t m, uint32_t w) {
  const u16x2 a = __builtin_bit_cast(u16x2, m);
  const u16x2 b = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

__device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

template <bool EXACT_DIV>
__device__ __forceinline__ float quotient(float x, float scale, float rcp) {
  if constexpr (EXACT_DIV) {
    return x / scale;
  } else {
    const float q0 = x * rcp;
    const float r = __builtin_fmaf(-q0, scale, x);
    return __builtin_fmaf(r, rcp, q0);
  }
}

// Round-half-even to integer and int8 pack of four quotients, |q| <= 127.5.
// Adding 1.5 * 2^23 makes the fp32 adder do the rounding (the sum's ulp is 1,
// nearest-even), and leaves the two's-complement integer in the low mantissa
// bits: the low byte of each sum is the int8 result.  v_perm_b32 gathers the
// four low bytes.  No clamp: for a finite row |rint(x / scale)| <= 127 always
// (checked for every fp16 pair on the CPU).
__device__ __forceinline__ uint32_t pack4(float a, float b, float c, float d) {
  constexpr float kMagic = 12582912.0f; // 1.5 * 2^23
  const uint32_t ua = __builtin_bit_cast(uint32_t, a + kMagic);
  const uint32_t ub = __builtin_bit_cast(uint32_t, b + kMagic);
  const uint32_t uc = __builtin_bit_cast(uint32_t, c + kMagic);
  const uint32_t ud = __builtin_bit_cast(uint32_t, d + kMagic);
  // selector bytes: 0-3 pick from the second operand, 4-7 from the first, 0x0c is zero
  const uint32_t lo = __builtin_amdgcn_perm(ub, ua, 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm(ud, uc, 0x04000c0cu);
  return lo | hi;
}

// Rows whose absmax is inf or NaN: a NaN quotient (inf/inf, x/NaN) maps to 0,
// which is what a NaN -> int8 conversion yields on the host.
__device__ __forceinline__ int8_t quant_special(float x, float scale) {
  const float qf = x / scale;
  if (qf != qf)
    return 0;
  return (int8_t)(int)__builtin_amdgcn_fmed3f(__builtin_rintf(qf), -127.f,
                                              127.f);
}

template <int TPR, int VPT, bool EXACT_DIV, bool NT>
__device__ __forceinline__ void quantize_regs(const _Float16 *x, size_t ldx,
                                              int8_t *q, size_t ldq,
                                              float *scale_out, size_t rows,
                                              size_t cols) {
  constexpr int kRowsPerGroup = kThreads / TPR;
  constexpr int kWaves = TPR / kWave;
  __shared__ uint32_t smax[kRowsPerGroup * kWaves];

  const int t = threadIdx.x % TPR;
  const int rg = threadIdx.x / TPR;
  const size_t row = (size_t)blockIdx.x * kRowsPerGroup + rg;
  const bool row_ok = row < rows; // uniform per wave
  const _Float16 *xr = x + row * ldx;
  int8_t *qr = q + row * ldq;

  // chunk j of this thread starts at column ((j*TPR)+t)*16
  u32x4 v[VPT][2];
  uint32_t m = 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t c = ((size_t)j * TPR + t) * 16;
    v[j][0] = u32x4{0, 0, 0, 0};
    v[j][1] = u32x4{0, 0, 0, 0};
    if (row_ok) {
      if (c + 16 <= cols) {
        v[j][0] = ldg<NT>(reinterpret_cast<const u32x4 *>(xr + c));
        v[j][1] = ldg<NT>(reinterpret_cast<const u32x4 *>(xr + c + 8));
      } else if (c < cols) {
        // ragged last chunk: element loads, zero fill (zero never raises the
        // absmax and is never stored)
        unsigned short e[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
          e[i] = (c + i < cols)
                     ? reinterpret_cast<const unsigned short *>(xr)[c + i]
                     : (unsigned short)0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[j][0][i] = (uint32_t)e[2 * i] | ((uint32_t)e[2 * i + 1] << 16);
          v[j][1][i] =
              (uint32_t)e[8 + 2 * i] | ((uint32_t)e[8 + 2 * i + 1] << 16);
        }
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        m = absmax_bits(m, v[j][h][i]);
  }
  m = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
  m = group_reduce<UMaxOp, kWaves>(m, smax + rg * kWaves);

  const float amax = half_bits_to_float(m);
  const float scale = amax / 127.0f;
  if (row_ok && t == 0)
    scale_out[row] = scale;
  const bool special = !(amax < INFINITY); // inf or NaN, uniform per row
  // An all-zero row divides by 1 instead of 0: every quotient is 0.
  const float div = (amax == 0.0f) ? 1.0f : scale;
  const float rcp = 1.0f / div;

#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t c = ((size_t)j * TPR + t) * 16;
    if (!row_ok || c >= cols)
      continue;
    if (special) {
      for (int i = 0; i < 16 && c + i < cols; ++i) {
        const uint32_t w = v[j][i / 8][(i % 8) / 2];
        const uint32_t bits = (i & 1) ? (w >> 16) : (w & 0xffffu);
        qr[c + i] = quant_special(half_bits_to_float(bits), scale);
      }
      continue;
    }
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // output word k holds elements 4k..4k+3 = input words 2k, 2k+1
      const uint32_t w0 = v[j][k / 2][(2 * k) % 4];
      const uint32_t w1 = v[j][k / 2][(2 * k) % 4 + 1];
      const float f0 = half_bits_to_float(w0 & 0xffffu);
      const float f1 = half_bits_to_float(w0 >> 16);
      const float f2 = half_bits_to_float(w1 & 0xffffu);
      const float f3 = half_bits_to_float(w1 >> 16);
      o[k] = pack4(quotient<EXACT_DIV>(f0, div, rcp),
                   quotient<EXACT_DIV>(f1, div, rcp),
                   quotient<EXACT_DIV>(f2, div, rcp),
                   quotient<EXACT_DIV>(f3, div, rcp));
    }
    if (c + 16 <= cols) {
      stg<NT>(reinterpret_cast<u32x4 *>(qr + c), o);
    } else {
      for (int i = 0; i < 16 && c + i < cols; ++i)
        qr[c + i] = (int8_t)((o[i / 4] >> (8 * (i % 4))) & 0xff);
    }
  }
}
// Word layout: a row is walked in 16-byte words of 8 fp16 values; lane t of the
// TPR lanes that share a row takes words t, t + TPR, ..., so every wave-level
// load covers 1 KiB of consecutive bytes and every wave-level store (8 int8
// values per lane) 512 consecutive bytes, exactly the access pattern of a plain
// copy.  (quantize_regs gives a lane 16 consecutive values so that it can
// store 16 bytes; its loads then touch every cache line twice, which costs
// about 6 % at 16384 x 4096.)  T / TPR rows share a workgroup.  Needs
// cols % 8 == 0, rows of x on 16-byte and rows of q on 8-byte boundaries, and
// cols <= 8 * TPR * VPT; FULL: cols == 8 * TPR * VPT and rows % (T / TPR) == 0,
// no predicates at all.
template <int TPR, int T, int VPT, bool FULL, bool NT>
__device__ __forceinline__ void quantize_words(const _Float16 *x, size_t ldx, int8_t *q,
                                               size_t ldq, float *scale_out, size_t rows,
                                               size_t cols) {
  constexpr int kRowsPerGroup = T / TPR;
  constexpr int kWaves = TPR / kWave;
  __shared__ uint32_t smax[kRowsPerGroup * kWaves];
  const int t = threadIdx.x % TPR;
  const int rg = threadIdx.x / TPR;
  const size_t row = (size_t)blockIdx.x * kRowsPerGroup + rg;
  const bool row_ok = FULL || row < rows; // uniform per wave
  const uint32_t words = (uint32_t)(cols / 8);
  const u32x4 *xr = reinterpret_cast<const u32x4 *>(x + (row_ok ? row : 0) * ldx);
  u32x4 v[VPT];
  uint32_t m = 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const uint32_t w = (uint32_t)j * TPR + t;
    if (FULL || (row_ok && w < words))
      v[j] = ldg<NT>(xr + w);
    else
      v[j] = u32x4{0, 0, 0, 0};
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      m = absmax_bits(m, v[j][i]);
  m = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
  m = group_reduce<UMaxOp, kWaves>(m, smax + rg * kWaves);

  const float amax = half_bits_to_float(m);
  const float scale = amax / 127.0f;
  if (row_ok && t == 0)
    scale_out[row] = scale;
  if (!row_ok)
    return;
  const bool special = !(amax < INFINITY); // inf or NaN, uniform per row
  const float div = (amax == 0.0f) ? 1.0f : scale;
  const float rcp = 1.0f / div;
  int8_t *qr = q + row * ldq;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const uint32_t w = (uint32_t)j * TPR + t;
    if (!FULL && w >= words)
      continue;
    if (special) {
      for (int i = 0; i < 8; ++i) {
        const uint32_t pair = v[j][i / 2];
        const uint32_t bits = (i & 1) ? (pair >> 16) : (pair & 0xffffu);
        qr[(size_t)w * 8 + i] = quant_special(half_bits_to_float(bits), scale);
      }
      continue;
    }
    u32x2 o;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t w0 = v[j][2 * k], w1 = v[j][2 * k + 1];
      o[k] = pack4(quotient<false>(half_bits_to_float(w0 & 0xffffu), div, rcp),
                   quotient<false>(half_bits_to_float(w0 >> 16), div, rcp),
                   quotient<false>(half_bits_to_float(w1 & 0xffffu), div, rcp),
                   quotient<false>(half_bits_to_float(w1 >> 16), div, rcp));
    }
    stg<NT>(reinterpret_cast<u32x2 *>(qr) + w, o);
  }
}

// Persistent form for rows of exactly 256 * 16 columns, 16-byte aligned: a
// workgroup strides over the rows, and the loads of its next row are issued
// before the absmax reduction of the current one, so requests stay in flight
// across the reduction and its barrier.  The two LDS slot sets alternate from
// row to row, which makes the one barrier inside the reduction sufficient.
template <bool NT>
__device__ __forceinline__ void quantize_persistent(const _Float16 *x, size_t ldx,
                                                    int8_t *q, size_t ldq,
                                                    float *scale_out, size_t rows) {
  constexpr int kWaves = kThreads / kWave;
  __shared__ uint32_t smax[2][kWaves];
  const int t = threadIdx.x;
  size_t row = blockIdx.x;
  u32x4 cur[2], nxt[2];
  if (row < rows) {
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + row * ldx + (size_t)t * 16);
    cur[0] = ldg<NT>(p);
    cur[1] = ldg<NT>(p + 1);
  }
  for (int it = 0; row < rows; row += gridDim.x, ++it) {
    const size_t next = row + gridDim.x;
    if (next < rows) {
      const u32x4 *p = reinterpret_cast<const u32x4 *>(x + next * ldx + (size_t)t * 16);
      nxt[0] = ldg<NT>(p);
      nxt[1] = ldg<NT>(p + 1);
    }
    uint32_t m = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        m = absmax_bits(m, cur[h][i]);
    m = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    m = group_reduce<UMaxOp, kWaves>(m, smax[it & 1]);
    const float amax = half_bits_to_float(m);
    const float scale = amax / 127.0f;
    if (t == 0)
      scale_out[row] = scale;
    int8_t *qr = q + row * ldq + (size_t)t * 16;
    if (!(amax < INFINITY)) { // inf or NaN in the row
      for (int i = 0; i < 16; ++i) {
        const uint32_t w = cur[i / 8][(i % 8) / 2];
        const uint32_t bits = (i & 1) ? (w >> 16) : (w & 0xffffu);
        qr[i] = quant_special(half_bits_to_float(bits), scale);
      }
    } else {
      const float div = (amax == 0.0f) ? 1.0f : scale;
      const float rcp = 1.0f / div;
      u32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t w0 = cur[k / 2][(2 * k) % 4];
        const uint32_t w1 = cur[k / 2][(2 * k) % 4 + 1];
        o[k] = pack4(quotient<false>(half_bits_to_float(w0 & 0xffffu), div, rcp),
                     quotient<false>(half_bits_to_float(w0 >> 16), div, rcp),
                     quotient<false>(half_bits_to_float(w1 & 0xffffu), div, rcp),
                     quotient<false>(half_bits_to_float(w1 >> 16), div, rcp));
      }
      stg<NT>(reinterpret_cast<u32x4 *>(qr), o);
    }
    cur[0] = nxt[0];
    cur[1] = nxt[1];
  }
}
// Rows that are not 16-byte aligned but still fit in registers: one workgroup
// per row, lane t holds groups t, t + 256, ... of V consecutive elements (V = 4,
// 2 or 1 as the leading dimensions allow: 8-, 4- or 2-byte loads and 4-, 2- or
// 1-byte stores).  The row crosses HBM once each way; every load is
// unconditional (a group past the end is read from group 0 and ignored) and
// issued before the first use.  The cols % V elements after the last whole group
// are handled one per lane.
template <int V, int EPL>
__device__ __forceinline__ void quantize_small(const _Float16 *x, size_t ldx, int8_t *q,
                                               size_t ldq, float *scale_out, size_t cols) {
  typedef unsigned short hx __attribute__((ext_vector_type(V)));
  typedef signed char qx __attribute__((ext_vector_type(V)));
  __shared__ uint32_t smax[kThreads / kWave];
  const size_t row = blockIdx.x;
  const unsigned short *xr = reinterpret_cast<const unsigned short *>(x) + row * ldx;
  int8_t *qr = q + row * ldq;
  const int t = threadIdx.x;
  const uint32_t n = (uint32_t)cols, whole = n / V, tail = n % V;

  // groups per lane that exist at all (uniform): the rest are skipped whole
  const uint32_t used = (whole + kThreads - 1) / kThreads;
  unsigned short v[EPL][V];
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    if ((uint32_t)j >= used) {
#pragma unroll
      for (int e = 0; e < V; ++e)
        v[j][e] = 0;
      continue;
    }
    const uint32_t g = (uint32_t)j * kThreads + t;
    const uint32_t gs = (g < whole) ? g : 0u;
    if constexpr (V == 1) {
      v[j][0] = __builtin_nontemporal_load(xr + (whole ? gs : 0u));
    } else {
      // whole == 0 only if cols < V: then nothing of this load is used, and
      // element 0 .. V-1 of the row may not all exist, so read one element
      hx w;
      if (whole) {
        w = __builtin_nontemporal_load(reinterpret_cast<const hx *>(xr) + gs);
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e)
          w[e] = 0;
      }
#pragma unroll
      for (int e = 0; e < V; ++e)
        v[j][e] = w[e];
    }
  }
  unsigned short tv = 0;
  if (V > 1 && (uint32_t)t < tail)
    tv = xr[whole * V + t];

  uint32_t m = tv & 0x7fffu;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const bool in = (uint32_t)j * kThreads + t < whole;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      v[j][e] = in ? v[j][e] : (unsigned short)0;
      const uint32_t b = v[j][e] & 0x7fffu;
      m = b > m ? b : m;
    }
  }
  m = group_reduce<UMaxOp, kThreads / kWave>(m, smax);
  const float amax = half_bits_to_float(m);
  const float scale = amax / 127.0f;
  if (t == 0)
    scale_out[row] = scale;
  const bool special = !(amax < INFINITY); // inf or NaN, uniform per row
  const float div = (amax == 0.0f) ? 1.0f : scale;
  const float rcp = 1.0f / div;
  auto one = [&](unsigned short bits) -> int8_t {
    const float f = half_bits_to_float(bits);
    if (special)
      return quant_special(f, scale);
    return (int8_t)(pack4(quotient<false>(f, div, rcp), 0.0f, 0.0f, 0.0f) & 0xff);
  };
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const uint32_t g = (uint32_t)j * kThreads + t;
    if (g >= whole)
      continue;
    if constexpr (V == 4) {
      if (!special) {
        const uint32_t o = pack4(quotient<false>(half_bits_to_float(v[j][0]), div, rcp),
                                 quotient<false>(half_bits_to_float(v[j][1]), div, rcp),
                                 quotient<false>(half_bits_to_float(v[j][2]), div, rcp),
                                 quotient<false>(half_bits_to_float(v[j][3]), div, rcp));
        __builtin_nontemporal_store(o, reinterpret_cast<uint32_t *>(qr) + g);
        continue;
      }
    }
    qx o;
#pragma unroll
    for (int e = 0; e < V; ++e)
      o[e] = one(v[j][e]);
    if constexpr (V == 1)
      qr[g] = o[0];
    else
      *(reinterpret_cast<qx *>(qr) + g) = o;
  }
  if (V > 1 && (uint32_t)t < tail)
    qr[whole * V + t] = one(tv);
}
} // namespace

extern "C" __global__ __launch_bounds__(256) void hcamd_quant_f16_i8_p256_v1_nt(
    const _Float16 *x, size_t ldx, int8_t *q, size_t ldq, float *scale,
    size_t rows, size_t cols) {
  quantize_persistent<true>(x, ldx, q, ldq, scale, rows);
}

#define HCAMD_QUANT(NAME, TPR, VPT, EXACT, NT)                                 \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const _Float16 *x, size_t ldx, int8_t *q, size_t ldq, float *scale,      \
      size_t rows, size_t cols) {                                              \
    quantize_regs<TPR, VPT, EXACT, NT>(x, ldx, q, ldq, scale, rows, cols);     \
  }

HCAMD_QUANT(hcamd_quant_f16_i8_w64_v1, 64, 1, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_w64_v2, 64, 2, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_w64_v4, 64, 4, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_w64_v4_nt, 64, 4, false, true)
HCAMD_QUANT(hcamd_quant_f16_i8_w64_v4_div, 64, 4, true, false)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v1, 256, 1, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v1_nt, 256, 1, false, true)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v1_div, 256, 1, true, false)
HCAMD_QUANT(hcamd_quant_f16_i8_g128_v2_nt, 128, 2, false, true)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v2, 256, 2, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v4, 256, 4, false, false)
HCAMD_QUANT(hcamd_quant_f16_i8_g256_v8, 256, 8, false, false)

// two rows per workgroup of 512 lanes, 256 lanes and two words per lane per row
#define HCAMD_QUANT_WORDS(NAME, FULL)                                          \
  extern "C" __global__ __launch_bounds__(512) void NAME(                      \
      const _Float16 *x, size_t ldx, int8_t *q, size_t ldq, float *scale,      \
      size_t rows, size_t cols) {                                              \
    quantize_words<256, 512, 2, FULL, true>(x, ldx, q, ldq, scale, rows, cols);\
  }
HCAMD_QUANT_WORDS(hcamd_quant_f16_i8_c256x2_w2_nt, false)
HCAMD_QUANT_WORDS(hcamd_quant_f16_i8_c256x2_w2_full_nt, true)

#define HCAMD_QUANT_SMALL(NAME, V, EPL)                                        \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const _Float16 *x, size_t ldx, int8_t *q, size_t ldq, float *scale,      \
      size_t rows, size_t cols) {                                              \
    quantize_small<V, EPL>(x, ldx, q, ldq, scale, cols);                       \
  }
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s4_e4, 4, 4)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s4_e8, 4, 8)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s4_e16, 4, 16)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s4_e32, 4, 32)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s2_e8, 2, 8)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s2_e16, 2, 16)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s2_e32, 2, 32)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s2_e64, 2, 64)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s1_e16, 1, 16)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s1_e32, 1, 32)
HCAMD_QUANT_SMALL(hcamd_quant_f16_i8_s1_e64, 1, 64)

// Streaming kernel: one workgroup per row, two sweeps (absmax, quantise) with
// element accesses and the compiler's IEEE division.  Any alignment, any
// number of columns.
extern "C" __global__ __launch_bounds__(256) void hcamd_quant_f16_i8_stream(
    const _Float16 *x, size_t ldx, int8_t *q, size_t ldq, float *scale_out,
    size_t rows, size_t cols) {
  __shared__ uint32_t smax[kThreads / kWave];
  const size_t row = blockIdx.x;
  const unsigned short *xr =
      reinterpret_cast<const unsigned short *>(x) + row * ldx;
  int8_t *qr = q + row * ldq;
  uint32_t m = 0;
  for (size_t c = threadIdx.x; c < cols; c += kThreads) {
    const uint32_t b = xr[c] & 0x7fffu;
    m = b > m ? b : m;
  }
  m = group_reduce<UMaxOp, kThreads / kWave>(m, smax);
  const float amax = half_bits_to_float(m);
  const float scale = amax / 127.0f;
  if (threadIdx.x == 0)
    scale_out[row] = scale;
  const float div = (amax == 0.0f) ? 1.0f : scale;
  for (size_t c = threadIdx.x; c < cols; c += kThreads)
    qr[c] = quant_special(half_bits_to_float(xr[c]), div);
}
