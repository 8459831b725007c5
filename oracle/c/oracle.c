/*
 * oracle.c - CPU restatement, in plain C, of the results the hc_amd kernels
 * must reproduce.  TEST INFRASTRUCTURE ONLY: nothing in the product may link,
 * load or call this file; tests, the smoke check and the benchmark's CPU
 * baseline are its only users.
 *
 * The reference expresses these computations tile by tile in its NumPy
 * simulator (python/hckernel/kernel_api.py:297-342 load/store,
 * python/hckernel/kernel_sim.py:144-163 group loop) and checks each against a
 * whole-array expression (pattern: python/hckernel/tests/test_examples.py:
 * 330-335 for softmax, :121,165 for dot).  Each function below restates one
 * such whole-array expression with IEEE-754 arithmetic written out by hand, so
 * that it does not share code with NumPy, which the tests use as the second,
 * independent statement of the same expression.
 *
 * Built without -ffast-math and with -ffp-contract=off: every operation
 * rounds exactly once, where written.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* ---- scalar conversions -------------------------------------------------- */

static inline uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* IEEE binary16 -> binary32, exact (every half is representable). */
float oracle_half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1f) /* inf / NaN: keep the payload in the top mantissa bits */
    return u2f(sign | 0x7f800000u | (man << 13));
  if (exp == 0) {
    if (man == 0)
      return u2f(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-08f; /* exact product */
    return u2f(f2u(v) | sign);
  }
  return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

/* IEEE binary32 -> binary16, round to nearest even; overflow to infinity,
 * gradual underflow to subnormals and zero (what NumPy's astype(float16) and
 * the GPU's v_cvt_f16_f32 do). */
uint16_t oracle_float_to_half(float f) {
  const uint32_t u = f2u(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) { /* inf or NaN */
    if (a == 0x7f800000u)
      return sign | 0x7c00u;
    return sign | 0x7e00u | (uint16_t)((a >> 13) & 0x3ffu); /* quiet NaN */
  }
  if (a >= 0x477ff000u) /* >= 65520: rounds to infinity */
    return sign | 0x7c00u;
  if (a < 0x33000001u) /* <= 2^-25: rounds to zero (tie goes to even = 0) */
    return sign;
  int32_t e = (int32_t)(a >> 23) - 127; /* unbiased */
  uint32_t man = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_exp;
  if (e < -14) { /* subnormal half: value = man * 2^(e-23), unit 2^-24 */
    shift = (uint32_t)(13 + (-14 - e));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(e + 15);
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u)))
    q++;
  /* q carries the implicit bit for normals: adding it to the exponent field
   * minus one makes mantissa overflow carry into the exponent correctly. */
  uint32_t r;
  if (half_exp == 0)
    r = q; /* may become 0x400 = smallest normal */
  else
    r = ((half_exp - 1u) << 10) + q;
  return sign | (uint16_t)r;
}

float oracle_bf16_to_float(uint16_t b) { return u2f((uint32_t)b << 16); }

/* binary32 -> bfloat16, round to nearest even; NaN stays NaN (quiet). */
uint16_t oracle_float_to_bf16(float f) {
  const uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (uint16_t)((u >> 16) | 0x0040u);
  const uint32_t bias = 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)((u + bias) >> 16);
}

/* ---- W1: c = a + b, fp32 -------------------------------------------------- */
void oracle_add_f32(const float *a, const float *b, float *c, size_t n) {
  for (size_t i = 0; i < n; ++i)
    c[i] = a[i] + b[i];
}

/* ---- W2: d = half(float(a) * float(b) + float(c)) ------------------------- */
void oracle_fma_f16(const uint16_t *a, size_t lda, const uint16_t *b,
                    size_t ldb, const uint16_t *c, size_t ldc, uint16_t *d,
                    size_t ldd, size_t rows, size_t cols) {
  for (size_t r = 0; r < rows; ++r)
    for (size_t k = 0; k < cols; ++k) {
      const float fa = oracle_half_to_float(a[r * lda + k]);
      const float fb = oracle_half_to_float(b[r * ldb + k]);
      const float fc = oracle_half_to_float(c[r * ldc + k]);
      const float p = fa * fb; /* exact: 11-bit x 11-bit significands */
      d[r * ldd + k] = oracle_float_to_half(p + fc);
    }
}

/* ---- W0: masked window copy ---------------------------------------------- */
void oracle_copy2d(size_t elem, const void *src, size_t src_rows,
                   size_t src_cols, ptrdiff_t ss0, ptrdiff_t ss1, void *dst,
                   size_t dst_rows, size_t dst_cols, ptrdiff_t ds0,
                   ptrdiff_t ds1) {
  const size_t rows = src_rows < dst_rows ? src_rows : dst_rows;
  const size_t cols = src_cols < dst_cols ? src_cols : dst_cols;
  for (size_t r = 0; r < rows; ++r)
    for (size_t k = 0; k < cols; ++k)
      memcpy((char *)dst + ((ptrdiff_t)r * ds0 + (ptrdiff_t)k * ds1) *
                               (ptrdiff_t)elem,
             (const char *)src + ((ptrdiff_t)r * ss0 + (ptrdiff_t)k * ss1) *
                                     (ptrdiff_t)elem,
             elem);
}

/* ---- W3: row softmax ------------------------------------------------------
 * np_softmax of test_examples.py:330-335.  Two statements: the fp32 one uses
 * the same operation order a straightforward fp32 program would (max, expf,
 * sequential fp32 sum, division); the fp64 one computes the mathematically
 * exact value to ~1e-16 and rounds once, and is the tighter yardstick. */
void oracle_softmax_f32(const float *x, size_t ldx, float *y, size_t ldy,
                        size_t rows, size_t cols) {
  for (size_t r = 0; r < rows; ++r) {
    const float *xr = x + r * ldx;
    float *yr = y + r * ldy;
    float m = -INFINITY;
    int has_nan = 0;
    for (size_t k = 0; k < cols; ++k) {
      if (xr[k] != xr[k])
        has_nan = 1;
      if (xr[k] > m)
        m = xr[k];
    }
    if (has_nan)
      m = NAN;
    float s = 0.0f;
    for (size_t k = 0; k < cols; ++k) {
      yr[k] = expf(xr[k] - m);
      s += yr[k];
    }
    for (size_t k = 0; k < cols; ++k)
      yr[k] = yr[k] / s;
  }
}

void oracle_softmax_f64(const float *x, size_t ldx, float *y, size_t ldy,
                        size_t rows, size_t cols) {
  for (size_t r = 0; r < rows; ++r) {
    const float *xr = x + r * ldx;
    float *yr = y + r * ldy;
    double m = -INFINITY;
    int has_nan = 0;
    for (size_t k = 0; k < cols; ++k) {
      if (xr[k] != xr[k])
        has_nan = 1;
      if ((double)xr[k] > m)
        m = (double)xr[k];
    }
    if (has_nan)
      m = NAN;
    double s = 0.0;
    for (size_t k = 0; k < cols; ++k)
      s += exp((double)xr[k] - m);
    for (size_t k = 0; k < cols; ++k)
      yr[k] = (float)(exp((double)xr[k] - m) / s);
  }
}

/* ---- W4: row absmax int8 quantisation --------------------------------------
 * xf = float(x); amax = max|xf| per row (NaN propagates, as numpy.max does);
 * scale = amax / 127.0f; q = clip(rint(xf / scale), -127, 127) as int8.
 * rintf rounds half to even in the default rounding mode.  A zero row gives
 * scale 0 and q 0 (the plain expression would give NaN: 0/0).  A NaN quotient
 * (inf/inf, x/NaN) gives q 0. */
static int8_t quant1(float xf, float div) {
  const float qf = xf / div;
  if (qf != qf)
    return 0;
  float r = rintf(qf);
  if (r > 127.0f)
    r = 127.0f;
  if (r < -127.0f)
    r = -127.0f;
  return (int8_t)(int)r;
}

void oracle_quantize_f16_i8(const uint16_t *x, size_t ldx, int8_t *q,
                            size_t ldq, float *scale, size_t rows,
                            size_t cols) {
  for (size_t r = 0; r < rows; ++r) {
    const uint16_t *xr = x + r * ldx;
    float amax = 0.0f;
    int has_nan = 0;
    for (size_t k = 0; k < cols; ++k) {
      const float a = fabsf(oracle_half_to_float(xr[k]));
      if (a != a)
        has_nan = 1;
      if (a > amax)
        amax = a;
    }
    if (has_nan)
      amax = NAN;
    const float s = amax / 127.0f;
    scale[r] = s;
    const float div = (amax == 0.0f) ? 1.0f : s;
    for (size_t k = 0; k < cols; ++k)
      q[r * ldq + k] = quant1(oracle_half_to_float(xr[k]), div);
  }
}

/* Exhaustive check behind the kernel's division shortcut.  For every finite
 * positive fp16 absmax with bit pattern in [amax_lo, amax_hi) and every finite
 * fp16 x (both signs) with |x| <= absmax:
 *     scale = absmax / 127; y = fl(1 / scale);
 *     q0 = x * y; r = fma(-q0, scale, x); q = fma(r, y, q0)
 * is compared with the IEEE quotient x / scale.  Returns the number of pairs
 * whose quotients differ in value; *sign_of_zero counts pairs that differ only
 * in the sign of a zero quotient (x = -0), *int_mismatch pairs whose rounded
 * integers differ, *checked the pairs visited, and *max_abs_q the largest
 * |rint(x / scale)| seen (127 means the clamp never acts). */
uint64_t oracle_quotient_shortcut_mismatches(uint32_t amax_lo, uint32_t amax_hi,
                                             uint64_t *sign_of_zero,
                                             uint64_t *int_mismatch,
                                             uint64_t *checked,
                                             float *max_abs_q) {
  uint64_t bad = 0, bad_zero = 0, bad_int = 0, n = 0;
  float maxq = 0.0f;
  if (amax_lo < 1)
    amax_lo = 1;
  if (amax_hi > 0x7c00u)
    amax_hi = 0x7c00u;
  for (uint32_t ab = amax_lo; ab < amax_hi; ++ab) {
    const float amax = oracle_half_to_float((uint16_t)ab);
    const float scale = amax / 127.0f;
    const float y = 1.0f / scale;
    for (uint32_t xb = 0; xb <= ab; ++xb) {
      for (int neg = 0; neg < 2; ++neg) {
        const float x =
            oracle_half_to_float((uint16_t)(xb | (neg ? 0x8000u : 0u)));
        const float exact = x / scale;
        const float q0 = x * y;
        const float r = fmaf(-q0, scale, x);
        const float fast = fmaf(r, y, q0);
        ++n;
        if (exact != fast)
          ++bad;
        else if (f2u(exact) != f2u(fast))
          ++bad_zero;
        if (rintf(exact) != rintf(fast))
          ++bad_int;
        const float a = fabsf(rintf(exact));
        if (a > maxq)
          maxq = a;
      }
    }
  }
  if (sign_of_zero)
    *sign_of_zero = bad_zero;
  if (int_mismatch)
    *int_mismatch = bad_int;
  if (checked)
    *checked = n;
  if (max_abs_q)
    *max_abs_q = maxq;
  return bad;
}

/* ---- W5: GEMM --------------------------------------------------------------
 * C = A * B with A[M,K] row-major bf16, B column-major given as Bt[N,K]
 * row-major bf16.  c32 (optional) receives the accumulated value before the
 * final rounding; c16 (optional) the bf16 result.  The fp32 statement
 * accumulates in k order in fp32 (each bf16 x bf16 product is exact in fp32);
 * the fp64 statement accumulates in double and rounds once. */
void oracle_gemm_bf16_f32acc(const uint16_t *a, size_t lda, const uint16_t *bt,
                             size_t ldb, uint16_t *c16, float *c32, size_t ldc,
                             size_t m, size_t n, size_t k) {
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (size_t p = 0; p < k; ++p)
        acc += oracle_bf16_to_float(a[i * lda + p]) *
               oracle_bf16_to_float(bt[j * ldb + p]);
      if (c32)
        c32[i * ldc + j] = acc;
      if (c16)
        c16[i * ldc + j] = oracle_float_to_bf16(acc);
    }
}

void oracle_gemm_bf16_f64acc(const uint16_t *a, size_t lda, const uint16_t *bt,
                             size_t ldb, uint16_t *c16, float *c32, size_t ldc,
                             size_t m, size_t n, size_t k) {
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      double acc = 0.0;
      for (size_t p = 0; p < k; ++p)
        acc += (double)oracle_bf16_to_float(a[i * lda + p]) *
               (double)oracle_bf16_to_float(bt[j * ldb + p]);
      if (c32)
        c32[i * ldc + j] = (float)acc;
      if (c16)
        c16[i * ldc + j] = oracle_float_to_bf16((float)acc);
    }
}

/* ---- launch geometry -------------------------------------------------------
 * gpu-runtime/hip-runtime/src/Runtime.cpp:161-191: a budget of 1024 work-items
 * is handed out dimension by dimension, x first; a dimension of size > 1 takes
 * min(size, budget) and divides the budget by that value rounded up to a power
 * of two. */
int oracle_suggest_block_size(const size_t *global, size_t *block,
                              size_t ndims) {
  if (ndims < 1 || ndims > 3)
    return 1;
  size_t budget = 1024;
  for (size_t i = 0; i < ndims; ++i) {
    if (global[i] > 1) {
      size_t l = global[i] < budget ? global[i] : budget;
      block[i] = l;
      size_t p = 1;
      while (p < l)
        p <<= 1;
      budget /= p;
    } else {
      block[i] = 1;
    }
  }
  return 0;
}

/* mlir/lib/Transforms/LowerHKernel.cpp:284-367: group counts are
 * ceil(work/group) per Python dimension; grid and block are those lists
 * reversed (last Python dimension -> x) and padded with ones to three. */
void oracle_launch_geometry(const size_t *work, const size_t *group,
                            size_t rank, size_t grid[3], size_t block[3]) {
  for (int i = 0; i < 3; ++i) {
    grid[i] = 1;
    block[i] = 1;
  }
  for (size_t i = 0; i < rank; ++i) {
    const size_t x = rank - 1 - i;
    grid[x] = (work[i] + group[i] - 1) / group[i];
    block[x] = group[i];
  }
}

/* ---- array forms of the scalar conversions (for bulk checks) --------------- */
void oracle_half_to_float_n(const uint16_t *h, float *f, size_t n) {
  for (size_t i = 0; i < n; ++i)
    f[i] = oracle_half_to_float(h[i]);
}
void oracle_float_to_half_n(const float *f, uint16_t *h, size_t n) {
  for (size_t i = 0; i < n; ++i)
    h[i] = oracle_float_to_half(f[i]);
}
void oracle_float_to_bf16_n(const float *f, uint16_t *b, size_t n) {
  for (size_t i = 0; i < n; ++i)
    b[i] = oracle_float_to_bf16(f[i]);
}
