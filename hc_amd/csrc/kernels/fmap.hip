// General elementwise map over fp32 / fp16 tiles with numpy.ma's activity rules:
// out[i] = f(in0[i], ..., in3[i]) for a postfix program f, the float sibling of
// the int32 map kernel.  It exists for what the fast fp32 map kernel leaves out
// of the operators the reference's tile wrapper forwards to numpy.ma
// (python/hckernel/kernel_api.py:157-211) -- // and %, the six comparisons --
// and for expressions in which the value numpy.ma leaves under a deactivated
// element is seen again.  Every stack entry carries, per element, whether the
// element is still active in it.  The rules are numpy.ma's (NumPy 2, float32;
// fp16 tiles: every operation in fp32 followed by FOP_R16, which is how
// NumPy's half loops work):
//   * the tile operators + - * give the first operand's value where an operand
//     is inactive; called as NumPy functions (`arg` bit 1) they compute from the
//     values whatever their activity.
//   * the tile operators / and // : the element becomes inactive if the divisor
//     is zero or the result is not finite (tested in the tile's type: `arg`
//     bit 0 = fp16), and its value becomes 0 + dividend; an active quotient has
//     0 * dividend added (numpy.ma's way of restoring the dividend), which
//     turns -0 into +0 unless the dividend is negative.
//   * % is ndarray's operator and reaches numpy.ma through __array_wrap__: the
//     remainder is computed everywhere; where the divisor is zero or the
//     dividend infinite (and neither is NaN) the element becomes inactive with
//     the value 1.  FOP_UDIV is numpy.divide called as a function: the same
//     test, value 1, otherwise the plain quotient.
//   * // and % follow NumPy's divmod: fmod, then the Python sign convention,
//     the quotient snapped to the nearest integer, signed zeros.
//   * numpy.sqrt / numpy.log: where the operand is inactive or outside the
//     domain (x < 0; x <= 0) the element is inactive with the value 0 / 1.
//     Functions without a domain (exp, abs, rint, maximum, minimum, negation)
//     compute from the values and keep the activity.
//   * ** : FOP_PSQRT is the square root of x ** 0.5 (the operand's value where
//     it is inactive), FOP_POWCHK what numpy.ma.power does afterwards: a result
//     that is not finite becomes inactive with the value 1e20.
//   * comparisons give 0 / 1 and are false for NaN except !=.  Under an inactive
//     result the tile operators == and != leave 1 / 0 where both operands are
//     inactive and 0 / 1 where one is (numpy.ma compares the activity there);
//     `arg` bit 1 (numpy.equal / not_equal called as functions) compares the values.
//   * FOP_ACTIVE is `tile.mask`: 1 where the element is active, 0 where not, a
//     plain array (every element active again).  FOP_SELECT is numpy.where: a
//     plain array too, chosen from the values whatever their activity.
//   * an int32 operand is converted when it is read (tile.astype(float32)).
//   * `arg` bit 4 on a binary operation: the second operand's activity does not
//     count (a bare numpy.ma array % tile, and the other operators numpy.ma does
//     not define itself: ndarray's operator converts the tile to its values).
//   * `arg` bit 2: the operands are plain NumPy arrays (what numpy.where, numpy.dot
//     and tile.mask return, and arithmetic of those), so the operation is NumPy's
//     own: IEEE quotients, remainders, roots and logarithms, nothing deactivated.
// The store skips inactive elements, or with store_all writes every value: a
// NumPy function returns a bare numpy.ma array, which the reference's store
// copies in full.
// Four stack entries in four fixed registers per element, four consecutive
// elements per lane (one 16-byte fp32 or 8-byte fp16 access per operand where
// rows allow it).  This is a correctness path for HBM-bound work, not tuned.
#include "common.h"
#include <type_traits>

using namespace hcamd;

namespace {
constexpr int kMaxIn = 4;
constexpr int kMaxProg = 48;

enum : uint32_t {
  FOP_END = 0, FOP_IN = 1, FOP_CONST = 2,
  FOP_ADD = 3, FOP_SUB = 4, FOP_MUL = 5, FOP_DIV = 6, FOP_FLOORDIV = 7, FOP_MOD = 8,
  FOP_MIN = 9, FOP_MAX = 10, FOP_UDIV = 11,
  FOP_LT = 12, FOP_LE = 13, FOP_EQ = 14, FOP_NE = 15, FOP_GE = 16, FOP_GT = 17,
  FOP_NEG = 18, FOP_ABS = 19, FOP_SQRT = 20, FOP_RINT = 21, FOP_EXP = 22, FOP_LOG = 23,
  FOP_R16 = 24, FOP_PSQRT = 25, FOP_POWCHK = 26,
  FOP_ACTIVE = 27, // `tile.mask`: 1 where the element is active in the entry, else 0; active again
  FOP_TANH = 28,
  // numpy.where(c, a, b) with c, a, b the three top entries (b on top): NumPy takes the
  // values whatever their activity and returns a plain array, so the result is active
  FOP_SELECT = 29,
  // more NumPy functions of one operand: computed from the values, activity kept;
  // log2 and log10 have numpy.ma's domain like log (inactive with the value 1)
  FOP_FLOOR = 30, FOP_CEIL = 31, FOP_TRUNC = 32, FOP_SIGN = 33, FOP_EXP2 = 34, FOP_LOG2 = 35,
  FOP_LOG10 = 36, FOP_LOG1P = 37, FOP_EXPM1 = 38, FOP_SIN = 39, FOP_COS = 40, FOP_RECIP = 41,
  // `tile[:] = value` and the in-place operators (tile op= x is tile[:] = tile op x): of the
  // two top entries (the tile below, the value on top) the value where it is active, the
  // tile's own element elsewhere; active where either is
  FOP_MERGE = 42,
};

struct Instr {
  uint16_t op;
  uint16_t arg;
  float imm;
};

struct FMapArgs {
  const void *in[kMaxIn];
  void *out;
  size_t ld[kMaxIn];
  size_t ldo;
  size_t rows, cols;
  uint32_t f16_mask; // bit i: operand i is fp16; bit 8 + i: operand i is int32 (converted when read)
  uint32_t out_type; // 0 fp32, 1 fp16, 2 one byte of 0 / 1
  uint32_t vec;      // every row of every operand and of the output starts 16-byte aligned
  uint32_t store_all; // write inactive elements too
  uint32_t n_instr;
  Instr prog[kMaxProg];
};

__device__ __forceinline__ bool finite(float x) { return __builtin_fabsf(x) < __builtin_inff(); }
__device__ __forceinline__ float round16(float x) {
  _Float16 h = (_Float16)x;
  asm volatile("" : "+v"(h));
  return (float)h;
}
// NumPy's maximum / minimum: a NaN wins, and of two equal values (+0 and -0) the second
__device__ __forceinline__ float nan_max(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float nan_min(float a, float b) { return (a < b || a != a) ? a : b; }

// NumPy's divmod for b != 0: the remainder takes the divisor's sign, the
// quotient is (a - mod) / b snapped to the nearest integer
__device__ __forceinline__ float np_divmod(float a, float b, float &mod) {
  mod = fmodf(a, b);
  float div = (a - mod) / b;
  if (mod != 0.0f) {
    if ((b < 0.0f) != (mod < 0.0f)) {
      mod += b;
      div -= 1.0f;
    }
  } else {
    mod = __builtin_copysignf(0.0f, b);
  }
  float fl;
  if (div != 0.0f) {
    fl = __builtin_floorf(div);
    if (div - fl > 0.5f)
      fl += 1.0f;
  } else {
    fl = __builtin_copysignf(0.0f, a / b);
  }
  return fl;
}
__device__ __forceinline__ float np_floor_divide(float a, float b) {
  if (b == 0.0f)
    return a / b;
  float mod;
  return np_divmod(a, b, mod);
}
__device__ __forceinline__ float np_remainder(float a, float b) {
  if (b == 0.0f)
    return fmodf(a, b);
  float mod;
  (void)np_divmod(a, b, mod);
  return mod;
}

// numpy.ma's test for a division: the divisor is zero or the dividend
// infinite, and neither is NaN (|a| * tiny >= |b| in float64)
__device__ __forceinline__ bool unsafe_divide(float a, float b) {
  return a == a && b == b && (b == 0.0f || __builtin_fabsf(a) == __builtin_inff());
}

// one binary operation; ok comes in as "active in both operands"
__device__ __forceinline__ float binary(uint32_t op, float a, float b, uint32_t arg, bool &ok,
                                        bool both_inactive) {
  const bool half = arg & 1u, as_function = arg & 2u;
  const bool plain = arg & 4u; // plain arrays: NumPy's own arithmetic
  switch (op) {
  case FOP_ADD: return (ok || as_function) ? a + b : a;
  case FOP_SUB: return (ok || as_function) ? a - b : a;
  case FOP_MUL: return (ok || as_function) ? a * b : a;
  case FOP_DIV:
  case FOP_FLOORDIV: {
    float r = op == FOP_DIV ? a / b : np_floor_divide(a, b);
    if (plain)
      return r;
    if (half)
      r = round16(r);
    if (!ok || b == 0.0f || !finite(r)) {
      ok = false;
      return 0.0f + a;
    }
    return r + 0.0f * a;
  }
  case FOP_MOD:
  case FOP_UDIV:
    if (!plain && unsafe_divide(a, b)) {
      ok = false;
      return 1.0f;
    }
    return op == FOP_MOD ? np_remainder(a, b) : a / b;
  // NumPy's half loops keep the first of two equal values, its float loops the
  // second; `arg` bit 3: the program evaluated the operands in the other order
  case FOP_MIN:
  case FOP_MAX: {
    const float x = (arg & 8u) ? b : a, y = (arg & 8u) ? a : b;
    if (op == FOP_MIN)
      return half ? ((x <= y || x != x) ? x : y) : nan_min(x, y);
    return half ? ((x >= y || x != x) ? x : y) : nan_max(x, y);
  }
  case FOP_LT: return a < b ? 1.0f : 0.0f;
  case FOP_LE: return a <= b ? 1.0f : 0.0f;
  // numpy.ma's == and != leave "both inactive" / "one inactive" under an
  // inactive result; numpy.equal / not_equal as functions compare the values
  case FOP_EQ: return (ok || as_function) ? (a == b ? 1.0f : 0.0f) : (both_inactive ? 1.0f : 0.0f);
  case FOP_NE: return (ok || as_function) ? (a != b ? 1.0f : 0.0f) : (both_inactive ? 0.0f : 1.0f);
  case FOP_GE: return a >= b ? 1.0f : 0.0f;
  default: return a > b ? 1.0f : 0.0f; // FOP_GT
  }
}
__device__ __forceinline__ float unary(uint32_t op, float a, uint32_t arg, bool &ok) {
  const bool plain = arg & 4u; // a plain array: NumPy's own function, NaN and infinities included
  switch (op) {
  case FOP_NEG: return -a;
  case FOP_ABS: return __builtin_fabsf(a);
  case FOP_SQRT:
    if (!plain && (!ok || a < 0.0f)) {
      ok = false;
      return 0.0f;
    }
    return __builtin_sqrtf(a);
  case FOP_LOG:
    if (!plain && (!ok || a <= 0.0f)) {
      ok = false;
      return 1.0f;
    }
    return logf(a);
  case FOP_LOG2:
  case FOP_LOG10:
    if (!plain && (!ok || a <= 0.0f)) {
      ok = false;
      return 1.0f;
    }
    return op == FOP_LOG2 ? log2f(a) : log10f(a);
  case FOP_RINT: return __builtin_rintf(a);
  case FOP_FLOOR: return __builtin_floorf(a);
  case FOP_CEIL: return __builtin_ceilf(a);
  case FOP_TRUNC: return __builtin_truncf(a);
  // numpy.sign: -1, 0 (the operand's zero is not kept: +0), 1, NaN for NaN
  case FOP_SIGN: return a > 0.0f ? 1.0f : a < 0.0f ? -1.0f : a == 0.0f ? 0.0f : a;
  case FOP_EXP2: return exp2f(a);
  case FOP_LOG1P: return log1pf(a);
  case FOP_EXPM1: return expm1f(a);
  case FOP_SIN: return sinf(a);
  case FOP_COS: return cosf(a);
  case FOP_RECIP: return 1.0f / a;
  case FOP_EXP: return expf(a);
  case FOP_TANH: return tanh_selects(a);
  case FOP_R16: return round16(a);
  case FOP_PSQRT: return ok ? __builtin_sqrtf(a) + 0.0f : a; // pow(-0, 0.5) is +0
  case FOP_ACTIVE: {
    const float r = ok ? 1.0f : 0.0f;
    ok = true;
    return r;
  }
  default: // FOP_POWCHK
    if (!finite(a)) {
      ok = false;
      return 1e20f;
    }
    return a;
  }
}
} // namespace

// V elements of a lane to a dispatch of the interpreter, consecutive in the row
// and moved in pieces of four (16 bytes of fp32, 8 of fp16).
namespace {
template <int V> __device__ __forceinline__ void fmap_row_pieces(const FMapArgs &a) {
  const size_t row = blockIdx.y;
  const size_t col0 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (col0 >= a.cols)
    return;
  const bool whole = col0 + V <= a.cols;
  float v[kMaxIn][V];
#pragma unroll
  for (int i = 0; i < kMaxIn; ++i) {
    if (!a.in[i]) { // uniform: operands are packed from 0
#pragma unroll
      for (int e = 0; e < V; ++e)
        v[i][e] = 0.0f;
      continue;
    }
    if ((a.f16_mask >> i) & 1) {
      const _Float16 *p = static_cast<const _Float16 *>(a.in[i]) + row * a.ld[i] + col0;
      if (a.vec && whole) {
#pragma unroll
        for (int g = 0; g < V / 4; ++g) {
          const f16x4 w = ldg<true>(reinterpret_cast<const f16x4 *>(p) + g);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[i][4 * g + e] = (float)w[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e)
          v[i][e] = col0 + e < a.cols ? (float)p[e] : 0.0f;
      }
    } else if ((a.f16_mask >> (8 + i)) & 1) {
      const int32_t *p = static_cast<const int32_t *>(a.in[i]) + row * a.ld[i] + col0;
#pragma unroll
      for (int e = 0; e < V; ++e)
        v[i][e] = col0 + e < a.cols ? (float)p[e] : 0.0f;
    } else {
      const float *p = static_cast<const float *>(a.in[i]) + row * a.ld[i] + col0;
      if (a.vec && whole) {
#pragma unroll
        for (int g = 0; g < V / 4; ++g) {
          const f32x4 w = ldg<true>(reinterpret_cast<const f32x4 *>(p) + g);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[i][4 * g + e] = w[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e)
          v[i][e] = col0 + e < a.cols ? p[e] : 0.0f;
      }
    }
  }
  // the stack and, beside every entry, whether the element is still active in it
  float t0[V], t1[V], t2[V], t3[V];
  bool k0[V], k1[V], k2[V], k3[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    t0[e] = t1[e] = t2[e] = t3[e] = 0.0f;
    k0[e] = k1[e] = k2[e] = k3[e] = true;
  }
  for (uint32_t pc = 0; pc < a.n_instr; ++pc) {
    const uint32_t op = a.prog[pc].op, arg = a.prog[pc].arg;
    const float imm = a.prog[pc].imm;
    if (op == FOP_IN || op == FOP_CONST) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        t3[e] = t2[e];
        t2[e] = t1[e];
        t1[e] = t0[e];
        k3[e] = k2[e];
        k2[e] = k1[e];
        k1[e] = k0[e];
        float x = imm;
        if (op == FOP_IN)
          x = arg == 0 ? v[0][e] : arg == 1 ? v[1][e] : arg == 2 ? v[2][e] : v[3][e];
        t0[e] = x;
        k0[e] = true;
      }
    } else if (op == FOP_SELECT) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        t0[e] = t2[e] != 0.0f ? t1[e] : t0[e];
        k0[e] = true;
        t1[e] = t3[e];
        k1[e] = k3[e];
      }
    } else if (op == FOP_MERGE) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        t0[e] = k0[e] ? t0[e] : t1[e];
        k0[e] = k0[e] || k1[e];
        t1[e] = t2[e];
        t2[e] = t3[e];
        k1[e] = k2[e];
        k2[e] = k3[e];
      }
    } else if (op >= FOP_NEG) {
      // one branch on the operation for all the elements of the lane: inside
      // `each` the operation is a constant and the function's own switch folds
      auto each = [&](auto tag) {
        constexpr uint32_t OP = decltype(tag)::value;
#pragma unroll
        for (int e = 0; e < V; ++e)
          t0[e] = unary(OP, t0[e], arg, k0[e]);
      };
#define HCAMD_FMAP_CASE(X)                                                       \
  case X:                                                                        \
    each(std::integral_constant<uint32_t, X>{});                                 \
    break;
      switch (op) {
        HCAMD_FMAP_CASE(FOP_NEG) HCAMD_FMAP_CASE(FOP_ABS) HCAMD_FMAP_CASE(FOP_SQRT) HCAMD_FMAP_CASE(FOP_RINT)
        HCAMD_FMAP_CASE(FOP_EXP) HCAMD_FMAP_CASE(FOP_LOG) HCAMD_FMAP_CASE(FOP_R16) HCAMD_FMAP_CASE(FOP_PSQRT)
        HCAMD_FMAP_CASE(FOP_ACTIVE) HCAMD_FMAP_CASE(FOP_TANH) HCAMD_FMAP_CASE(FOP_FLOOR) HCAMD_FMAP_CASE(FOP_CEIL)
        HCAMD_FMAP_CASE(FOP_TRUNC) HCAMD_FMAP_CASE(FOP_SIGN) HCAMD_FMAP_CASE(FOP_EXP2) HCAMD_FMAP_CASE(FOP_LOG2)
        HCAMD_FMAP_CASE(FOP_LOG10) HCAMD_FMAP_CASE(FOP_LOG1P) HCAMD_FMAP_CASE(FOP_EXPM1) HCAMD_FMAP_CASE(FOP_SIN)
        HCAMD_FMAP_CASE(FOP_COS) HCAMD_FMAP_CASE(FOP_RECIP)
      default:
        each(std::integral_constant<uint32_t, FOP_POWCHK>{});
        break;
      }
    } else {
      auto each = [&](auto tag) {
        constexpr uint32_t OP = decltype(tag)::value;
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const bool second = k0[e] || (arg & 16u);
          bool ok = k1[e] && second;
          t0[e] = binary(OP, t1[e], t0[e], arg, ok, !k1[e] && !second);
          k0[e] = ok;
          t1[e] = t2[e];
          t2[e] = t3[e];
          k1[e] = k2[e];
          k2[e] = k3[e];
        }
      };
      switch (op) {
        HCAMD_FMAP_CASE(FOP_ADD) HCAMD_FMAP_CASE(FOP_SUB) HCAMD_FMAP_CASE(FOP_MUL) HCAMD_FMAP_CASE(FOP_DIV)
        HCAMD_FMAP_CASE(FOP_FLOORDIV) HCAMD_FMAP_CASE(FOP_MOD) HCAMD_FMAP_CASE(FOP_MIN) HCAMD_FMAP_CASE(FOP_MAX)
        HCAMD_FMAP_CASE(FOP_UDIV) HCAMD_FMAP_CASE(FOP_LT) HCAMD_FMAP_CASE(FOP_LE) HCAMD_FMAP_CASE(FOP_EQ)
        HCAMD_FMAP_CASE(FOP_NE) HCAMD_FMAP_CASE(FOP_GE)
      default:
        each(std::integral_constant<uint32_t, FOP_GT>{});
        break;
      }
#undef HCAMD_FMAP_CASE
    }
  }
  bool ok[V];
#pragma unroll
  for (int e = 0; e < V; ++e)
    ok[e] = k0[e] || a.store_all != 0;
  bool all_ok = true;
#pragma unroll
  for (int e = 0; e < V; ++e)
    all_ok = all_ok && ok[e];
  if (a.out_type == 2) {
    uint8_t *o = static_cast<uint8_t *>(a.out) + row * a.ldo + col0;
#pragma unroll
    for (int e = 0; e < V; ++e)
      if (col0 + e < a.cols && ok[e])
        o[e] = (uint8_t)(t0[e] != 0.0f);
  } else if (a.out_type == 1) {
    _Float16 *o = static_cast<_Float16 *>(a.out) + row * a.ldo + col0;
    if (a.vec && whole && all_ok) {
#pragma unroll
      for (int g = 0; g < V / 4; ++g) {
        f16x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w[e] = (_Float16)t0[4 * g + e];
        stg<true>(reinterpret_cast<f16x4 *>(o) + g, w);
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (col0 + e < a.cols && ok[e])
          o[e] = (_Float16)t0[e];
    }
  } else {
    float *o = static_cast<float *>(a.out) + row * a.ldo + col0;
    if (a.vec && whole && all_ok) {
#pragma unroll
      for (int g = 0; g < V / 4; ++g) {
        f32x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w[e] = t0[4 * g + e];
        stg<true>(reinterpret_cast<f32x4 *>(o) + g, w);
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (col0 + e < a.cols && ok[e])
          o[e] = t0[e];
    }
  }
}
} // namespace
extern "C" __global__ __launch_bounds__(256) void hcamd_fmap(FMapArgs a) { fmap_row_pieces<4>(a); }
// eight elements of a lane to a dispatch, for rows of 2048 columns or more
extern "C" __global__ __launch_bounds__(256) void hcamd_fmap_v8(FMapArgs a) { fmap_row_pieces<8>(a); }

// ---- elementwise expressions of gathered tiles ------------------------------------
// out_g[mo(e)] = f(in0_g[m0(e)], ...) for every group g and tile element e: what
// a body computes that loads its tiles through index mappings, or stores one
// through a mapping, outside a matrix product (CurrentGroup.load / store with
// mapping=..., python/hckernel/kernel_api.py:304-310,319-335).  x_g is the
// window of buffer x that starts at starts[g][d] along dimension d; element e
// of a tile sits at index[e][d] of the window and is active if 0 <= index[e][d]
// < shape[d] - starts[g][d] for every d (the reference's bounds test; an
// unmapped operand has the identity table).  Inactive operand elements are
// zeros that deactivate what is computed from them under the rules above;
// inactive output positions are not written, and neither are deactivated
// results unless store_all.  One tile element per lane: the accesses are
// gathers, so there is nothing to vectorise.
namespace {
struct GatherMapOperand {
  const int32_t *starts; // [groups][4]
  const int32_t *index;  // [tile elements][4]
  uint32_t shape[4];     // 1 for the dimensions the buffer does not have
  uint32_t strides[4];   // in elements
};
struct GatherMapArgs {
  const void *in[kMaxIn];
  void *out;
  GatherMapOperand op[kMaxIn + 1]; // the inputs, then the output
  uint32_t n_in, tile_elems, chunks; // chunks: workgroups per group
  uint32_t f16_mask;  // bit i: operand i is fp16; bit 8 + i: operand i is int32 (converted when read)
  uint32_t out_type;  // 0 fp32, 1 fp16, 2 one byte of 0 / 1
  uint32_t store_all; // write deactivated results too: 1 as computed, 2 as NaN (0 in a bool buffer)
  uint32_t copy_bytes; // != 0: no program, operand 0 is copied as elements of this many bytes
  uint32_t n_instr;
  Instr prog[kMaxProg];
};
// offset of element e of group g in elements, or -1 if the element is inactive
__device__ __forceinline__ int64_t gather_offset(const GatherMapOperand &o, uint32_t g, uint32_t e) {
  int64_t at = 0;
  bool inside = true;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int32_t st = o.starts[(size_t)g * 4 + d], ix = o.index[(size_t)e * 4 + d];
    inside = inside && ix >= 0 && (int64_t)ix < (int64_t)o.shape[d] - st;
    at += ((int64_t)st + ix) * o.strides[d];
  }
  return inside ? at : -1;
}
} // namespace

extern "C" __global__ __launch_bounds__(256) void hcamd_gather_fmap(GatherMapArgs a) {
  const uint32_t g = blockIdx.x / a.chunks;
  const uint32_t e = (blockIdx.x % a.chunks) * 256 + threadIdx.x;
  if (e >= a.tile_elems)
    return;
  const int64_t dst = gather_offset(a.op[a.n_in], g, e);
  if (dst < 0)
    return;
  if (a.copy_bytes) {
    const int64_t src = gather_offset(a.op[0], g, e);
    if (src < 0)
      return;
    switch (a.copy_bytes) {
    case 1: static_cast<uint8_t *>(a.out)[dst] = static_cast<const uint8_t *>(a.in[0])[src]; break;
    case 2: static_cast<uint16_t *>(a.out)[dst] = static_cast<const uint16_t *>(a.in[0])[src]; break;
    case 4: static_cast<uint32_t *>(a.out)[dst] = static_cast<const uint32_t *>(a.in[0])[src]; break;
    default: static_cast<uint64_t *>(a.out)[dst] = static_cast<const uint64_t *>(a.in[0])[src]; break;
    }
    return;
  }
  float v[kMaxIn];
  bool act[kMaxIn];
#pragma unroll
  for (int i = 0; i < kMaxIn; ++i) {
    v[i] = 0.0f;
    act[i] = false;
    if (i < (int)a.n_in) {
      const int64_t at = gather_offset(a.op[i], g, e);
      act[i] = at >= 0;
      if (at >= 0)
        v[i] = ((a.f16_mask >> i) & 1)         ? (float)static_cast<const _Float16 *>(a.in[i])[at]
               : ((a.f16_mask >> (8 + i)) & 1) ? (float)static_cast<const int32_t *>(a.in[i])[at]
                                               : static_cast<const float *>(a.in[i])[at];
    }
  }
  float t0 = 0.0f, t1 = 0.0f, t2 = 0.0f, t3 = 0.0f;
  bool k0 = true, k1 = true, k2 = true, k3 = true;
  for (uint32_t pc = 0; pc < a.n_instr; ++pc) {
    const uint32_t op = a.prog[pc].op, arg = a.prog[pc].arg;
    if (op == FOP_IN || op == FOP_CONST) {
      t3 = t2, t2 = t1, t1 = t0;
      k3 = k2, k2 = k1, k1 = k0;
      t0 = a.prog[pc].imm;
      k0 = true;
      if (op == FOP_IN) {
        t0 = arg == 0 ? v[0] : arg == 1 ? v[1] : arg == 2 ? v[2] : v[3];
        k0 = arg == 0 ? act[0] : arg == 1 ? act[1] : arg == 2 ? act[2] : act[3];
      }
    } else if (op == FOP_MERGE) {
      t0 = k0 ? t0 : t1;
      k0 = k0 || k1;
      t1 = t2, t2 = t3;
      k1 = k2, k2 = k3;
    } else if (op == FOP_SELECT) {
      t0 = t2 != 0.0f ? t1 : t0;
      k0 = true;
      t1 = t3;
      k1 = k3;
    } else if (op >= FOP_NEG) {
      t0 = unary(op, t0, arg, k0);
    } else {
      const bool second = k0 || (arg & 16u);
      bool ok = k1 && second;
      t0 = binary(op, t1, t0, arg, ok, !k1 && !second);
      k0 = ok;
      t1 = t2, t2 = t3;
      k1 = k2, k2 = k3;
    }
  }
  if (!(k0 || a.store_all))
    return;
  if (!k0 && a.store_all == 2)
    t0 = a.out_type == 2 ? 0.0f : __builtin_nanf("");
  if (a.out_type == 2)
    static_cast<uint8_t *>(a.out)[dst] = (uint8_t)(t0 != 0.0f);
  else if (a.out_type == 1)
    static_cast<_Float16 *>(a.out)[dst] = (_Float16)t0;
  else
    static_cast<float *>(a.out)[dst] = t0;
}
