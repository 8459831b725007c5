// Fused elementwise map over int32 tiles: out[i] = f(in0[i], ..., in3[i]) for an
// integer expression f given as a short postfix program, the integer sibling of
// the fp32 map kernel.  It covers what the reference's tile wrapper forwards
// to NumPy for integer tiles (python/hckernel/kernel_api.py:157-211): + - *
// // % minimum maximum & | ^ << >> comparisons, negation, abs, bitwise not, with
// NumPy's int32 semantics:
//   * + - * and negation wrap around (two's complement);
//   * // rounds towards minus infinity and % takes the sign of the divisor;
//   * an element whose divisor is zero becomes INACTIVE, as numpy.ma makes it,
//     and stays inactive through everything computed from it: nothing is stored
//     for it.  (Two exceptions, numpy.ma's own: its test is
//     |a| * tiny >= |b|, and |INT_MIN| overflows to a negative number, so
//     INT_MIN // 0 and INT_MIN % 0 stay active with NumPy's result 0, and a
//     divisor INT_MIN deactivates whatever the dividend is.)
//   * << and >> with a count outside 0..31 give 0 (>> of a negative value: -1),
//     which is what NumPy defines; >> is arithmetic;
//   * comparisons give 0 / 1.
//   * IOP_SELECT is numpy.where: it picks from the values, whatever became of
//     their activity (the dividend under a failed //, 1 under a failed %), and
//     the result is a plain array, every element of which is stored.
// The evaluation stack has four entries held in four fixed registers per
// element (top of stack in t0; a push moves the others down, a pop moves them
// up), so no register is ever indexed.  A lane owns four consecutive elements
// of a row: one 16-byte access per operand where rows allow it.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kMaxIn = 4;
constexpr int kMaxProg = 32;
constexpr int kV = 4; // elements per lane

enum : uint32_t {
  IOP_END = 0, IOP_IN = 1, IOP_CONST = 2,
  IOP_ADD = 3, IOP_SUB = 4, IOP_MUL = 5, IOP_FLOORDIV = 6, IOP_MOD = 7, IOP_MIN = 8, IOP_MAX = 9,
  IOP_AND = 10, IOP_OR = 11, IOP_XOR = 12, IOP_SHL = 13, IOP_SHR = 14,
  IOP_LT = 15, IOP_LE = 16, IOP_EQ = 17, IOP_NE = 18, IOP_GE = 19, IOP_GT = 20,
  IOP_NEG = 21, IOP_ABS = 22, IOP_NOT = 23, IOP_LNOT = 24,
  IOP_ACTIVE = 25, // 1 where the element is still active, else 0; the element is active again
  IOP_SELECT = 26, // numpy.where(c, a, b) with c, a, b the three top entries (b on top): the element is active again
};

struct Instr {
  uint16_t op;
  uint16_t arg;
  int32_t imm; // the bit pattern the float field of the host structure carries
};

struct IMapArgs {
  const int32_t *in[kMaxIn];
  void *out;
  size_t ld[kMaxIn];
  size_t ldo;
  size_t rows, cols;
  uint32_t out_u8; // the output holds one byte per element (bool results)
  uint32_t vec;    // every row of every operand and of the output starts 16-byte aligned
  uint32_t n_instr;
  Instr prog[kMaxProg];
};

__device__ __forceinline__ int32_t wrap_add(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
__device__ __forceinline__ int32_t wrap_sub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
__device__ __forceinline__ int32_t wrap_mul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }

// floor division and the remainder that goes with it; ok is cleared for b == 0,
// and the value is what numpy.ma leaves under the deactivated result (the
// dividend of //, the fill value 1 of %), which numpy.where may pick up
__device__ __forceinline__ int32_t floor_div(int32_t a, int32_t b, bool &ok) {
  if (b == 0) {
    ok = ok && a == INT32_MIN;
    return a == INT32_MIN ? 0 : a;
  }
  if (b == INT32_MIN) { // numpy.ma's test sees |INT_MIN| as a negative number: always deactivated
    ok = false;
    return a;
  }
  if (b == -1)
    return wrap_sub(0, a); // INT_MIN / -1 wraps instead of trapping
  int32_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0)))
    --q;
  return q;
}
__device__ __forceinline__ int32_t floor_mod(int32_t a, int32_t b, bool &ok) {
  if (b == 0) {
    ok = ok && a == INT32_MIN;
    return a == INT32_MIN ? 0 : 1;
  }
  if (b == INT32_MIN) {
    ok = false;
    return 1;
  }
  if (b == -1)
    return 0;
  int32_t r = a % b;
  if (r != 0 && ((r < 0) != (b < 0)))
    r += b;
  return r;
}

__device__ __forceinline__ int32_t binary(uint32_t op, int32_t a, int32_t b, bool &ok) {
  switch (op) {
  case IOP_ADD: return wrap_add(a, b);
  case IOP_SUB: return wrap_sub(a, b);
  case IOP_MUL: return wrap_mul(a, b);
  case IOP_FLOORDIV: return floor_div(a, b, ok);
  case IOP_MOD: return floor_mod(a, b, ok);
  case IOP_MIN: return a < b ? a : b;
  case IOP_MAX: return a > b ? a : b;
  case IOP_AND: return a & b;
  case IOP_OR: return a | b;
  case IOP_XOR: return a ^ b;
  case IOP_SHL: return (uint32_t)b < 32u ? (int32_t)((uint32_t)a << b) : 0;
  case IOP_SHR: return (uint32_t)b < 32u ? (a >> b) : (a < 0 ? -1 : 0);
  case IOP_LT: return a < b;
  case IOP_LE: return a <= b;
  case IOP_EQ: return a == b;
  case IOP_NE: return a != b;
  case IOP_GE: return a >= b;
  default: return a > b; // IOP_GT
  }
}
__device__ __forceinline__ int32_t unary(uint32_t op, int32_t a) {
  switch (op) {
  case IOP_NEG: return wrap_sub(0, a);
  case IOP_ABS: return a < 0 ? wrap_sub(0, a) : a;
  case IOP_NOT: return ~a;
  default: return a == 0; // IOP_LNOT
  }
}
} // namespace

extern "C" __global__ __launch_bounds__(256) void hcamd_imap_i32(IMapArgs a) {
  const size_t row = blockIdx.y;
  const size_t col0 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * kV;
  if (col0 >= a.cols)
    return;
  const bool whole = col0 + kV <= a.cols;
  int32_t v[kMaxIn][kV];
#pragma unroll
  for (int i = 0; i < kMaxIn; ++i) {
    if (!a.in[i]) { // uniform: operands are packed from 0
#pragma unroll
      for (int e = 0; e < kV; ++e)
        v[i][e] = 0;
      continue;
    }
    const int32_t *p = a.in[i] + row * a.ld[i] + col0;
    if (a.vec && whole) {
      const u32x4 w = *reinterpret_cast<const u32x4 *>(p);
#pragma unroll
      for (int e = 0; e < kV; ++e)
        v[i][e] = (int32_t)w[e];
    } else {
#pragma unroll
      for (int e = 0; e < kV; ++e)
        v[i][e] = col0 + e < a.cols ? p[e] : 0;
    }
  }
  int32_t t0[kV], t1[kV], t2[kV], t3[kV];
  bool ok[kV];
#pragma unroll
  for (int e = 0; e < kV; ++e) {
    t0[e] = t1[e] = t2[e] = t3[e] = 0;
    ok[e] = true;
  }
  for (uint32_t pc = 0; pc < a.n_instr; ++pc) {
    const uint32_t op = a.prog[pc].op, arg = a.prog[pc].arg;
    const int32_t imm = a.prog[pc].imm;
    if (op == IOP_IN || op == IOP_CONST) {
#pragma unroll
      for (int e = 0; e < kV; ++e) {
        t3[e] = t2[e];
        t2[e] = t1[e];
        t1[e] = t0[e];
        int32_t x = imm;
        if (op == IOP_IN)
          x = arg == 0 ? v[0][e] : arg == 1 ? v[1][e] : arg == 2 ? v[2][e] : v[3][e];
        t0[e] = x;
      }
    } else if (op == IOP_ACTIVE) {
      // `tile.mask`: a plain array of which elements are active, every one of
      // them a value that is stored
#pragma unroll
      for (int e = 0; e < kV; ++e) {
        t0[e] = ok[e] ? 1 : 0;
        ok[e] = true;
      }
    } else if (op == IOP_SELECT) {
      // numpy.where returns a plain array: chosen from the values, every element active
#pragma unroll
      for (int e = 0; e < kV; ++e) {
        t0[e] = t2[e] != 0 ? t1[e] : t0[e];
        t1[e] = t3[e];
        ok[e] = true;
      }
    } else if (op >= IOP_NEG) {
#pragma unroll
      for (int e = 0; e < kV; ++e)
        t0[e] = unary(op, t0[e]);
    } else {
#pragma unroll
      for (int e = 0; e < kV; ++e) {
        t0[e] = binary(op, t1[e], t0[e], ok[e]);
        t1[e] = t2[e];
        t2[e] = t3[e];
      }
    }
  }
  const bool all_ok = ok[0] && ok[1] && ok[2] && ok[3];
  if (a.out_u8) {
    uint8_t *o = static_cast<uint8_t *>(a.out) + row * a.ldo + col0;
#pragma unroll
    for (int e = 0; e < kV; ++e)
      if (col0 + e < a.cols && ok[e])
        o[e] = (uint8_t)(t0[e] != 0);
  } else {
    int32_t *o = static_cast<int32_t *>(a.out) + row * a.ldo + col0;
    if (a.vec && whole && all_ok) {
      u32x4 w;
#pragma unroll
      for (int e = 0; e < kV; ++e)
        w[e] = (uint32_t)t0[e];
      *reinterpret_cast<u32x4 *>(o) = w;
    } else {
#pragma unroll
      for (int e = 0; e < kV; ++e)
        if (col0 + e < a.cols && ok[e])
          o[e] = t0[e];
    }
  }
}
