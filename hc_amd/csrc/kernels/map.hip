// Fused elementwise map: out[i] = f(in0[i], ..., in3[i]) for an expression f
// that is handed to the kernel as a short postfix program, so that a kernel body
// made of loads, arithmetic and one store runs as ONE pass over HBM without any
// code being generated at run time.
//
// The program runs on a four-entry evaluation stack of fp32 values.  The stack
// pointer is uniform over the whole grid, so the interpreter switches on it and
// on the opcode with scalar branches only, and every stack entry has a fixed
// register in each arm: no indexed register access, no spills.  One pass of the
// program serves eight elements per lane (the scalar unit issues one
// instruction per SIMD every four cycles, and the two dozen scalar compares and
// branches of a dispatch are what an interpreted instruction costs; more
// elements per pass would amortise them, but the registers that takes cost more
// in occupancy than it gains).  Operands stay packed in registers as
// loaded (16 bytes per eight fp16, 32 per eight fp32) and are converted when
// the program pushes them, which keeps the kernel at four waves per SIMD.
//
// Arithmetic is IEEE fp32 with no contraction (a*b+c is two roundings, as in
// NumPy); R16 rounds the top of the stack to fp16 and back, which is how
// arithmetic on fp16 tiles is expressed (for + - * / sqrt, rounding the fp32
// result to fp16 equals computing in fp16 directly).  MAX/MIN propagate NaN like
// numpy.maximum / numpy.minimum.
//
// Storage types: fp32 and fp16 per operand.  Flat form: all operands contiguous
// and 16-byte aligned, treated as one vector.  Strided form: a rows x cols
// window with a leading dimension per operand, any alignment, one scalar access
// per element.
#include "common.h"

#include <type_traits>

#pragma clang fp contract(off)

using namespace hcamd;

namespace {
constexpr int kThreads = 256;
constexpr int kDepth = 4;    // evaluation stack entries
constexpr int kMaxIn = 4;    // operands
constexpr int kMaxProg = 32; // instructions
#ifndef HCAMD_MAP_WAVES
#define HCAMD_MAP_WAVES 5 // resident waves per SIMD the flat kernel is compiled for
#endif
constexpr int kN = 8; // elements per lane per run of the program (one chunk)

// Opcodes.  The numbering is part of the C ABI (hcamdLaunchMap).
enum : uint32_t {
  OP_END = 0,
  OP_IN = 1,    // push operand `arg`
  OP_CONST = 2, // push imm
  // pop b, pop a, push a op b
  OP_ADD = 3,
  OP_SUB = 4,
  OP_MUL = 5,
  OP_DIV = 6,
  OP_MAX = 7,
  OP_MIN = 8,
  OP_RSUB = 9,  // b - a
  OP_RDIV = 10, // b / a
  // top = top op imm
  OP_ADDI = 11,
  OP_SUBI = 12,
  OP_MULI = 13,
  OP_DIVI = 14,
  OP_MAXI = 15,
  OP_MINI = 16,
  OP_RSUBI = 17, // imm - top
  OP_RDIVI = 18, // imm / top
  // top = f(top)
  OP_NEG = 19,
  OP_ABS = 20,
  OP_SQRT = 21,
  OP_RINT = 22,
  OP_EXP = 23,
  OP_LOG = 24,
  OP_TANH = 25,
  OP_R16 = 26, // round to fp16 and back
  // top = top op operand `arg` (a binary operation whose right side is an
  // operand: one dispatch instead of two)
  OP_ADD_IN = 27,
  OP_SUB_IN = 28,
  OP_MUL_IN = 29,
  OP_DIV_IN = 30,
  OP_MAX_IN = 31,
  OP_MIN_IN = 32,
  OP_RSUB_IN = 33, // operand - top
  OP_RDIV_IN = 34, // operand / top
  OP_COUNT = 35,
  // The tile operator `/` as numpy.ma computes it: a quotient that is not finite
  // (a zero divisor gives one) deactivates its element, whose value becomes the
  // dividend.  `arg` bit 8 (any `arg` for MDIV / RMDIV): the tile is fp16 and
  // the quotient is rounded to fp16 before the test.
  OP_MDIV = 35,
  OP_RMDIV = 36,
  OP_MDIVI = 37,
  OP_RMDIVI = 38,
  OP_MDIV_IN = 39,
  OP_RMDIV_IN = 40,
  OP_CLEAR = 41,  // every element active again (a NumPy function returns a plain array)
  OP_POWCHK = 42, // numpy.ma.power: a result that is not finite deactivates, value 1e20
  OP_MSQRT = 43,  // numpy.sqrt of a tile: x < 0 deactivates, value 0
  OP_MLOG = 44,   // numpy.log of a tile: x <= 0 deactivates, value 1
  // 45 .. 55 are the row programs' scalar forms (below): the highest opcodes,
  // so that one comparison finds them
};

struct Instr {
  uint16_t op;
  uint16_t arg;
  float imm;
};

struct MapArgs {
  const void *in[kMaxIn];
  void *out;
  size_t ld[kMaxIn]; // leading dimensions in elements (strided form)
  size_t ldo;
  size_t rows, cols; // flat form: rows = 1, cols = element count
  uint32_t f16_mask; // bit i: operand i is fp16; bit 8: the output is fp16
  uint32_t n_instr;
  Instr prog[kMaxProg];
};

// NumPy's maximum / minimum: a NaN wins, and of two equal values (+0 and -0) the second
__device__ __forceinline__ float nan_max(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float nan_min(float a, float b) { return (a < b || a != a) ? a : b; }
__device__ __forceinline__ float round16(float x) {
  _Float16 h = (_Float16)x;
  asm volatile("" : "+v"(h)); // keep the conversion pair from being folded
  return (float)h;
}

template <int OP> __device__ __forceinline__ float binary(float a, float b) {
  if constexpr (OP == OP_ADD) return a + b;
  if constexpr (OP == OP_SUB) return a - b;
  if constexpr (OP == OP_MUL) return a * b;
  if constexpr (OP == OP_DIV) return a / b;
  if constexpr (OP == OP_MAX) return nan_max(a, b);
  if constexpr (OP == OP_MIN) return nan_min(a, b);
  if constexpr (OP == OP_RSUB) return b - a;
  if constexpr (OP == OP_RDIV) return b / a;
  return a;
}
template <int OP> __device__ __forceinline__ float unary(float a) {
  if constexpr (OP == OP_NEG) return -a;
  if constexpr (OP == OP_ABS) return __builtin_fabsf(a);
  if constexpr (OP == OP_SQRT) return __builtin_sqrtf(a);
  if constexpr (OP == OP_RINT) return __builtin_rintf(a);
  if constexpr (OP == OP_EXP) return expf(a);
  if constexpr (OP == OP_LOG) return logf(a);
  if constexpr (OP == OP_TANH) return tanh_selects(a);
  if constexpr (OP == OP_R16) return round16(a);
  return a;
}

// Operands of one chunk of N elements, as loaded: N fp16 in w[..][0 .. N/8-1],
// or N fp32 in w[..][0 .. N/4-1].  The kernels below work on chunks of eight;
// so do the row programs (the chunk size is a parameter because sixteen was tried there).
template <int N> struct RawT {
  u32x4 w[kMaxIn][N / 4];
};
template <int N> struct StackT {
  float st[kDepth][N];
  uint32_t bad; // bit e: element e of the chunk is inactive (masked operators only)
};
using Raw = RawT<kN>;
using Stack = StackT<kN>;

template <int N>
__device__ __forceinline__ void unpack(const RawT<N> &raw, int i, bool f16, float *dst) {
  // The empty asm statements pin the conversion to the arm that pushes the
  // operand: hoisted out of the interpreter loop it would hold N more
  // registers per operand for the whole pass.
  if (f16) {
#pragma unroll
    for (int j = 0; j < N / 8; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t w = raw.w[i][j][e];
        asm volatile("" : "+v"(w));
        dst[8 * j + 2 * e] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
        dst[8 * j + 2 * e + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N / 4; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t w = raw.w[i][j][e];
        asm volatile("" : "+v"(w));
        dst[4 * j + e] = __builtin_bit_cast(float, w);
      }
    }
  }
}

template <int SP, int OP, int N> __device__ __forceinline__ void do_binary(StackT<N> &r) {
  if constexpr (SP >= 2) {
#pragma unroll
    for (int e = 0; e < N; ++e)
      r.st[SP - 2][e] = binary<OP>(r.st[SP - 2][e], r.st[SP - 1][e]);
  }
}
template <int SP, int OP, int N>
__device__ __forceinline__ void do_imm(StackT<N> &r, float imm) {
  if constexpr (SP >= 1) {
    // the same operation with the immediate as the second operand
    constexpr int B = OP == OP_ADDI   ? OP_ADD
                      : OP == OP_SUBI ? OP_SUB
                      : OP == OP_MULI ? OP_MUL
                      : OP == OP_DIVI ? OP_DIV
                      : OP == OP_MAXI ? OP_MAX
                      : OP == OP_MINI ? OP_MIN
                      : OP == OP_RSUBI ? OP_RSUB
                                       : OP_RDIV;
#pragma unroll
    for (int e = 0; e < N; ++e)
      r.st[SP - 1][e] = binary<B>(r.st[SP - 1][e], imm);
  }
}
template <int SP, int OP, int N>
__device__ __forceinline__ void do_operand(StackT<N> &r, const RawT<N> &raw, uint32_t f16_mask,
                                           uint32_t arg) {
  if constexpr (SP >= 1) {
    constexpr int B = OP - OP_ADD_IN + OP_ADD; // the plain binary operation
    float t[N];
    switch (arg) {
    case 0: unpack(raw, 0, f16_mask & 1, t); break;
    case 1: unpack(raw, 1, f16_mask & 2, t); break;
    case 2: unpack(raw, 2, f16_mask & 4, t); break;
    default: unpack(raw, 3, f16_mask & 8, t); break;
    }
#pragma unroll
    for (int e = 0; e < N; ++e)
      r.st[SP - 1][e] = binary<B>(r.st[SP - 1][e], t[e]);
  }
}
template <int SP, int OP, int N> __device__ __forceinline__ void do_unary(StackT<N> &r) {
  if constexpr (SP >= 1) {
#pragma unroll
    for (int e = 0; e < N; ++e)
      r.st[SP - 1][e] = unary<OP>(r.st[SP - 1][e]);
  }
}

__device__ __forceinline__ bool is_finite(float x) { return __builtin_fabsf(x) < INFINITY; }
// num / den under numpy.ma's rule, into `dst`
template <int N, int B0 = 0> // B0: the bit of element 0
__device__ __forceinline__ void masked_div(uint32_t &bad_bits, float *dst, const float *num,
                                           const float *den, bool half) {
  uint32_t bad = bad_bits;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float n = num[e];
    float q = n / den[e];
    if (half)
      q = round16(q);
    const bool good = is_finite(q);
    // numpy.ma adds 0 * dividend to the quotient (it restores the dividend under
    // the mask that way): a quotient of -0 becomes +0 unless the dividend is negative
    q += 0.0f * n;
    dst[e] = good ? q : 0.0f + n;
    bad |= good ? 0u : (1u << (B0 + e));
  }
  bad_bits = bad;
}
// the same with one of the two a scalar (an immediate, a row scalar): v = v / s, or v = s / v
template <int N, bool REVERSED>
__device__ __forceinline__ void masked_div_scalar(uint32_t &bad_bits, float *v, float s, bool half) {
  uint32_t bad = bad_bits;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float n = REVERSED ? s : v[e];
    float q = REVERSED ? s / v[e] : v[e] / s;
    if (half)
      q = round16(q);
    const bool good = is_finite(q);
    q += 0.0f * n;
    v[e] = good ? q : 0.0f + n;
    bad |= good ? 0u : (1u << e);
    if (e % 4 == 3)
      __builtin_amdgcn_sched_barrier(0);
  }
  bad_bits = bad;
}
// numpy.sqrt / numpy.log of a tile: outside the domain the element is
// deactivated and holds numpy.ma's fill value (0 and 1)
template <bool LOG, int N> __device__ __forceinline__ void domain_fn(uint32_t &bad_bits, float *x) {
  uint32_t bad = bad_bits;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float v = x[e];
    const bool out = LOG ? v <= 0.0f : v < 0.0f;
    const float y = LOG ? logf(v) : __builtin_sqrtf(v);
    x[e] = out ? (LOG ? 1.0f : 0.0f) : y;
    bad |= out ? (1u << e) : 0u;
  }
  bad_bits = bad;
}
// numpy.ma.power: a result that is not finite deactivates, value 1e20
template <int N> __device__ __forceinline__ void powchk_fn(uint32_t &bad_bits, float *x) {
  uint32_t bad = bad_bits;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const bool good = is_finite(x[e]);
    x[e] = good ? x[e] : 1e20f;
    bad |= good ? 0u : (1u << e);
  }
  bad_bits = bad;
}
template <int SP, int OP, int N>
__device__ __forceinline__ void do_masked(StackT<N> &r, const RawT<N> &raw, uint32_t f16_mask, uint32_t arg,
                                          float imm) {
  if constexpr (OP == OP_MDIV || OP == OP_RMDIV) {
    if constexpr (SP >= 2) {
      if constexpr (OP == OP_MDIV)
        masked_div<N>(r.bad, r.st[SP - 2], r.st[SP - 2], r.st[SP - 1], arg != 0);
      else
        masked_div<N>(r.bad, r.st[SP - 2], r.st[SP - 1], r.st[SP - 2], arg != 0);
    }
  } else if constexpr (SP >= 1) {
    float t[N];
    if constexpr (OP == OP_MDIVI || OP == OP_RMDIVI) {
#pragma unroll
      for (int e = 0; e < N; ++e) t[e] = imm;
    } else {
      switch (arg & 3u) {
      case 0: unpack(raw, 0, f16_mask & 1, t); break;
      case 1: unpack(raw, 1, f16_mask & 2, t); break;
      case 2: unpack(raw, 2, f16_mask & 4, t); break;
      default: unpack(raw, 3, f16_mask & 8, t); break;
      }
    }
    const bool half = (arg & 0x100u) != 0;
    if constexpr (OP == OP_MDIVI || OP == OP_MDIV_IN)
      masked_div<N>(r.bad, r.st[SP - 1], r.st[SP - 1], t, half);
    else
      masked_div<N>(r.bad, r.st[SP - 1], t, r.st[SP - 1], half);
  }
}
template <int SP, bool LOG, int N> __device__ __forceinline__ void do_domain(StackT<N> &r) {
  if constexpr (SP >= 1)
    domain_fn<LOG, N>(r.bad, r.st[SP - 1]);
}
template <int SP, int N> __device__ __forceinline__ void do_powchk(StackT<N> &r) {
  if constexpr (SP >= 1)
    powchk_fn<N>(r.bad, r.st[SP - 1]);
}

// One instruction with SP entries on the stack; returns the new stack pointer.
// The host has verified the program, so pushes never overflow and pops never
// underflow; the guards only keep impossible arms out of the code.
template <int SP, int N>
__device__ __forceinline__ int step(StackT<N> &r, const RawT<N> &raw, uint32_t f16_mask,
                                    uint32_t op, uint32_t arg, float imm) {
  switch (op) {
  case OP_IN:
    if constexpr (SP < kDepth) {
      switch (arg) {
      case 0: unpack(raw, 0, f16_mask & 1, r.st[SP]); break;
      case 1: unpack(raw, 1, f16_mask & 2, r.st[SP]); break;
      case 2: unpack(raw, 2, f16_mask & 4, r.st[SP]); break;
      default: unpack(raw, 3, f16_mask & 8, r.st[SP]); break;
      }
    }
    return SP + 1;
  case OP_CONST:
    if constexpr (SP < kDepth) {
#pragma unroll
      for (int e = 0; e < N; ++e) r.st[SP][e] = imm;
    }
    return SP + 1;
#define HCAMD_BIN(OP)                                                          \
  case OP:                                                                     \
    do_binary<SP, OP>(r);                                                      \
    return SP - 1;
    HCAMD_BIN(OP_ADD)
    HCAMD_BIN(OP_SUB)
    HCAMD_BIN(OP_MUL)
    HCAMD_BIN(OP_DIV)
    HCAMD_BIN(OP_MAX)
    HCAMD_BIN(OP_MIN)
    HCAMD_BIN(OP_RSUB)
    HCAMD_BIN(OP_RDIV)
#undef HCAMD_BIN
#define HCAMD_IMM(OP)                                                          \
  case OP:                                                                     \
    do_imm<SP, OP>(r, imm);                                                    \
    return SP;
    HCAMD_IMM(OP_ADDI)
    HCAMD_IMM(OP_SUBI)
    HCAMD_IMM(OP_MULI)
    HCAMD_IMM(OP_DIVI)
    HCAMD_IMM(OP_MAXI)
    HCAMD_IMM(OP_MINI)
    HCAMD_IMM(OP_RSUBI)
    HCAMD_IMM(OP_RDIVI)
#undef HCAMD_IMM
#define HCAMD_UN(OP)                                                           \
  case OP:                                                                     \
    do_unary<SP, OP>(r);                                                       \
    return SP;
    HCAMD_UN(OP_NEG)
    HCAMD_UN(OP_ABS)
    HCAMD_UN(OP_SQRT)
    HCAMD_UN(OP_RINT)
    HCAMD_UN(OP_EXP)
    HCAMD_UN(OP_LOG)
    HCAMD_UN(OP_TANH)
    HCAMD_UN(OP_R16)
#undef HCAMD_UN
#define HCAMD_OPND(OP)                                                         \
  case OP:                                                                     \
    do_operand<SP, OP>(r, raw, f16_mask, arg);                                 \
    return SP;
    HCAMD_OPND(OP_ADD_IN)
    HCAMD_OPND(OP_SUB_IN)
    HCAMD_OPND(OP_MUL_IN)
    HCAMD_OPND(OP_DIV_IN)
    HCAMD_OPND(OP_MAX_IN)
    HCAMD_OPND(OP_MIN_IN)
    HCAMD_OPND(OP_RSUB_IN)
    HCAMD_OPND(OP_RDIV_IN)
#undef HCAMD_OPND
  case OP_MDIV:
    do_masked<SP, OP_MDIV>(r, raw, f16_mask, arg, imm);
    return SP - 1;
  case OP_RMDIV:
    do_masked<SP, OP_RMDIV>(r, raw, f16_mask, arg, imm);
    return SP - 1;
#define HCAMD_MASKED(OP)                                                       \
  case OP:                                                                     \
    do_masked<SP, OP>(r, raw, f16_mask, arg, imm);                             \
    return SP;
    HCAMD_MASKED(OP_MDIVI)
    HCAMD_MASKED(OP_RMDIVI)
    HCAMD_MASKED(OP_MDIV_IN)
    HCAMD_MASKED(OP_RMDIV_IN)
#undef HCAMD_MASKED
  case OP_CLEAR:
    r.bad = 0;
    return SP;
  case OP_POWCHK:
    do_powchk<SP>(r);
    return SP;
  case OP_MSQRT:
    do_domain<SP, false>(r);
    return SP;
  case OP_MLOG:
    do_domain<SP, true>(r);
    return SP;
  default:
    return SP;
  }
}

// Runs the program; the result is r.st[0].  Instructions are fetched with
// scalar loads from the argument block, the next one before the current one is
// dispatched.
__device__ __forceinline__ void run_program(const MapArgs &a, const Raw &raw,
                                            uint32_t f16_mask, Stack &r) {
  int sp = 0;
  r.bad = 0;
  Instr next = a.prog[0];
  for (uint32_t pc = 0; pc < a.n_instr; ++pc) {
    const Instr cur = next;
    next = a.prog[(pc + 1) & (kMaxProg - 1)];
    const uint32_t op = cur.op, arg = cur.arg;
    const float imm = cur.imm;
    switch (sp) {
    case 0: sp = step<0>(r, raw, f16_mask, op, arg, imm); break;
    case 1: sp = step<1>(r, raw, f16_mask, op, arg, imm); break;
    case 2: sp = step<2>(r, raw, f16_mask, op, arg, imm); break;
    case 3: sp = step<3>(r, raw, f16_mask, op, arg, imm); break;
    default: sp = step<4>(r, raw, f16_mask, op, arg, imm); break;
    }
  }
}

// ---- operand access -------------------------------------------------------------
__device__ __forceinline__ void store_elem(void *p, bool f16, size_t i, float v);
// bad: bit e set = element e is inactive and keeps what the output holds
__device__ __forceinline__ void store_chunk(void *p, bool f16, size_t chunk,
                                            const float *src, uint32_t bad = 0) {
  if (bad & 0xffu) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (!((bad >> e) & 1u))
        store_elem(p, f16, chunk * 8 + e, src[e]);
    return;
  }
  if (f16) {
    f16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (_Float16)src[e];
    stg<true>(static_cast<f16x8 *>(p) + chunk, v);
  } else {
    f32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = src[e];
      hi[e] = src[4 + e];
    }
    f32x4 *q = static_cast<f32x4 *>(p) + 2 * chunk;
    stg<true>(q, lo);
    stg<true>(q + 1, hi);
  }
}
__device__ __forceinline__ float load_elem(const void *p, bool f16, size_t i) {
  return f16 ? (float)static_cast<const _Float16 *>(p)[i]
             : static_cast<const float *>(p)[i];
}
__device__ __forceinline__ void store_elem(void *p, bool f16, size_t i, float v) {
  if (f16)
    static_cast<_Float16 *>(p)[i] = (_Float16)v;
  else
    static_cast<float *>(p)[i] = v;
}
// Element-wise gather of one chunk: slot e of every operand from index idx(e),
// zero where idx(e) is out of range; kept as fp32 whatever the operand type.
template <class Index>
__device__ __forceinline__ void gather(const MapArgs &a, uint32_t n_in, Raw &raw,
                                       Index index) {
#pragma unroll
  for (int i = 0; i < kMaxIn; ++i)
    if (i < (int)n_in) {
#pragma unroll
      for (int e = 0; e < kN; ++e) {
        size_t off;
        const bool ok = index(i, e, off);
        const float v = ok ? load_elem(a.in[i], (a.f16_mask >> i) & 1, off) : 0.0f;
        raw.w[i][e / 4][e % 4] = __builtin_bit_cast(uint32_t, v);
      }
    }
}

template <int T> __device__ __forceinline__ void finish_sum(float acc, float *cell) {
  __shared__ float slots[T / kWave];
  const float total = group_reduce<SumOp, T / kWave>(acc, slots);
  if (threadIdx.x == 0)
    unsafeAtomicAdd(cell, total);
}

// Flat form of the map-reduce (SUM = true: all results added up into one fp32
// cell; SUM = false, one stored result per element, is kept for measurements).
//
// Chunk = eight consecutive elements.  A pass of a lane covers U chunks, 256
// apart; workgroup g starts at chunk g * 256 * U and strides by gridDim.x * 256
// * U.  The loads of all U chunks are issued together, then the program runs on
// one chunk after the other, so a lane keeps U times the bytes in flight for the
// same number of registers when there are few operands (NIN) or all of them are
// fp16 (HALF).  The staged chunks are shifted down one place per run instead of
// being indexed, and the loop over them is kept rolled, which keeps a single
// copy of the interpreter in the code.  Every lane makes the same number of
// passes and runs; out-of-range ones are predicated off, so the interpreter's
// control flow stays uniform.  The elements after the last whole chunk are
// finished by the last lane of the last workgroup, one by one.
template <int NIN, int U, bool HALF, bool SUM>
__device__ __forceinline__ void map_flat(const MapArgs &a, const uint32_t n_in) {
  // The reduction runs with 1024 lanes per workgroup: one workgroup fills a CU,
  // so a launch ends in a few hundred atomic additions to the one cell, not
  // thousands (they are served one after the other, some 15 ns each).
  constexpr int kThreads = SUM ? 1024 : 256;
  constexpr int W = HALF ? 1 : 2;
  const size_t n = a.cols;
  const size_t n_chunks = n / 8;
  const size_t stride = (size_t)gridDim.x * (kThreads * U);
  const size_t passes = (n_chunks + stride - 1) / stride;
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  size_t c0 = (size_t)blockIdx.x * (kThreads * U) + threadIdx.x;
  const bool all_f32 = (a.f16_mask & ((1u << n_in) - 1u)) == 0;
  float acc = 0.0f;
  Raw raw;
  Stack r;
  for (size_t p = 0; p < passes; ++p, c0 += stride) {
    u32x4 staged[NIN][U][W];
#pragma unroll
    for (int i = 0; i < NIN; ++i)
      if (i < (int)n_in) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const size_t chunk = c0 + (size_t)u * kThreads;
          if (chunk < n_chunks) {
            const bool f16 = HALF || ((a.f16_mask >> i) & 1);
            bool done = false;
            if constexpr (SUM && !HALF) {
              // a sum does not care which elements a lane adds: two runs of four,
              // 256 elements apart, so that the wave's accesses are whole cache lines
              if (all_f32 && (chunk | 63) < n_chunks) {
                const u32x4 *q =
                    static_cast<const u32x4 *>(a.in[i]) + 2 * (chunk & ~(size_t)63) + (chunk & 63);
                staged[i][u][0] = ldg<true>(q);
                staged[i][u][1] = ldg<true>(q + 64);
                done = true;
              }
            }
            if (!done) {
              const u32x4 *q = static_cast<const u32x4 *>(a.in[i]) + (f16 ? chunk : 2 * chunk);
              staged[i][u][0] = ldg<true>(q);
              if constexpr (!HALF)
                if (!f16)
                  staged[i][u][1] = ldg<true>(q + 1);
            }
          }
        }
      }
#pragma nounroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < NIN; ++i) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
          raw.w[i][w] = staged[i][0][w];
#pragma unroll
          for (int k = 0; k + 1 < U; ++k)
            staged[i][k][w] = staged[i][k + 1][w];
        }
      }
      run_program(a, raw, a.f16_mask, r);
      const size_t chunk = c0 + (size_t)u * kThreads;
      if (chunk < n_chunks) {
        if constexpr (SUM) {
#pragma unroll
          for (int e = 0; e < kN; ++e)
            acc += ((r.bad >> e) & 1u) ? 0.0f : r.st[0][e];
        } else {
          store_chunk(a.out, out_f16, chunk, r.st[0], r.bad);
        }
      }
    }
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == kThreads - 1 && n_chunks * 8 < n) {
    gather(a, n_in, raw, [&](int, int e, size_t &off) {
      off = n_chunks * 8 + e;
      return off < n;
    });
    run_program(a, raw, 0, r);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (n_chunks * 8 + e < n && !((r.bad >> e) & 1u)) {
        if constexpr (SUM)
          acc += r.st[0][e];
        else
          store_elem(a.out, out_f16, n_chunks * 8 + e, r.st[0][e]);
      }
  }
  if constexpr (SUM)
    finish_sum<kThreads>(acc, static_cast<float *>(a.out));
}

// Strided form: a work item is a run of 256 * 8 columns of one row; lane t takes
// columns t, t + 256, ... of the run, so a wave reads consecutive elements.  The
// map launches one workgroup per item (blockIdx.y = row, x = run); the reduction
// launches a grid capped by the host whose workgroups stride over the items, row
// after row, and ends in one atomic addition per workgroup.
template <bool SUM>
__device__ __forceinline__ void map_strided(const MapArgs &a, const uint32_t n_in) {
  float acc = 0.0f;
  auto item = [&](const size_t row, const size_t run) {
    const size_t col0 = run * (kThreads * kN) + threadIdx.x;
    Raw raw;
    gather(a, n_in, raw, [&](int i, int e, size_t &off) {
      const size_t col = col0 + (size_t)e * kThreads;
      off = row * a.ld[i] + col;
      return col < a.cols;
    });
    Stack r;
    run_program(a, raw, 0, r);
#pragma unroll
    for (int e = 0; e < kN; ++e) {
      const size_t col = col0 + (size_t)e * kThreads;
      if (col < a.cols && !((r.bad >> e) & 1u)) {
        if constexpr (SUM)
          acc += r.st[0][e];
        else
          store_elem(a.out, (a.f16_mask >> 8) & 1, row * a.ldo + col, r.st[0][e]);
      }
    }
  };
  if constexpr (SUM) {
    const size_t runs = (a.cols + kThreads * kN - 1) / (kThreads * kN);
    const size_t items = a.rows * runs;
    for (size_t i = blockIdx.x; i < items; i += gridDim.x)
      item(i / runs, i % runs);
    finish_sum<kThreads>(acc, static_cast<float *>(a.out));
  } else {
    item(blockIdx.y, blockIdx.x);
  }
}

// Row form for windows whose rows start on 16-byte boundaries: the work items
// are the chunks of all rows, numbered row after row (a row has cols / 8 whole
// chunks and, when cols is not a multiple of 8, one short chunk at its end), and
// lane t of workgroup g takes item g * T + t, then strides by the grid.  Whole
// chunks move with 16-byte accesses like the flat form; a short chunk is read
// element by element (every load issued, from the row's first element where the
// column is past the end, and zeroed afterwards) and packed the way a whole
// chunk arrives, so one run of the interpreter serves both.  The reduction runs
// 1024-lane workgroups on a grid capped by the host, so that it ends in a few
// hundred atomic additions however many rows there are.
template <bool SUM>
__device__ __forceinline__ void map_rows(const MapArgs &a, const uint32_t n_in) {
  constexpr int T = SUM ? 1024 : 256;
  const uint32_t whole = (uint32_t)(a.cols / 8);
  const uint32_t rem = (uint32_t)(a.cols % 8);
  const uint32_t per_row = whole + (rem ? 1u : 0u);
  const uint32_t items = (uint32_t)a.rows * per_row;
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  float acc = 0.0f;
  // every lane makes the same number of passes: the interpreter's control flow
  // stays uniform, passes past the end are predicated off
  auto pass = [&](const uint32_t item) {
    Raw raw;
    Stack r;
    const bool live = item < items;
    const uint32_t row = live ? item / per_row : 0;
    const uint32_t c = live ? item - row * per_row : 0;
    const bool shortc = live && c == whole; // only with rem != 0
    // whole chunks: every lane loads (idle and short-chunk lanes the row's
    // first chunk), so that no load sits in a divergent branch
    const uint32_t cv = (live && !shortc) ? c : 0;
    if (whole) {
#pragma unroll
      for (int i = 0; i < kMaxIn; ++i)
        if (i < (int)n_in) {
          const bool f16 = (a.f16_mask >> i) & 1;
          const char *base = static_cast<const char *>(a.in[i]) +
                             (size_t)row * a.ld[i] * (f16 ? 2 : 4);
          const u32x4 *q = reinterpret_cast<const u32x4 *>(base) + (f16 ? cv : 2 * cv);
          raw.w[i][0] = ldg<true>(q);
          if (!f16)
            raw.w[i][1] = ldg<true>(q + 1);
        }
    }
    if (shortc) {
#pragma unroll
      for (int i = 0; i < kMaxIn; ++i)
        if (i < (int)n_in) {
          const bool f16 = (a.f16_mask >> i) & 1;
          const char *base = static_cast<const char *>(a.in[i]) +
                             (size_t)row * a.ld[i] * (f16 ? 2 : 4);
          uint32_t v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const size_t at = (uint32_t)e < rem ? (size_t)whole * 8 + e : 0;
            v[e] = f16 ? (uint32_t) reinterpret_cast<const uint16_t *>(base)[at]
                       : reinterpret_cast<const uint32_t *>(base)[at];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = (uint32_t)e < rem ? v[e] : 0u;
          if (f16) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              raw.w[i][0][e] = v[2 * e] | (v[2 * e + 1] << 16);
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              raw.w[i][e / 4][e % 4] = v[e];
          }
        }
    }
    run_program(a, raw, a.f16_mask, r);
    if (live) {
      if constexpr (SUM) {
#pragma unroll
        for (int e = 0; e < kN; ++e)
          acc += ((!shortc || (uint32_t)e < rem) && !((r.bad >> e) & 1u)) ? r.st[0][e] : 0.0f;
      } else {
        char *orow = static_cast<char *>(a.out) + (size_t)row * a.ldo * (out_f16 ? 2 : 4);
        if (!shortc) {
          store_chunk(orow, out_f16, c, r.st[0], r.bad);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if ((uint32_t)e < rem && !((r.bad >> e) & 1u))
              store_elem(orow, out_f16, (size_t)whole * 8 + e, r.st[0][e]);
        }
      }
    }
  };
  if constexpr (SUM) {
    const uint32_t stride = gridDim.x * T;
    const uint32_t passes = (items + stride - 1) / stride;
    uint32_t item = blockIdx.x * T + threadIdx.x;
    for (uint32_t p = 0; p < passes; ++p, item += stride)
      pass(item);
    finish_sum<T>(acc, static_cast<float *>(a.out));
  } else {
    pass(blockIdx.x * T + threadIdx.x); // the host launches one lane per item
  }
}
} // namespace

// Map-reduce note: a lane adds up the values of its own elements in fp32, a wave
// folds its lanes with DPP, the four waves meet in LDS, and one lane per
// workgroup issues a single hardware fp32 atomic add; the host caps the grid so
// that at most a few thousand atomics reach the cell.  The order of the
// additions differs from run to run: the result is a correctly computed fp32
// sum, not a bit-reproducible one.
#define HCAMD_MAP_FLAT(NAME, NIN, U, HALF, SUM)                                \
  extern "C" __global__ __launch_bounds__(SUM ? 1024 : 256) __attribute__((    \
      amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void             \
  NAME(const MapArgs a, const uint32_t n_in) {                                 \
    map_flat<NIN, U, HALF, SUM>(a, n_in);                                      \
  }
// name: operands it can take / chunks per pass; h = all operands fp16
HCAMD_MAP_FLAT(hcamd_map_sum_flat_n4u1, 4, 1, false, true)
HCAMD_MAP_FLAT(hcamd_map_sum_flat_n2u2, 2, 2, false, true)
HCAMD_MAP_FLAT(hcamd_map_sum_flat_n1u4, 1, 4, false, true)
HCAMD_MAP_FLAT(hcamd_map_sum_flat_n4u2h, 4, 2, true, true)
HCAMD_MAP_FLAT(hcamd_map_sum_flat_n2u4h, 2, 4, true, true)
// The map itself with one or two fp16 operands: a single chunk per lane
// (hcamd_map_flat below) is 16 or 32 bytes in flight, too few to fill the memory
// system (8192 x 8192: 56 -> 45 us with one operand).  With fp32 operands the
// same form measured slower than one chunk per lane (96 -> 107 us).
HCAMD_MAP_FLAT(hcamd_map_flat_n2u4h, 2, 4, true, false)

// The two commonest reductions without the interpreter: sum(x) and sum(x * y)
// over flat fp32 arrays (a dot product; y = x gives a sum of squares).  One
// 1024-lane workgroup per CU strides over the data with four independent 16-byte
// loads per operand in flight and four partial sums per lane; the end is the
// same as above, one atomic addition per workgroup.
template <bool DOT>
__device__ __forceinline__ void reduce_f32(const float *__restrict__ x,
                                           const float *__restrict__ y,
                                           float *cell, size_t n) {
  const size_t n4 = n / 4;
  const size_t stride = (size_t)gridDim.x * 1024;
  const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
  const f32x4 *y4 = reinterpret_cast<const f32x4 *>(y);
  f32x4 part[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
    part[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  size_t c = (size_t)blockIdx.x * 1024 + threadIdx.x;
  for (; c + 3 * stride < n4; c += 4 * stride) {
    f32x4 a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a[u] = ldg<true>(x4 + c + u * stride);
      if constexpr (DOT)
        b[u] = ldg<true>(y4 + c + u * stride);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      part[u] = DOT ? part[u] + a[u] * b[u] : part[u] + a[u];
  }
  for (; c < n4; c += stride) {
    const f32x4 a = ldg<true>(x4 + c);
    part[0] = DOT ? part[0] + a * ldg<true>(y4 + c) : part[0] + a;
  }
  const f32x4 s = (part[0] + part[1]) + (part[2] + part[3]);
  float acc = (s.x + s.y) + (s.z + s.w);
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 1023)
    for (size_t i = n4 * 4; i < n; ++i)
      acc += DOT ? x[i] * y[i] : x[i];
  finish_sum<1024>(acc, cell);
}
extern "C" __global__ __launch_bounds__(1024) void hcamd_sum_f32(
    const float *x, float *cell, size_t n) {
  reduce_f32<false>(x, x, cell, n);
}
extern "C" __global__ __launch_bounds__(1024) void hcamd_dot_f32(
    const float *x, const float *y, float *cell, size_t n) {
  reduce_f32<true>(x, y, cell, n);
}

// The two commonest reductions down columns without the interpreter: the sums
// of x and of x * x over the rows of a band of a dense fp32 window, into
// partial[band][column] (the first of the two launches of a column reduction;
// the second one, which folds the bands and runs the post program, is the
// general kernel's).  A lane owns four consecutive columns, a wave 256 (1 KiB of
// every row it reads), the W waves of a workgroup take the rows of the band
// in turns, U rows in flight each with an accumulator of its own; the
// accumulators fold in a fixed order, then the waves through LDS in theirs, so
// the result is the same from run to run.  The product is rounded before it is
// added, as the interpreter's multiply-then-fold does.
template <bool SQ, int W, int U, class Finish>
__device__ __forceinline__ void cols_sum_f32(const float *__restrict__ x, size_t ld, uint32_t cols,
                                             uint32_t rows, uint32_t band, Finish finish) {
  __shared__ f32x4 fold[W][kWave];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const uint32_t col = (blockIdx.x * kWave + lane) * 4;
  const uint32_t first = blockIdx.y * band;
  const uint32_t end = (uint32_t)min((uint64_t)first + band, (uint64_t)rows);
  const bool there = col < cols; // cols is a multiple of 4
  f32x4 acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    acc[u] = f32x4{-0.0f, -0.0f, -0.0f, -0.0f}; // (the identity of IEEE addition)
  auto add = [](f32x4 &to, const f32x4 v) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      to[e] += SQ ? __fmul_rn(v[e], v[e]) : v[e];
  };
  if (there) {
    const float *p = x + (size_t)(first + wave) * ld + col;
    uint32_t r = first + wave;
    for (; r + W * (U - 1) < end; r += W * U, p += (size_t)(W * U) * ld) {
      f32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        v[u] = ldg<true>(reinterpret_cast<const f32x4 *>(p + (size_t)(W * u) * ld));
#pragma unroll
      for (int u = 0; u < U; ++u)
        add(acc[u], v[u]);
    }
    // the rows left over, in the accumulators they would have had
#pragma unroll
    for (int u = 0; u < U - 1; ++u)
      if (r + W * u < end)
        add(acc[u], ldg<true>(reinterpret_cast<const f32x4 *>(p + (size_t)(W * u) * ld)));
  }
#pragma unroll
  for (int step = 1; step < U; step *= 2)
#pragma unroll
    for (int u = 0; u + step < U; u += 2 * step)
      acc[u] += acc[u + step];
  fold[wave][lane] = acc[0];
  __syncthreads();
  if (wave == 0 && there) {
    f32x4 part[W];
#pragma unroll
    for (int w = 0; w < W; ++w)
      part[w] = fold[w][lane];
#pragma unroll
    for (int step = 1; step < W; step *= 2)
#pragma unroll
      for (int w = 0; w + step < W; w += 2 * step)
        part[w] += part[w + step];
    finish(part[0], col);
  }
}
#define HCAMD_COLS_SUM(NAME, SQ, W, U)                                                    \
  extern "C" __global__ __launch_bounds__(W * 64) void NAME(                              \
      const float *x, size_t ld, float *partial, uint32_t cols, uint32_t cols_pad,       \
      uint32_t rows, uint32_t band) {                                                     \
    cols_sum_f32<SQ, W, U>(x, ld, cols, rows, band, [&](const f32x4 total, uint32_t col) { \
      *reinterpret_cast<f32x4 *>(partial + (size_t)blockIdx.y * cols_pad + col) = total;  \
    });                                                                                   \
  }
// 16 waves to a workgroup measured fastest, and many short bands (root mean
// square down the columns of 4096 x 8192, both launches; bands of 32 / 48 / 64
// rows): 16 waves x 1 row in flight 24.1 / 24.2 / 27.8 us, 16 x 2 24.5 / 24.7 /
// 27.0, 16 x 4 24.7 / 24.5 / 27.0, 8 x 2 24.7 / 24.3 / 29.9, 4 x 4 27.5 / 25.7 /
// 37.5, 2 x 8 28.3 / 26.1 / 35.9: what counts is the number of waves the launch
// has, each with a row or two to fetch (a read-only stream of the same bytes
// takes 19.9 us, this kernel's launch alone 21.1-21.5 us).
HCAMD_COLS_SUM(hcamd_cols_sum_f32, false, 16, 2)
HCAMD_COLS_SUM(hcamd_cols_sumsq_f32, true, 16, 2)
HCAMD_COLS_SUM(hcamd_cols_sum_f32_w4u8, false, 4, 8)
HCAMD_COLS_SUM(hcamd_cols_sumsq_f32_w4u8, true, 4, 8)

// The map itself: one chunk per lane, one pass, no loop around the interpreter
// (several chunks per pass, or a persistent grid, measured slower here: the
// stores of one workgroup already overlap the loads of the next).
extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void hcamd_map_flat(
    const MapArgs a, const uint32_t n_in) {
  const size_t n = a.cols;
  const size_t n_chunks = n / 8;
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
  // fp32 among the operands or as the output, and the 64 chunks of this wave
  // all there: a lane's eight elements are two runs of four, 256 elements
  // apart, so that each of its two 16-byte accesses to fp32 data is one of 64
  // consecutive ones (1 KiB of whole cache lines per wave and instruction;
  // fp16 data of the same elements: two 8-byte accesses, 512 bytes of whole
  // lines each).  Eight consecutive fp32 elements per lane make every
  // instruction touch 2 KiB of lines and use half of each.
  const size_t wave_first = c & ~(size_t)63, lane = c & 63;
  const uint32_t present = ((1u << n_in) - 1u) | 0x100u;
  const bool split = (~a.f16_mask & present) != 0 && wave_first + 64 <= n_chunks;
  Raw raw;
  // (one branch on the layout around all the loads, not one per operand: the
  // loads of an arm then go out back to back)
  if (split) {
#pragma unroll
    for (int i = 0; i < kMaxIn; ++i)
      if (i < (int)n_in) {
        if ((a.f16_mask >> i) & 1) {
          const u32x2 *q = static_cast<const u32x2 *>(a.in[i]) + 2 * wave_first + lane;
          const u32x2 lo = ldg<true>(q), hi = ldg<true>(q + 64);
          raw.w[i][0] = u32x4{lo.x, lo.y, hi.x, hi.y};
        } else {
          const u32x4 *q = static_cast<const u32x4 *>(a.in[i]) + 2 * wave_first + lane;
          raw.w[i][0] = ldg<true>(q);
          raw.w[i][1] = ldg<true>(q + 64);
        }
      }
  } else if (c < n_chunks) {
#pragma unroll
    for (int i = 0; i < kMaxIn; ++i)
      if (i < (int)n_in) {
        if ((a.f16_mask >> i) & 1) {
          raw.w[i][0] = ldg<true>(static_cast<const u32x4 *>(a.in[i]) + c);
        } else {
          const u32x4 *q = static_cast<const u32x4 *>(a.in[i]) + 2 * c;
          raw.w[i][0] = ldg<true>(q);
          raw.w[i][1] = ldg<true>(q + 1);
        }
      }
  }
  Stack r;
  run_program(a, raw, a.f16_mask, r);
  if (split && out_f16) {
    _Float16 *o = static_cast<_Float16 *>(a.out) + 8 * wave_first + 4 * lane;
    if (r.bad & 0xffu) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (!((r.bad >> e) & 1u))
          o[(e / 4) * 256 + e % 4] = (_Float16)r.st[0][e];
    } else {
      f16x4 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = (_Float16)r.st[0][e];
        hi[e] = (_Float16)r.st[0][4 + e];
      }
      stg<true>(reinterpret_cast<f16x4 *>(o), lo);
      stg<true>(reinterpret_cast<f16x4 *>(o + 256), hi);
    }
  } else if (split) {
    float *o = static_cast<float *>(a.out) + 8 * wave_first + 4 * lane;
    if (r.bad & 0xffu) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (!((r.bad >> e) & 1u))
          o[(e / 4) * 256 + e % 4] = r.st[0][e];
    } else {
      stg<true>(reinterpret_cast<f32x4 *>(o), f32x4{r.st[0][0], r.st[0][1], r.st[0][2], r.st[0][3]});
      stg<true>(reinterpret_cast<f32x4 *>(o + 256), f32x4{r.st[0][4], r.st[0][5], r.st[0][6], r.st[0][7]});
    }
  } else if (c < n_chunks) {
    store_chunk(a.out, out_f16, c, r.st[0], r.bad);
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 255 && n_chunks * 8 < n) {
    gather(a, n_in, raw, [&](int, int e, size_t &off) {
      off = n_chunks * 8 + e;
      return off < n;
    });
    run_program(a, raw, 0, r);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (n_chunks * 8 + e < n && !((r.bad >> e) & 1u))
        store_elem(a.out, out_f16, n_chunks * 8 + e, r.st[0][e]);
  }
}

extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void hcamd_map_strided(
    const MapArgs a, const uint32_t n_in) {
  map_strided<false>(a, n_in);
}
extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void hcamd_map_sum_strided(
    const MapArgs a, const uint32_t n_in) {
  map_strided<true>(a, n_in);
}
extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void hcamd_map_rows(
    const MapArgs a, const uint32_t n_in) {
  map_rows<false>(a, n_in);
}
extern "C" __global__ __launch_bounds__(1024)
__attribute__((amdgpu_waves_per_eu(HCAMD_MAP_WAVES, HCAMD_MAP_WAVES))) void hcamd_map_sum_rows(
    const MapArgs a, const uint32_t n_in) {
  map_rows<true>(a, n_in);
}

// ---- reductions along columns -------------------------------------------------------
// out[c] = post(fold over the rows r of f(in0[r][c], ...)) for a rows x cols
// window: f is the map program, the fold is a sum, a NaN-propagating maximum or
// minimum, and post is a second short program whose operand 0 is the folded
// value (the division of a mean, the square root of a norm).
//
// A lane owns eight columns and walks down the rows.  L lanes share a row (64,
// or the next power of two above the chunks of a narrow row, so that a wave
// covers 64 / L rows at a time and no lane idles); blockIdx.x numbers blocks of
// 8 * L columns.  Where every row of every operand starts on a 16-byte boundary
// a lane's columns are consecutive and move with 16-byte accesses; otherwise the
// columns of a block are dealt to its lanes one by one, so that the element
// accesses of a wave are coalesced (columns are independent: any assignment
// works as long as operands and result agree).  An operand with leading
// dimension 0 is a vector that every row uses.  The waves of a workgroup take
// turns down the workgroup's band of rows; at the end the lanes that share
// columns fold through cross-lane exchanges and the waves meet in LDS.
// blockIdx.y numbers the bands: with more than one, the folded values go to
// partial[band][column] (fp32, `cols_pad` per band) and the host launches the
// kernel again on the bands as the rows of an fp32 operand; the launch with one
// band runs `post` and stores.  Nothing is atomic and every order is fixed:
// results are the same from run to run.
namespace {
constexpr int kPostProg = 8;
enum : uint32_t { COL_SUM = 0, COL_MAX = 1, COL_MIN = 2 };
struct ColArgs {
  float *partial;       // bands x cols_pad, used when gridDim.y > 1
  uint32_t cols_pad;    // multiple of 8, at least cols
  uint32_t band;        // rows per band
  uint32_t kind;
  uint32_t lanes;       // L
  uint32_t interleaved; // columns of a block dealt to the lanes one by one
  uint32_t out_vec;     // the result may be written 16 bytes at a time
  uint32_t n_post;
  uint32_t masked;      // the program has numpy.ma's division / domain forms: inactive elements are left out
  uint32_t fill_empty;  // finishing launch of a maximum / minimum: the identity (no active element) becomes 1e20
  Instr post[kPostProg];
};

__device__ __forceinline__ void run_post(const ColArgs &c, const Raw &raw, Stack &r) {
  int sp = 0;
  Instr next = c.post[0];
  for (uint32_t pc = 0; pc < c.n_post; ++pc) {
    const Instr cur = next;
    next = c.post[(pc + 1) & (kPostProg - 1)];
    const uint32_t op = cur.op, arg = cur.arg;
    const float imm = cur.imm;
    switch (sp) {
    case 0: sp = step<0>(r, raw, 0u, op, arg, imm); break;
    case 1: sp = step<1>(r, raw, 0u, op, arg, imm); break;
    case 2: sp = step<2>(r, raw, 0u, op, arg, imm); break;
    case 3: sp = step<3>(r, raw, 0u, op, arg, imm); break;
    default: sp = step<4>(r, raw, 0u, op, arg, imm); break;
    }
  }
}

// ---- chains: programs that never hold two values at once ------------------------
// An operand (or a constant), then operations that change the value in place:
// the evaluation stack is one value per element, so one dispatch can work on
// several chunks of a lane at once (NE = 16 elements) where the general
// interpreter above affords 8.  The host recognises such programs and folds
// `x x mul` with two equal halves into `x sq`.
constexpr uint32_t OP_SQ = 63; // top = top * top; made by the host, not part of the C ABI

// Four elements at a time: the fence keeps the scheduler from interleaving all
// NE, whose temporaries (a division, an exponential) would not fit.
#define HCAMD_CHAIN_EACH(EXPR)                                                    \
  _Pragma("unroll") for (int g = E0 / 4; g < E1 / 4; ++g) {                       \
    _Pragma("unroll") for (int e = 4 * g; e < 4 * g + 4; ++e) { EXPR; }           \
    __builtin_amdgcn_sched_barrier(0);                                            \
  }

__device__ __forceinline__ bool chain_reads(uint32_t op) {
  return op == OP_IN || (op >= OP_ADD_IN && op <= OP_RDIV_IN) || op == OP_MDIV_IN ||
         op == OP_RMDIV_IN;
}
// v = v op operand for the instructions that name an operand; rhs(e) is the
// operand's element e, read straight from where it was loaded to.
// Elements E0 .. E1-1 of v (all of it, or the part whose operand words are at hand).
template <int NE, int E0 = 0, int E1 = NE, class Rhs>
__device__ __forceinline__ void chain_operand(uint32_t op, float (&v)[NE], uint32_t &bad, bool half,
                                              Rhs rhs) {
  auto apply = [&](auto at) {
    switch (op) {
    case OP_IN: HCAMD_CHAIN_EACH(v[e] = at(e)) break;
    case OP_ADD_IN: HCAMD_CHAIN_EACH(v[e] = v[e] + at(e)) break;
    case OP_SUB_IN: HCAMD_CHAIN_EACH(v[e] = v[e] - at(e)) break;
    case OP_MUL_IN: HCAMD_CHAIN_EACH(v[e] = v[e] * at(e)) break;
    case OP_DIV_IN: HCAMD_CHAIN_EACH(v[e] = v[e] / at(e)) break;
    case OP_MAX_IN: HCAMD_CHAIN_EACH(v[e] = nan_max(v[e], at(e))) break;
    case OP_MIN_IN: HCAMD_CHAIN_EACH(v[e] = nan_min(v[e], at(e))) break;
    case OP_RSUB_IN: HCAMD_CHAIN_EACH(v[e] = at(e) - v[e]) break;
    case OP_RDIV_IN: HCAMD_CHAIN_EACH(v[e] = at(e) / v[e]) break;
    default: { // the numpy.ma quotients
      float x[E1 - E0];
#pragma unroll
      for (int e = E0; e < E1; ++e) x[e - E0] = at(e);
      if (op == OP_MDIV_IN)
        masked_div<E1 - E0, E0>(bad, v + E0, v + E0, x, half);
      else
        masked_div<E1 - E0, E0>(bad, v + E0, x, v + E0, half);
    }
    }
  };
  rhs(apply);
}
// The operand as P chunks of loaded words: 8 fp16 in w[p][0], 8 fp32 in
// w[p][0..1].  (The empty asm statements pin conversions and products of an
// operand that stays in registers to the arm that uses them: hoisted out of the
// surrounding loops, as loop invariants, they would each hold 8 P registers.)
// `word(p, j, c)` is component c of word j of chunk p.
template <class Word> __device__ __forceinline__ auto chain_words(Word word, bool f16) {
  return [word, f16](auto apply) {
    if (f16)
      apply([&](int e) {
        uint32_t x = word(e / 8, 0, (e % 8) / 2);
        asm volatile("" : "+v"(x));
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(e % 2 ? x >> 16 : x & 0xffffu));
      });
    else
      apply([&](int e) {
        uint32_t x = word(e / 8, (e % 8) / 4, e % 4);
        asm volatile("" : "+v"(x));
        return __builtin_bit_cast(float, x);
      });
  };
}
// every other instruction of a chain
template <int NE>
__device__ __forceinline__ void chain_plain(uint32_t op, float (&v)[NE], uint32_t &bad, float imm,
                                            bool half) {
  constexpr int E0 = 0, E1 = NE;
  switch (op) {
  case OP_CONST: HCAMD_CHAIN_EACH(v[e] = imm) break;
  case OP_ADDI: HCAMD_CHAIN_EACH(v[e] = v[e] + imm) break;
  case OP_SUBI: HCAMD_CHAIN_EACH(v[e] = v[e] - imm) break;
  case OP_MULI: HCAMD_CHAIN_EACH(v[e] = v[e] * imm) break;
  case OP_DIVI: HCAMD_CHAIN_EACH(v[e] = v[e] / imm) break;
  case OP_MAXI: HCAMD_CHAIN_EACH(v[e] = nan_max(v[e], imm)) break;
  case OP_MINI: HCAMD_CHAIN_EACH(v[e] = nan_min(v[e], imm)) break;
  case OP_RSUBI: HCAMD_CHAIN_EACH(v[e] = imm - v[e]) break;
  case OP_RDIVI: HCAMD_CHAIN_EACH(v[e] = imm / v[e]) break;
  case OP_NEG: HCAMD_CHAIN_EACH(v[e] = -v[e]) break;
  case OP_ABS: HCAMD_CHAIN_EACH(v[e] = __builtin_fabsf(v[e])) break;
  case OP_SQRT: HCAMD_CHAIN_EACH(v[e] = __builtin_sqrtf(v[e])) break;
  case OP_RINT: HCAMD_CHAIN_EACH(v[e] = __builtin_rintf(v[e])) break;
  case OP_EXP: HCAMD_CHAIN_EACH(v[e] = expf(v[e])) break;
  case OP_LOG: HCAMD_CHAIN_EACH(v[e] = logf(v[e])) break;
  case OP_TANH: HCAMD_CHAIN_EACH(v[e] = tanh_selects(v[e])) break;
  case OP_R16: HCAMD_CHAIN_EACH(v[e] = round16(v[e])) break;
  case OP_SQ: HCAMD_CHAIN_EACH(v[e] = v[e] * v[e]) break;
  case OP_MDIVI:
    masked_div_scalar<NE, false>(bad, v, imm, half);
    break;
  case OP_RMDIVI:
    masked_div_scalar<NE, true>(bad, v, imm, half);
    break;
  case OP_CLEAR:
    bad = 0;
    break;
  case OP_POWCHK:
    powchk_fn<NE>(bad, v);
    break;
  case OP_MSQRT:
    domain_fn<false, NE>(bad, v);
    break;
  case OP_MLOG:
    domain_fn<true, NE>(bad, v);
    break;
  default:
    break;
  }
}
#undef HCAMD_CHAIN_EACH
// an operation on a row scalar that numpy.ma would deactivate the result of
__device__ __forceinline__ bool chain_scalar_fails(uint32_t op, float sv, float imm) {
  return op == OP_MDIVI    ? !is_finite(sv / imm)
         : op == OP_RMDIVI ? !is_finite(imm / sv)
         : op == OP_MSQRT  ? sv < 0.0f
         : op == OP_MLOG   ? sv <= 0.0f
         : op == OP_POWCHK ? !is_finite(sv)
                           : false;
}
// one instruction of a chain on one value (the stages that compute with row scalars)
__device__ __forceinline__ void chain_scalar(uint32_t op, float &sv, float imm) {
  switch (op) {
  case OP_CONST: sv = imm; break;
  case OP_ADDI: sv = sv + imm; break;
  case OP_SUBI: sv = sv - imm; break;
  case OP_MULI: sv = sv * imm; break;
  case OP_DIVI: sv = sv / imm; break;
  case OP_MAXI: sv = nan_max(sv, imm); break;
  case OP_MINI: sv = nan_min(sv, imm); break;
  case OP_RSUBI: sv = imm - sv; break;
  case OP_RDIVI: sv = imm / sv; break;
  case OP_NEG: sv = -sv; break;
  case OP_ABS: sv = __builtin_fabsf(sv); break;
  case OP_SQRT: sv = __builtin_sqrtf(sv); break;
  case OP_RINT: sv = __builtin_rintf(sv); break;
  case OP_EXP: sv = expf(sv); break;
  case OP_LOG: sv = logf(sv); break;
  case OP_TANH: sv = tanh_selects(sv); break;
  case OP_R16: sv = round16(sv); break;
  case OP_SQ: sv = sv * sv; break;
  // numpy.ma's forms, for a value that is stored whatever becomes of its activity:
  // a failed quotient leaves the dividend, the functions their fill values
  case OP_MDIVI: {
    const float q = sv / imm;
    sv = is_finite(q) ? q + 0.0f * sv : 0.0f + sv;
    break;
  }
  case OP_RMDIVI: {
    const float q = imm / sv;
    sv = is_finite(q) ? q + 0.0f * imm : 0.0f + imm;
    break;
  }
  case OP_MSQRT: sv = sv < 0.0f ? 0.0f : __builtin_sqrtf(sv); break;
  case OP_MLOG: sv = sv <= 0.0f ? 1.0f : logf(sv); break;
  default: break;
  }
}

__device__ __forceinline__ float col_fold(uint32_t kind, float a, float b) {
  return kind == COL_SUM ? a + b : kind == COL_MAX ? nan_max(a, b) : nan_min(a, b);
}
} // namespace

// The launch that finishes a sum down the columns without the interpreter: the
// bands of partial[band][column] added up by the kernel above (the bands are its
// rows), then a post program of at most four instructions that change the value
// in place with an immediate or none (the division of a mean, the root of a
// norm), given as kernel arguments, and an fp32 result.  The general kernel
// takes 7.4 us for 64 bands of 8192 columns, most of it dependent loads of
// arguments and instructions one after the other.
struct FoldPost {
  uint32_t n;
  uint32_t op[4];
  float imm[4];
};
extern "C" __global__ __launch_bounds__(1024) void hcamd_cols_fold_f32(
    const float *partial, size_t ld, float *out, uint32_t cols, uint32_t bands, const FoldPost post) {
  cols_sum_f32<false, 16, 4>(partial, ld, cols, bands, bands, [&](f32x4 total, uint32_t col) {
    float v[4] = {total[0], total[1], total[2], total[3]};
    for (uint32_t i = 0; i < post.n; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        chain_scalar(post.op[i], v[e], post.imm[i]);
    *reinterpret_cast<f32x4 *>(out + col) = f32x4{v[0], v[1], v[2], v[3]};
  });
}
namespace {

// NIN: operands the kernel is compiled for; U: turns a wave has in flight (their
// loads are issued together, then the program runs on one after the other:
// fewer operands leave registers for more rows).
template <int NIN, int U>
__device__ __forceinline__ void reduce_cols(const MapArgs &a, const ColArgs &c, const uint32_t n_in) {
  constexpr int kWaves = kThreads / kWave;
  __shared__ float slots[kWaves - 1][kWave][kN + 1];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const uint32_t cols = (uint32_t)a.cols, rows = (uint32_t)a.rows;
  const uint32_t L = c.lanes, R = kWave / L;
  const uint32_t cl = lane & (L - 1), sub = lane / L;
  // column of element e: first + e * step
  const uint32_t chunk = blockIdx.x * L + cl;
  const uint32_t first = c.interleaved ? blockIdx.x * L * kN + cl : chunk * kN;
  const uint32_t step = c.interleaved ? L : 1u;
  const uint32_t n_valid = first >= cols ? 0u
                           : (cols - first + step - 1) / step < (uint32_t)kN
                               ? (cols - first + step - 1) / step
                               : (uint32_t)kN;
  const uint32_t row_begin = blockIdx.y * c.band;
  const uint32_t row_end = row_begin + c.band < rows ? row_begin + c.band : rows;
  // -0 is the identity of IEEE addition (0 would turn a column of -0 into +0)
  const float identity =
      c.kind == COL_SUM ? -0.0f : c.kind == COL_MAX ? -__builtin_inff() : __builtin_inff();
  float acc[kN];
#pragma unroll
  for (int e = 0; e < kN; ++e)
    acc[e] = identity;
  // 16-byte accesses: consecutive columns and a wave of whole chunks
  const bool vec = !c.interleaved && __builtin_amdgcn_ballot_w64(n_valid != (uint32_t)kN) == 0;
  // All operands fp32: a lane's eight columns are two runs of four, 4 L columns
  // apart, so that the L lanes of a row read 16 L consecutive bytes with each of
  // their two accesses (whole cache lines; eight consecutive columns per lane
  // make every access touch twice the lines and use half of each).
  const bool split = vec && (a.f16_mask & ((1u << n_in) - 1u)) == 0;
  const uint32_t run_a = blockIdx.x * L * kN + 4 * cl, run_b = run_a + 4 * L;
  Raw raw;
  Stack r;
  // the rows of the turn that starts at row0, requested (rows past the end: not)
  auto request = [&](uint32_t row0, u32x4 (&staged)[NIN][U][2]) {
#pragma unroll
    for (int i = 0; i < NIN; ++i)
      if (i < (int)n_in) {
        const bool f16 = (a.f16_mask >> i) & 1;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t row = row0 + u * kWaves * R + sub;
          if (row < row_end) {
            const char *base =
                static_cast<const char *>(a.in[i]) + (size_t)row * a.ld[i] * (f16 ? 2 : 4);
            if (split) {
              const u32x4 *q = reinterpret_cast<const u32x4 *>(base) + run_a / 4;
              staged[i][u][0] = ldg<true>(q);
              staged[i][u][1] = ldg<true>(q + L);
            } else if (vec) {
              const u32x4 *q = reinterpret_cast<const u32x4 *>(base) + (f16 ? chunk : 2 * chunk);
              staged[i][u][0] = ldg<true>(q);
              if (!f16)
                staged[i][u][1] = ldg<true>(q + 1);
            } else {
              uint32_t v[kN];
#pragma unroll
              for (int e = 0; e < kN; ++e) {
                const uint32_t at = (uint32_t)e < n_valid ? first + e * step : 0u;
                v[e] = f16 ? (uint32_t) reinterpret_cast<const uint16_t *>(base)[at]
                           : reinterpret_cast<const uint32_t *>(base)[at];
              }
              if (f16) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  staged[i][u][0][e] = v[2 * e] | (v[2 * e + 1] << 16);
              } else {
#pragma unroll
                for (int e = 0; e < kN; ++e)
                  staged[i][u][e / 4][e % 4] = v[e];
              }
            }
          }
        }
      }
  };
#pragma nounroll
  for (uint32_t row0 = row_begin + wave * R; row0 < row_end; row0 += kWaves * R * U) {
    u32x4 staged[NIN][U][2];
    request(row0, staged);
#pragma nounroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < NIN; ++i) {
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          raw.w[i][w] = staged[i][0][w];
#pragma unroll
          for (int k = 0; k + 1 < U; ++k)
            staged[i][k][w] = staged[i][k + 1][w];
        }
      }
      run_program(a, raw, a.f16_mask, r);
      if (row0 + u * kWaves * R + sub < row_end) {
        if (c.masked) { // uniform
          // (numpy.ma adds up a sum's deactivated elements as +0: a column of them is +0, not the identity -0)
#pragma unroll
          for (int e = 0; e < kN; ++e)
            acc[e] = ((r.bad >> e) & 1u) ? (c.kind == COL_SUM ? acc[e] + 0.0f : acc[e])
                                         : col_fold(c.kind, acc[e], r.st[0][e]);
        } else {
#pragma unroll
          for (int e = 0; e < kN; ++e)
            acc[e] = col_fold(c.kind, acc[e], r.st[0][e]);
        }
      }
    }
  }
  // lanes that share columns (the rows of one turn), then the waves in order
  for (uint32_t s = L; s < (uint32_t)kWave; s <<= 1) {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      acc[e] = col_fold(c.kind, acc[e], __shfl_xor(acc[e], (int)s, kWave));
  }
  if (wave != 0) {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      slots[wave - 1][lane][e] = acc[e];
  }
  __syncthreads();
  if (wave != 0 || sub != 0)
    return;
#pragma unroll
  for (int w = 0; w < kWaves - 1; ++w)
#pragma unroll
    for (int e = 0; e < kN; ++e)
      acc[e] = col_fold(c.kind, acc[e], slots[w][lane][e]);
  if (gridDim.y > 1) {
    float *dst = c.partial + (size_t)blockIdx.y * c.cols_pad;
    if (!c.interleaved && n_valid) { // cols_pad covers whole chunks
      f32x4 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = acc[e];
        hi[e] = acc[4 + e];
      }
      *reinterpret_cast<f32x4 *>(dst + (split ? run_a : first)) = lo;
      *reinterpret_cast<f32x4 *>(dst + (split ? run_b : first + 4)) = hi;
    } else {
#pragma unroll
      for (int e = 0; e < kN; ++e)
        if ((uint32_t)e < n_valid)
          dst[first + e * step] = acc[e];
    }
    return;
  }
  if (c.fill_empty) { // uniform
#pragma unroll
    for (int e = 0; e < kN; ++e)
      acc[e] = acc[e] == identity ? 1e20f : acc[e];
  }
  if (c.n_post) {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      raw.w[0][e / 4][e % 4] = __builtin_bit_cast(uint32_t, acc[e]);
    run_post(c, raw, r);
  } else {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      r.st[0][e] = acc[e];
  }
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  if (split) {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      store_elem(a.out, out_f16, (size_t)(e < 4 ? run_a + e : run_b + e - 4), r.st[0][e]);
  } else if (c.out_vec && !c.interleaved && n_valid == (uint32_t)kN) {
    store_chunk(a.out, out_f16, chunk, r.st[0]);
  } else {
#pragma unroll
    for (int e = 0; e < kN; ++e)
      if ((uint32_t)e < n_valid)
        store_elem(a.out, out_f16, (size_t)first + e * step, r.st[0][e]);
  }
}
} // namespace

// Four waves per SIMD: the eight running values per lane on top of the
// interpreter's registers spill at five.
#define HCAMD_REDUCE_COLS(NAME, NIN, U)                                        \
  extern "C" __global__ __launch_bounds__(256) __attribute__((                 \
      amdgpu_waves_per_eu(4, 4))) void                                         \
  NAME(const MapArgs a, const ColArgs c, const uint32_t n_in) {                \
    reduce_cols<NIN, U>(a, c, n_in);                                           \
  }
HCAMD_REDUCE_COLS(hcamd_map_reduce_cols_n4u1, 4, 1)
HCAMD_REDUCE_COLS(hcamd_map_reduce_cols_n2u2, 2, 2)
HCAMD_REDUCE_COLS(hcamd_map_reduce_cols_n1u4, 1, 4)

// ---- row programs ---------------------------------------------------------------
// Bodies that mix elementwise arithmetic with reductions along the rows of a
// tile (normalisations, softmax-like expressions, row sums): a list of stages,
// each a postfix program of the interpreter above, run row by row.
//
//   SUM / MAX / MIN  the program's value at every element of the row is folded
//                    into row scalar `dst`
//   SCALAR           the program reads row scalars only; its value becomes row
//                    scalar `dst`
//   STORE            the program's value at every element is stored to the
//                    output tile
//   STORE_COL        as SCALAR, stored to out[row * ldo] (dst 1: unless the row's result is deactivated)
//
// A program reaches row scalars through the RED opcodes, which are rewritten on
// the fly into the immediate forms of the interpreter with the scalar as the
// immediate, so the interpreter itself does not know about them.  Column
// operands (one value per row) are row scalars that are loaded instead of
// computed.  Row scalars are wave-uniform: their home is a few LDS cells per
// wave, and a stage starts by reading them into one vector register, scalar k
// in lane k, from which a readlane fetches the one an instruction names.
//
// LPR lanes share a row (256: one row per workgroup; 64: one row per wave,
// four rows per workgroup).  A lane's chunks of the row are LPR chunks apart.
// Every stage loads the operands it uses again; a row that a workgroup has just
// read is still in L2, so only the first read goes to HBM.  (Keeping the rows
// in LDS between the stages, each lane its own chunks, measured 10 to 70 %
// slower: the kernel is bound by the interpreter's instruction issue, not by
// the reads, and the LDS footprint costs occupancy.)  Reductions add in a fixed
// order for a given shape: results are reproducible from run to run.
namespace {
constexpr int kMaxRed = 16;
constexpr int kMaxStages = 16;
constexpr int kRowProg = 128;
constexpr int kRowN = 8; // elements per lane per run of a stage's program (16: registers cost more than the halved dispatch gains)
enum : uint32_t {
  OP_RED = 45,     // push row scalar `arg`
  OP_ADD_RED = 46, // top = top op row scalar `arg`, in the order of OP_ADD_IN..
  OP_RDIV_RED = 53,
  OP_MDIV_RED = 54,  // top / row scalar and row scalar / top under numpy.ma's rule
  OP_RMDIV_RED = 55, // (`arg` bits 0..3: the scalar, bit 8: fp16)
  OP_RED0 = 56,      // push row scalar `arg` as a value, deactivated or not
  OP_MASQRT = 57,    // numpy.ma.sqrt (scalar stages): not finite or x < 0 deactivates, value x
};
// flags in `arg` of the instructions of scalar stages (beside bit 8, fp16)
constexpr uint32_t kFuncForm = 0x200; // called as a NumPy function: computed on the values, deactivated or not
constexpr uint32_t kSwapped = 0x400;  // commutative operation whose running value is the second operand
constexpr uint32_t kKeepDead = 0x800; // unary operation that leaves a deactivated value as it is (x ** 0.5:
                                      // numpy.ma.power keeps its operand where that is inactive)
enum : uint32_t {
  ST_SUM = 0, ST_MAX = 1, ST_MIN = 2, ST_SCALAR = 3, ST_STORE = 4, ST_STORE_COL = 5,
  ST_COUNT = 6 // the number of active elements of the program's value, as fp32
};

struct Stage {
  uint16_t begin, end; // instructions [begin, end)
  uint8_t kind, dst;
  uint8_t load_mask; // operands this stage reads
  uint8_t masked;    // honour the inactive bits: numpy.ma's forms, or a row scalar read that may be deactivated
  uint16_t red_mask; // row scalars this stage reads that may be deactivated
  uint8_t live_pos;  // scalar stages: the result is active iff this row scalar is positive (0xff: not used)
  uint8_t frozen;    // STORE stages: deactivated elements are stored too, with what numpy.ma leaves in them
};

struct RowArgs {
  const void *in[kMaxIn];
  const void *col[kMaxIn]; // column operands: row scalars 0 .. n_col-1
  void *out;
  size_t ld[kMaxIn]; // row stride in elements (0: the same vector for every row)
  size_t ldo;
  size_t rows, cols;
  uint32_t f16_mask; // bit i: operand i is fp16; bit 8: the output; bit 16+k: column k
  uint32_t vec_mask; // bit i: rows of operand i start on 16-byte boundaries; bit 8: the output
  uint32_t interleaved; // columns are dealt to lanes one by one (then vec_mask is 0)
  uint32_t n_col, n_stages, passes;
  uint32_t hold, hold_last; // chain kernels: the operand that stays in LDS for the row, and the last instruction that reads it
  uint32_t all_f32;         // chain kernels: every operand in use and the output are fp32
  Stage stage[kMaxStages];
  Instr prog[kRowProg];
  // Two launches for programs whose row scalars can be deactivated (a quotient
  // that is not finite, a root or a logarithm outside its domain): the chain
  // kernels, which keep no such books, run every row, store nothing of a row on
  // which an operation on a row scalar failed and say so in deferred[row]; the
  // general kernel then runs the rows marked in only[] (the same array).
  uint8_t *deferred;
  const uint8_t *only;
};

struct NanMaxOp {
  using T = float;
  static __device__ __forceinline__ float identity() { return -INFINITY; }
  static __device__ __forceinline__ float apply(float a, float b) { return nan_max(a, b); }
};
struct NanMinOp {
  using T = float;
  static __device__ __forceinline__ float identity() { return INFINITY; }
  static __device__ __forceinline__ float apply(float a, float b) { return nan_min(a, b); }
};

__device__ __forceinline__ float uniform(float x) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}
// The row scalars come in as one vector register, scalar k in lane k (the same
// in every wave of a row): reading one is a single readlane with the index in
// a scalar register.
__device__ __forceinline__ void run_stage(const RowArgs &a, uint32_t begin, uint32_t end,
                                          const RawT<kRowN> &raw, StackT<kRowN> &r,
                                          uint32_t reds) {
  int sp = 0;
  r.bad = 0;
  Instr next = a.prog[begin & (kRowProg - 1)];
  for (uint32_t pc = begin; pc < end; ++pc) {
    const Instr cur = next;
    next = a.prog[(pc + 1) & (kRowProg - 1)];
    const uint32_t arg = cur.arg;
    // RED forms become the immediate forms with the row scalar as the immediate.
    // The rewritten opcode is hidden from the optimiser behind an empty asm
    // statement: an opcode whose value is known on some path would be threaded
    // into the dispatch below and tear its arms apart.
    uint32_t op = cur.op;
    uint32_t imm_bits = __builtin_bit_cast(uint32_t, cur.imm);
    if (op >= OP_RED && op <= OP_RED0) {
      imm_bits = __builtin_amdgcn_readlane(reds, arg & (kMaxRed - 1));
      op = (op == OP_RED || op == OP_RED0) ? (uint32_t)OP_CONST
           : op >= OP_MDIV_RED             ? op - OP_MDIV_RED + OP_MDIVI
                                           : op - OP_ADD_RED + OP_ADDI;
    }
    asm volatile("" : "+s"(op), "+s"(imm_bits));
    const float imm = __builtin_bit_cast(float, imm_bits);
    // The arms differ only in the stack entries they touch.  The marker
    // comments keep them apart: merged into one arm, every operation would
    // pick its entries with per-element selects, eight times the vector work.
    switch (sp) {
    case 0: asm volatile("; stack depth 0"); sp = step<0>(r, raw, a.f16_mask, op, arg, imm); break;
    case 1: asm volatile("; stack depth 1"); sp = step<1>(r, raw, a.f16_mask, op, arg, imm); break;
    case 2: asm volatile("; stack depth 2"); sp = step<2>(r, raw, a.f16_mask, op, arg, imm); break;
    case 3: asm volatile("; stack depth 3"); sp = step<3>(r, raw, a.f16_mask, op, arg, imm); break;
    default: asm volatile("; stack depth 4"); sp = step<4>(r, raw, a.f16_mask, op, arg, imm); break;
    }
  }
}

// One value as numpy.ma computes with it: the value and whether it is deactivated.
// The tile operators + - * leave their first operand's value in a deactivated
// result, the quotient leaves the dividend's, NumPy functions compute on the
// values regardless (numpy.sqrt and numpy.log put their fill value where the
// domain fails or the argument is deactivated already).
struct MaValue {
  float v;
  bool dead;
};
// `op`: one of the unary opcodes (OP_NEG .. OP_R16, OP_POWCHK, OP_MSQRT, OP_MLOG, OP_MASQRT)
__device__ __forceinline__ bool ma_is_unary(uint32_t op) {
  return (op >= OP_NEG && op <= OP_R16) || op == OP_POWCHK || op == OP_MSQRT || op == OP_MLOG ||
         op == OP_MASQRT;
}
__device__ __forceinline__ MaValue ma_unary(uint32_t op, MaValue x, uint32_t arg) {
  const float v = x.v;
  if ((arg & kKeepDead) && x.dead)
    return x;
  switch (op) {
  case OP_NEG: return {-v, x.dead};
  case OP_ABS: return {__builtin_fabsf(v), x.dead};
  case OP_SQRT: return {__builtin_sqrtf(v), x.dead};
  case OP_RINT: return {__builtin_rintf(v), x.dead};
  case OP_EXP: return {expf(v), x.dead};
  case OP_LOG: return {logf(v), x.dead};
  case OP_TANH: return {tanh_selects(v), x.dead};
  case OP_R16: return {round16(v), x.dead};
  case OP_MSQRT: {
    const bool out = x.dead || v < 0.0f;
    return {out ? 0.0f : __builtin_sqrtf(v), out};
  }
  case OP_MLOG: {
    const bool out = x.dead || v <= 0.0f;
    return {out ? 1.0f : logf(v), out};
  }
  case OP_MASQRT: {
    const float r = __builtin_sqrtf(v);
    const bool out = x.dead || !is_finite(r) || v < 0.0f;
    return {out ? v : r, out};
  }
  default: { // OP_POWCHK
    const bool out = !is_finite(v);
    return {out ? 1e20f : v, x.dead || out};
  }
  }
}
// `base`: OP_ADD .. OP_RDIV, OP_MDIV, OP_RMDIV with `run` the running value (the
// deeper stack entry, or the top of an immediate / operand / row-scalar form) and
// `other` the other operand; `flags`: kFuncForm, kSwapped; `half`: the quotient
// is rounded to fp16 before it is tested.
__device__ __forceinline__ MaValue ma_binary(uint32_t base, uint32_t flags, bool half, MaValue run,
                                             MaValue other) {
  MaValue l = run, r = other; // first and second operand
  const bool reversed = base == OP_RSUB || base == OP_RDIV || base == OP_RMDIV;
  if (reversed || (flags & kSwapped)) {
    l = other;
    r = run;
  }
  const bool gone = l.dead || r.dead;
  if (base == OP_MDIV || base == OP_RMDIV) {
    float q = l.v / r.v;
    if (half)
      q = round16(q);
    const bool good = is_finite(q) && !gone;
    return {good ? q + 0.0f * l.v : 0.0f + l.v, !good};
  }
  float y;
  switch (base) {
  case OP_ADD: y = l.v + r.v; break;
  case OP_SUB:
  case OP_RSUB: y = l.v - r.v; break;
  case OP_MUL: y = l.v * r.v; break;
  case OP_DIV:
  case OP_RDIV: y = l.v / r.v; break;
  case OP_MAX: y = nan_max(l.v, r.v); break;
  default: y = nan_min(l.v, r.v); break;
  }
  const bool keeps_first =
      !(flags & kFuncForm) && (base == OP_ADD || base == OP_SUB || base == OP_RSUB || base == OP_MUL);
  return {gone && keeps_first ? l.v : y, gone};
}
// The plain binary operation behind an immediate, operand or row-scalar form
// (0: `op` is none of them).
__device__ __forceinline__ uint32_t ma_base_of(uint32_t op) {
  if (op >= OP_ADDI && op <= OP_RDIVI) return op - OP_ADDI + OP_ADD;
  if (op >= OP_ADD_IN && op <= OP_RDIV_IN) return op - OP_ADD_IN + OP_ADD;
  if (op >= OP_ADD_RED && op <= OP_RDIV_RED) return op - OP_ADD_RED + OP_ADD;
  if (op == OP_MDIVI || op == OP_MDIV_IN || op == OP_MDIV_RED) return OP_MDIV;
  if (op == OP_RMDIVI || op == OP_RMDIV_IN || op == OP_RMDIV_RED) return OP_RMDIV;
  return 0u;
}

// A stage that computes with row scalars only (SCALAR, STORE_COL), as numpy.ma
// computes on values that may be deactivated: every stack entry is a value and a
// "deactivated" bit.  What a deactivated row scalar holds matters where it is
// stored all the same (a per-row result is a bare numpy.ma array, written in
// full) and where a variance reads a sum whose terms were all inactive.
// Everything here is uniform over the lanes of a row.  `dead`: bit k = row
// scalar k is deactivated.
struct ScalarResult {
  float value;
  bool dead;
};
__device__ __forceinline__ ScalarResult run_scalar_stage(const RowArgs &a, uint32_t begin, uint32_t end,
                                                         const float *cells, uint32_t dead) {
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  uint32_t dbits = 0; // bit i: stack entry i is deactivated
  int sp = 0;
  auto get = [&](int i) {
    return MaValue{i == 0 ? s0 : i == 1 ? s1 : i == 2 ? s2 : s3, ((dbits >> i) & 1u) != 0};
  };
  auto put = [&](int i, MaValue x) {
    s0 = i == 0 ? x.v : s0;
    s1 = i == 1 ? x.v : s1;
    s2 = i == 2 ? x.v : s2;
    s3 = i == 3 ? x.v : s3;
    dbits = (dbits & ~(1u << i)) | (x.dead ? 1u << i : 0u);
  };
#pragma nounroll
  for (uint32_t pc = begin; pc < end; ++pc) {
    const Instr cur = a.prog[pc & (kRowProg - 1)];
    const uint32_t op = cur.op, arg = cur.arg;
    const uint32_t slot = arg & (kMaxRed - 1);
    if (op == OP_CONST) {
      put(sp++, {cur.imm, false});
    } else if (op == OP_RED || op == OP_RED0) {
      put(sp++, {cells[slot], op == OP_RED && ((dead >> slot) & 1u)});
    } else if (ma_is_unary(op)) {
      if (sp >= 1)
        put(sp - 1, ma_unary(op, get(sp - 1), arg));
    } else if ((op >= OP_ADD && op <= OP_RDIV) || op == OP_MDIV || op == OP_RMDIV) {
      if (sp >= 2) { // (any `arg` but the form flags marks an fp16 quotient)
        put(sp - 2, ma_binary(op, arg, (arg & 0x1ffu) != 0, get(sp - 2), get(sp - 1)));
        --sp;
      }
    } else if (const uint32_t base = ma_base_of(op); base != 0 && sp >= 1) {
      const bool red = op >= OP_ADD_RED;
      const MaValue other{red ? cells[slot] : cur.imm, red && ((dead >> slot) & 1u)};
      put(sp - 1, ma_binary(base, arg, (arg & 0x100u) != 0, get(sp - 1), other));
    }
  }
  return ScalarResult{s0, (dbits & 1u) != 0};
}

// A STORE stage that keeps what numpy.ma leaves in deactivated elements (the
// stored value is a bare numpy.ma array, written in full, and a tile operator
// follows an operation that can deactivate): the same rules, element by
// element, for a program that pushes one value and changes it in place.  The
// host sends only such programs here; their instructions carry the form flags.
__device__ __forceinline__ void run_frozen_stage(const RowArgs &a, uint32_t begin, uint32_t end,
                                                 const RawT<kRowN> &raw, StackT<kRowN> &r,
                                                 const float *cells, uint32_t dead) {
  float(&v)[kRowN] = r.st[0];
  uint32_t bad = 0;
  auto operand = [&](uint32_t i, float *t) {
    switch (i & 3u) {
    case 0: unpack(raw, 0, a.f16_mask & 1, t); break;
    case 1: unpack(raw, 1, a.f16_mask & 2, t); break;
    case 2: unpack(raw, 2, a.f16_mask & 4, t); break;
    default: unpack(raw, 3, a.f16_mask & 8, t); break;
    }
  };
#pragma nounroll
  for (uint32_t pc = begin; pc < end; ++pc) {
    const Instr cur = a.prog[pc & (kRowProg - 1)];
    const uint32_t op = cur.op, arg = cur.arg;
    const uint32_t slot = arg & (kMaxRed - 1);
    if (op == OP_IN) {
      operand(arg, v);
    } else if (op == OP_CONST || op == OP_RED || op == OP_RED0) {
      const float x = op == OP_CONST ? cur.imm : cells[slot];
#pragma unroll
      for (int e = 0; e < kRowN; ++e)
        v[e] = x;
      bad = (op == OP_RED && ((dead >> slot) & 1u)) ? ~0u : 0u;
    } else if (op == OP_CLEAR) {
      bad = 0;
    } else if (ma_is_unary(op)) {
#pragma unroll
      for (int e = 0; e < kRowN; ++e) {
        const MaValue y = ma_unary(op, {v[e], ((bad >> e) & 1u) != 0}, arg);
        v[e] = y.v;
        bad = (bad & ~(1u << e)) | (y.dead ? 1u << e : 0u);
      }
    } else if (const uint32_t base = ma_base_of(op); base != 0) {
      float t[kRowN];
      bool other_dead = false;
      if ((op >= OP_ADD_IN && op <= OP_RDIV_IN) || op == OP_MDIV_IN || op == OP_RMDIV_IN) {
        operand(arg, t);
      } else {
        const bool red = op >= OP_ADD_RED;
        other_dead = red && ((dead >> slot) & 1u);
#pragma unroll
        for (int e = 0; e < kRowN; ++e)
          t[e] = red ? cells[slot] : cur.imm;
      }
#pragma unroll
      for (int e = 0; e < kRowN; ++e) {
        const MaValue y = ma_binary(base, arg, (arg & 0x100u) != 0, {v[e], ((bad >> e) & 1u) != 0},
                                    {t[e], other_dead});
        v[e] = y.v;
        bad = (bad & ~(1u << e)) | (y.dead ? 1u << e : 0u);
      }
    }
  }
  r.bad = 0; // every element is stored
}

// Where a lane stands in its row during pass p.
// Element e of the lane's chunk is column first + e * step of the row, inside
// the row for e < n_valid.  Two assignments of columns to lanes exist.  With
// step 1 a lane holds kRowN consecutive columns: the form for rows that start
// on 16-byte boundaries in every operand, moved with 16-byte accesses.  With
// step = the number of lanes that share the row, the lanes interleave, so that
// the element-wise accesses that unaligned rows need are coalesced (a wave
// reads consecutive elements); a program does not care which columns share a
// lane as long as all operands and the output agree.
struct Place {
  uint32_t first, step;
  uint32_t n_valid;
};

// The chunk `at` of operand i's row, as loaded.  A wave whose lanes all stand
// on whole chunks of 16-byte aligned rows (or on nothing) uses 16-byte loads.
// Any other wave reads element by element in all its lanes, every load issued
// (from the row's first element where the column is past the end) and zeroed
// afterwards.  The choice is per wave, not per lane: a load in a branch that
// only some lanes take would be waited for on the spot, together with every
// load issued before it.
__device__ __forceinline__ void load_chunk(const RowArgs &a, int i, const char *base, Place at,
                                           u32x4 (&w)[kRowN / 4]) {
  const bool f16 = (a.f16_mask >> i) & 1;
  const bool vec = (a.vec_mask >> i) & 1; // implies at least one whole chunk per row
  const bool partial = at.n_valid != kRowN && at.n_valid != 0; // never with step != 1: no vec bits
#pragma unroll
  for (int j = 0; j < kRowN / 4; ++j) // never a value left over from another chunk
    w[j] = u32x4{0u, 0u, 0u, 0u};
  if (vec && __builtin_amdgcn_ballot_w64(partial) == 0) {
    if (f16) {
      const u32x4 *q = reinterpret_cast<const u32x4 *>(base) + at.first / 8;
#pragma unroll
      for (int j = 0; j < kRowN / 8; ++j)
        w[j] = ldg<false>(q + j);
    } else {
      const u32x4 *q = reinterpret_cast<const u32x4 *>(base) + at.first / 4;
#pragma unroll
      for (int j = 0; j < kRowN / 4; ++j)
        w[j] = ldg<false>(q + j);
    }
  } else {
    // The empty asm statement keeps the index arithmetic of this seldom-taken
    // path in this path (the compiler would hoist it into every pass).
    uint32_t first = at.first;
    asm volatile("" : "+v"(first));
    uint32_t v[kRowN];
    if (f16) {
#pragma unroll
      for (int e = 0; e < kRowN; ++e)
        v[e] = reinterpret_cast<const uint16_t *>(
            base)[(uint32_t)e < at.n_valid ? first + e * at.step : 0u];
    } else {
#pragma unroll
      for (int e = 0; e < kRowN; ++e)
        v[e] = reinterpret_cast<const uint32_t *>(
            base)[(uint32_t)e < at.n_valid ? first + e * at.step : 0u];
    }
#pragma unroll
    for (int e = 0; e < kRowN; ++e)
      v[e] = (uint32_t)e < at.n_valid ? v[e] : 0u;
    if (f16) {
#pragma unroll
      for (int j = 0; j < kRowN / 8; ++j)
        w[j] = u32x4{v[8 * j] | (v[8 * j + 1] << 16), v[8 * j + 2] | (v[8 * j + 3] << 16),
                     v[8 * j + 4] | (v[8 * j + 5] << 16), v[8 * j + 6] | (v[8 * j + 7] << 16)};
    } else {
#pragma unroll
      for (int j = 0; j < kRowN / 4; ++j)
        w[j] = u32x4{v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
    }
  }
}

template <int LPR> __device__ __forceinline__ void row_program(const RowArgs &a) {
  __shared__ float slots[2][kThreads / kWave];
  __shared__ float red_cells[kThreads / kWave][kMaxRed];
  const uint32_t t = threadIdx.x, lane = t % LPR;
  float *cells = red_cells[t / kWave];
  const size_t row_at = (size_t)blockIdx.x * (kThreads / LPR) + t / LPR;
  const bool row_live = row_at < a.rows && (!a.only || a.only[row_at]);
  if (LPR == kThreads && a.only && !row_live)
    return; // (one row to a workgroup: the branch is uniform)
  const size_t row = row_live ? row_at : 0; // idle lanes compute on row 0 and store nothing
  const uint32_t whole = (uint32_t)(a.cols / kRowN), rem = (uint32_t)(a.cols % kRowN);
  const uint32_t per_row = whole + (rem ? 1u : 0u);
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  const uint32_t cols = (uint32_t)a.cols;
  auto place = [&](uint32_t p) {
    if (a.interleaved) {
      const uint32_t first = p * (LPR * kRowN) + lane;
      const bool live = row_live && first < cols;
      const uint32_t n = (cols - first + LPR - 1) / LPR;
      return Place{live ? first : 0u, (uint32_t)LPR,
                   !live ? 0u : n < (uint32_t)kRowN ? n : (uint32_t)kRowN};
    }
    const uint32_t c = p * LPR + lane;
    const bool live = row_live && c < per_row;
    return Place{live ? c * kRowN : 0u, 1u, !live ? 0u : c == whole ? rem : (uint32_t)kRowN};
  };
  if (t % kWave < kMaxRed)
    cells[t % kWave] = 0.0f;
#pragma unroll
  for (int k = 0; k < kMaxIn; ++k)
    if (k < (int)a.n_col)
      cells[k] = uniform(load_elem(a.col[k], (a.f16_mask >> (16 + k)) & 1, row));

  // where this lane's row starts in every operand and in the output
  const char *bases[kMaxIn];
#pragma unroll
  for (int i = 0; i < kMaxIn; ++i)
    bases[i] = static_cast<const char *>(a.in[i]) +
               row * a.ld[i] * (((a.f16_mask >> i) & 1) ? 2 : 4);
  char *const orow = static_cast<char *>(a.out) + row * a.ldo * (out_f16 ? 2 : 4);

  uint32_t parity = 0;
  uint32_t dead = 0; // bit k: row scalar k is deactivated (the same in every lane of a row)
#pragma nounroll
  for (uint32_t s = 0; s < a.n_stages; ++s) {
    const Stage st = a.stage[s];
    const uint32_t kind = st.kind;
    if (kind == ST_SCALAR || kind == ST_STORE_COL) {
      ScalarResult res = run_scalar_stage(a, st.begin, st.end, cells, dead);
      if (st.live_pos != 0xff)
        res.dead = !(cells[st.live_pos & (kMaxRed - 1)] > 0.0f);
      if (kind == ST_SCALAR) {
        const uint32_t bit = 1u << (st.dst & (kMaxRed - 1));
        cells[st.dst & (kMaxRed - 1)] = uniform(res.value);
        dead = res.dead ? dead | bit : dead & ~bit;
      } else if (row_live && lane == 0 && !(st.dst && res.dead)) {
        // (dst 1: the value is a tile, whose deactivated rows are not stored)
        store_elem(a.out, out_f16, row * a.ldo, res.value);
      }
      continue;
    }
    const uint32_t n_pass = a.passes;
    // every element of a stage that reads a deactivated row scalar is inactive
    const bool row_gone = (dead & st.red_mask) != 0;
    // the row scalars, scalar k in lane k
    const uint32_t reds = __builtin_bit_cast(uint32_t, cells[t & (kMaxRed - 1)]);
    float acc = kind == ST_MAX ? -INFINITY : kind == ST_MIN ? INFINITY : 0.0f;
    float taken = 0.0f; // active elements folded (stages that honour the inactive bits)
    StackT<kRowN> r;
#pragma nounroll
    for (uint32_t p = 0; p < n_pass; ++p) {
      const Place at = place(p);
      RawT<kRowN> raw;
#pragma unroll
      for (int i = 0; i < kMaxIn; ++i) {
        if ((st.load_mask >> i) & 1) {
          load_chunk(a, i, bases[i], at, raw.w[i]);
        }
      }
      if (st.frozen)
        run_frozen_stage(a, st.begin, st.end, raw, r, cells, dead);
      else
        run_stage(a, st.begin, st.end, raw, r, reds);
      // a wave whose lanes all hold whole chunks folds them without masks
      const bool all_whole = __builtin_amdgcn_ballot_w64(at.n_valid != kRowN) == 0;
      if (st.masked) {
        // a stage with numpy.ma's forms, or one that reads a row scalar that may
        // be deactivated (uniform: the host marks it): elements that a division
        // or a domain function deactivated are neither stored nor folded
        if (row_gone && !st.frozen)
          r.bad = ~0u;
        const bool whole_chunk = kind == ST_STORE && ((a.vec_mask >> 8) & 1) && at.n_valid == kRowN &&
                                 r.bad == 0;
        if (whole_chunk) {
#pragma unroll
          for (int j = 0; j < kRowN / 8; ++j)
            store_chunk(orow, out_f16, at.first / 8 + j, r.st[0] + 8 * j);
        }
#pragma unroll
        for (int e = 0; e < kRowN; ++e) {
          const bool take = (uint32_t)e < at.n_valid && !((r.bad >> e) & 1u);
          if (kind == ST_STORE) {
            if (take && !whole_chunk)
              store_elem(orow, out_f16, at.first + e * at.step, r.st[0][e]);
          } else if (kind == ST_SUM) {
            acc += take ? r.st[0][e] : 0.0f;
          } else if (kind == ST_MAX) {
            acc = take ? nan_max(acc, r.st[0][e]) : acc;
          } else if (kind == ST_MIN) {
            acc = take ? nan_min(acc, r.st[0][e]) : acc;
          }
          taken += take ? 1.0f : 0.0f;
        }
      } else if (kind == ST_STORE) {
        if (((a.vec_mask >> 8) & 1) && at.n_valid == kRowN) {
#pragma unroll
          for (int j = 0; j < kRowN / 8; ++j)
            store_chunk(orow, out_f16, at.first / 8 + j, r.st[0] + 8 * j);
        } else {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            if ((uint32_t)e < at.n_valid)
              store_elem(orow, out_f16, at.first + e * at.step, r.st[0][e]);
        }
      } else if (kind == ST_SUM) {
        if (all_whole) {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc += r.st[0][e];
        } else {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc += (uint32_t)e < at.n_valid ? r.st[0][e] : 0.0f;
        }
      } else if (kind == ST_MAX) {
        if (all_whole) {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc = nan_max(acc, r.st[0][e]);
        } else {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc = (uint32_t)e < at.n_valid ? nan_max(acc, r.st[0][e]) : acc;
        }
      } else if (kind == ST_MIN) {
        if (all_whole) {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc = nan_min(acc, r.st[0][e]);
        } else {
#pragma unroll
          for (int e = 0; e < kRowN; ++e)
            acc = (uint32_t)e < at.n_valid ? nan_min(acc, r.st[0][e]) : acc;
        }
      } else if (kind == ST_COUNT) {
        taken += (float)at.n_valid; // nothing can be inactive but what lies past the row's end
      }
    }
    if (kind <= ST_MIN || kind == ST_COUNT) {
      constexpr int W = LPR / kWave;
      float total;
      if (kind == ST_MAX)
        total = group_reduce<NanMaxOp, W>(acc, slots[parity]);
      else if (kind == ST_MIN)
        total = group_reduce<NanMinOp, W>(acc, slots[parity]);
      else
        total = group_reduce<SumOp, W>(kind == ST_COUNT ? taken : acc, slots[parity]);
      parity ^= 1;
      const uint32_t bit = 1u << (st.dst & (kMaxRed - 1));
      if (st.masked && kind != ST_COUNT) {
        // a fold over no active element at all is deactivated, and holds what
        // numpy.ma leaves there: 0 for a sum, its fill value for a maximum or minimum
        const bool none = group_reduce<SumOp, W>(taken, slots[parity]) == 0.0f;
        parity ^= 1;
        total = none ? (kind == ST_SUM ? 0.0f : 1e20f) : total;
        dead = none ? dead | bit : dead & ~bit;
      } else {
        dead &= ~bit;
      }
      cells[st.dst & (kMaxRed - 1)] = total;
    }
  }
}
} // namespace

extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(4, 4))) void hcamd_row_program_w256(const RowArgs a) {
  row_program<256>(a);
}
extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(4, 4))) void hcamd_row_program_w64(const RowArgs a) {
  row_program<64>(a);
}

// ---- row programs whose stages are chains ------------------------------------------
// Most bodies with row reductions compile to stages that never hold two values
// at once: an operand, then operations that change it in place (`in sub_red exp`,
// `in sub_red mdiv_red mul_in add_in`).  For those the evaluation stack is one
// value per element, and a lane can afford all of its row at once: P chunks of
// eight (P = 1, 2, 4; rows of at most P * LPR chunks on LPR = 64 ... 1024 lanes),
// so that one dispatch of an instruction works on 8 P elements instead of 8 and
// the dispatch, which is what bounds the general kernel above, is paid a P-th as
// often.  The operand most instructions read (`hold`) is fetched once per row and
// lives in LDS, each lane its own words (so nothing has to be synchronised),
// written there by the loads themselves (buffer_load ... lds), which is also how
// the next row arrives while the last stage still runs: a workgroup takes rows
// in turns, and requests the next one as soon as this one has been read for the
// last time.  Every other operand is fetched by the instruction that names it,
// two chunks at a time.  That leaves the registers to the running values.  The
// host decides (hcamdLaunchRowProgram): every stage a chain, whole chunks only
// (columns a multiple of 8, 16-byte aligned rows), at most 4096 chunks; `x x
// mul` with equal halves arrives as `x sq`.  Everything else is as above: the
// same stages, row scalars, numpy.ma forms and fixed order of additions (lane
// order differs from the general kernel's, so sums agree with it to rounding,
// not bit for bit).
namespace {
typedef __attribute__((address_space(3))) void *row_lds_ptr;

template <int LPR, int P> __device__ __forceinline__ void row_chain(const RowArgs &a) {
  constexpr int NE = 8 * P;
  constexpr int CH = P < 2 ? P : 2; // chunks of another operand fetched at a time
  constexpr int T = LPR < kThreads ? kThreads : LPR; // threads of a workgroup
  constexpr uint32_t R = T / LPR;                     // rows per workgroup and turn
  __shared__ float slots[2][T / kWave];
  __shared__ float red_cells[T / kWave][kMaxRed];
  __shared__ __attribute__((aligned(1024))) u32x4 row_words[P][2][T];
  const uint32_t t = threadIdx.x, lane = t % LPR;
  float *cells = red_cells[t / kWave];
  const uint32_t per_row = (uint32_t)(a.cols / 8);
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  uint32_t parity = 0;
  const size_t turns = (a.rows + R - 1) / R;
  // (`ln`: the lane's number in its row, handed in through an empty asm statement
  // where addresses are made: computed from `lane` itself they are loop
  // invariants, and a dozen hoisted address registers spill)
  auto chunk_at = [&](int p, uint32_t ln) {
    const uint32_t c = (uint32_t)p * LPR + ln;
    return c < per_row ? c : 0u;
  };
  // Everything fp32 (the operands in use and the output; the host says): where
  // all 64 chunks of a wave exist, a lane's eight elements are two runs of four,
  // 256 elements apart, so that each of its two 16-byte accesses is one of 64
  // consecutive ones (whole cache lines; eight consecutive elements per lane
  // make every access touch 2 KiB of lines and use half of each).  `split(p)`
  // is the same for every operand, the output and every stage, which is all
  // that element-wise work and reductions along the row need.
  const bool all_f32 = a.all_f32 != 0;
  auto split = [&](int p) {
    return all_f32 && (uint32_t)p * LPR + (lane & ~(uint32_t)(kWave - 1)) + kWave <= per_row;
  };
  // the two 16-byte words of chunk c, in units of 16 bytes from the row's start
  auto word_at = [&](uint32_t c, bool sp, int j) {
    return sp ? 2 * (c & ~(uint32_t)(kWave - 1)) + (c & (kWave - 1)) + (uint32_t)j * kWave : 2 * c + (uint32_t)j;
  };
  auto row_of = [&](size_t turn) { // idle waves compute on row 0 and store nothing
    const size_t r = turn * R + t / LPR;
    return r < a.rows ? r : (size_t)0;
  };
  // operand i's chunks p0 .. p0 + CH - 1 of row r, into registers
  auto request = [&](uint32_t i, size_t r, int p0, u32x4 (&w)[CH][2]) {
    const void *in = a.in[0];
    size_t ld = a.ld[0];
#pragma unroll
    for (int k = 1; k < kMaxIn; ++k) {
      in = i == (uint32_t)k ? a.in[k] : in;
      ld = i == (uint32_t)k ? a.ld[k] : ld;
    }
    const bool f16 = (a.f16_mask >> i) & 1;
    const char *b = static_cast<const char *>(in) + r * ld * (f16 ? 2 : 4);
    uint32_t ln = lane;
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int p = 0; p < CH; ++p) {
      if (f16) {
        w[p][0] = ldg<false>(reinterpret_cast<const u32x4 *>(b) + chunk_at(p0 + p, ln));
        w[p][1] = u32x4{0u, 0u, 0u, 0u};
      } else {
        const uint32_t c = chunk_at(p0 + p, ln);
        const bool sp = split(p0 + p);
        w[p][0] = ldg<false>(reinterpret_cast<const u32x4 *>(b) + word_at(c, sp, 0));
        w[p][1] = ldg<false>(reinterpret_cast<const u32x4 *>(b) + word_at(c, sp, 1));
      }
    }
  };
  // The held operand's row r, from memory straight into this wave's words of
  // row_words.  A wave belongs to one row (LPR >= 64), so the row's address is
  // wave-uniform: it goes into the buffer descriptor, the lane's part into the
  // 32-bit offset (a row is shorter than 2^31 bytes: the host has checked).
  const uint32_t hold = a.hold & (kMaxIn - 1);
  const bool hold_f16 = (a.f16_mask >> hold) & 1;
  const void *hold_in = a.in[0];
  size_t hold_ld = a.ld[0];
#pragma unroll
  for (int k = 1; k < kMaxIn; ++k) {
    hold_in = hold == (uint32_t)k ? a.in[k] : hold_in;
    hold_ld = hold == (uint32_t)k ? a.ld[k] : hold_ld;
  }
  auto fetch_row = [&](size_t r) {
    const uint64_t at = reinterpret_cast<uint64_t>(hold_in) + r * hold_ld * (hold_f16 ? 2 : 4);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)at);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(at >> 32));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<void *>(((uint64_t)hi << 32) | lo), 0, (int)(a.cols * (hold_f16 ? 2 : 4)),
        0x00020000);
    const uint32_t wave_first = __builtin_amdgcn_readfirstlane(t & ~(uint32_t)(kWave - 1));
    uint32_t ln = lane;
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const uint32_t c = chunk_at(p, ln);
      if (hold_f16) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (row_lds_ptr)&row_words[p][0][wave_first], 16,
                                                 (int)(c * 16u), 0, 0, 0);
      } else {
        const bool sp = split(p);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (row_lds_ptr)&row_words[p][0][wave_first], 16,
                                                 (int)(word_at(c, sp, 0) * 16u), 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (row_lds_ptr)&row_words[p][1][wave_first], 16,
                                                 (int)(word_at(c, sp, 1) * 16u), 0, 0, 0);
      }
    }
  };
  fetch_row(row_of(blockIdx.x));
#pragma nounroll
  for (size_t turn = blockIdx.x; turn < turns; turn += gridDim.x) {
  const size_t row_at = turn * R + t / LPR;
  const bool row_live = row_at < a.rows;
  const size_t row = row_of(turn);
  uint32_t live = 0; // bit p: chunk p of this lane exists
#pragma unroll
  for (int p = 0; p < P; ++p)
    live |= (row_live && (uint32_t)p * LPR + lane < per_row) ? 1u << p : 0u;
  bool died = false; // an operation on a row scalar of this row failed (the same in every lane of the row)
  if (t % kWave < kMaxRed)
    cells[t % kWave] = 0.0f;
#pragma unroll
  for (int k = 0; k < kMaxIn; ++k)
    if (k < (int)a.n_col)
      cells[k] = uniform(load_elem(a.col[k], (a.f16_mask >> (16 + k)) & 1, row));
  char *const orow = static_cast<char *>(a.out) + row * a.ldo * (out_f16 ? 2 : 4);
  // the row requested by the turn before (or above) has to be there
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

#pragma nounroll
  for (uint32_t s = 0; s < a.n_stages; ++s) {
    const Stage st = a.stage[s];
    const uint32_t kind = st.kind;
    const uint32_t reds = __builtin_bit_cast(uint32_t, cells[t & (kMaxRed - 1)]);
    auto decode = [&](Instr cur, uint32_t &op, float &imm) {
      op = cur.op;
      uint32_t imm_bits = __builtin_bit_cast(uint32_t, cur.imm);
      if (op >= OP_RED && op != OP_SQ) {
        imm_bits = __builtin_amdgcn_readlane(reds, cur.arg & (kMaxRed - 1));
        op = op == OP_RED        ? (uint32_t)OP_CONST
             : op >= OP_MDIV_RED ? op - OP_MDIV_RED + OP_MDIVI
                                 : op - OP_ADD_RED + OP_ADDI;
      }
      asm volatile("" : "+s"(op), "+s"(imm_bits));
      imm = __builtin_bit_cast(float, imm_bits);
    };
    Instr next = a.prog[st.begin & (kRowProg - 1)];
    if (kind == ST_SCALAR || kind == ST_STORE_COL) {
      float sv = 0.0f;
#pragma nounroll
      for (uint32_t pc = st.begin; pc < st.end; ++pc) {
        const Instr cur = next;
        next = a.prog[(pc + 1) & (kRowProg - 1)];
        uint32_t op;
        float imm;
        decode(cur, op, imm);
        died = died || chain_scalar_fails(op, sv, imm);
        chain_scalar(op, sv, imm);
      }
      if (kind == ST_SCALAR)
        cells[st.dst & (kMaxRed - 1)] = uniform(sv);
      else if (row_live && lane == 0 && !(a.deferred && died))
        store_elem(a.out, out_f16, row * a.ldo, sv);
      continue;
    }
    float v[NE];
    uint32_t bad = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e)
      v[e] = 0.0f;
#pragma nounroll
    for (uint32_t pc = st.begin; pc < st.end; ++pc) {
      const Instr cur = next;
      next = a.prog[(pc + 1) & (kRowProg - 1)];
      const uint32_t arg = cur.arg;
      uint32_t op;
      float imm;
      decode(cur, op, imm);
      const bool half = (arg & 0x100u) != 0;
      if (chain_reads(op)) {
        const uint32_t i = arg & (kMaxIn - 1);
        const bool f16 = (a.f16_mask >> i) & 1;
        // CH chunks at a time: their words, then the operation on those elements
        auto part = [&](auto number) {
          constexpr int h = decltype(number)::value;
          u32x4 w[CH][2];
          if (i == hold) {
#pragma unroll
            for (int p = 0; p < CH; ++p)
#pragma unroll
              for (int j = 0; j < 2; ++j)
                w[p][j] = row_words[CH * h + p][j][t];
          } else {
            request(i, row, CH * h, w);
          }
          chain_operand<NE, 8 * CH * h, 8 * CH * (h + 1)>(
              op, v, bad, half, chain_words([&](int p, int j, int c) { return w[p - CH * h][j][c]; }, f16));
        };
        part(std::integral_constant<int, 0>{});
        if constexpr (P > CH)
          part(std::integral_constant<int, 1>{});
        if (i == hold && pc == a.hold_last && turn + gridDim.x < turns) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the words have been read
          fetch_row(row_of(turn + gridDim.x));
        }
      } else {
        chain_plain<NE>(op, v, bad, imm, half);
      }
    }

    if (kind <= ST_MIN) {
      float acc = kind == ST_MAX ? -INFINITY : kind == ST_MIN ? INFINITY : 0.0f;
      if (__builtin_amdgcn_ballot_w64(bad != 0 || live != (1u << P) - 1u) == 0) {
        if (kind == ST_SUM) {
#pragma unroll
          for (int e = 0; e < NE; ++e) acc += v[e];
        } else if (kind == ST_MAX) {
#pragma unroll
          for (int e = 0; e < NE; ++e) acc = nan_max(acc, v[e]);
        } else {
#pragma unroll
          for (int e = 0; e < NE; ++e) acc = nan_min(acc, v[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
          const bool take = ((live >> (e / 8)) & 1u) && !((bad >> e) & 1u);
          if (kind == ST_SUM)
            acc += take ? v[e] : 0.0f;
          else if (kind == ST_MAX)
            acc = take ? nan_max(acc, v[e]) : acc;
          else
            acc = take ? nan_min(acc, v[e]) : acc;
        }
      }
      constexpr int W = LPR / kWave;
      float total;
      float *mine = slots[parity] + (t / LPR) * W;
      if (kind == ST_SUM)
        total = group_reduce<SumOp, W>(acc, mine);
      else if (kind == ST_MAX)
        total = group_reduce<NanMaxOp, W>(acc, mine);
      else
        total = group_reduce<NanMinOp, W>(acc, mine);
      parity ^= 1;
      cells[st.dst & (kMaxRed - 1)] = total;
    } else {
      // (an offset the compiler cannot see through, not the pointer itself: a
      // laundered pointer is no longer known to be global and would store flat)
      uint32_t ln = lane, zero = 0;
      asm volatile("" : "+v"(zero), "+v"(ln));
      char *o = orow + zero;
      const bool skip = a.deferred && died;
#pragma unroll
      for (int p = 0; p < P; ++p)
        if (((live >> p) & 1u) && !skip) {
          const uint32_t c = (uint32_t)p * LPR + ln, none = (bad >> (8 * p)) & 0xffu;
          if (split(p)) { // fp32 output, two runs of four
            float *dst = reinterpret_cast<float *>(o);
            const uint32_t e0 = 4 * word_at(c, true, 0), e1 = 4 * word_at(c, true, 1);
            if (none) {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (!((none >> e) & 1u))
                  dst[(e < 4 ? e0 : e1) + e % 4] = v[8 * p + e];
            } else {
              stg<true>(reinterpret_cast<f32x4 *>(dst + e0),
                        f32x4{v[8 * p], v[8 * p + 1], v[8 * p + 2], v[8 * p + 3]});
              stg<true>(reinterpret_cast<f32x4 *>(dst + e1),
                        f32x4{v[8 * p + 4], v[8 * p + 5], v[8 * p + 6], v[8 * p + 7]});
            }
          } else {
            store_chunk(o, out_f16, c, v + 8 * p, none);
          }
        }
    }
  }
  if (a.deferred && row_live && lane == 0)
    a.deferred[row_at] = died ? 1 : 0;
  } // turns
}
} // namespace

// (one and two chunks per lane leave registers for six waves per SIMD)
#define HCAMD_ROW_CHAIN(LPR, P, T)                                                       \
  extern "C" __global__ __launch_bounds__(T)                                              \
      __attribute__((amdgpu_waves_per_eu(P <= 2 ? 6 : 4, P <= 2 ? 6 : 4)))                \
  void hcamd_row_program_chain_w##LPR##_p##P(const RowArgs a) {                          \
    row_chain<LPR, P>(a);                                                                 \
  }
HCAMD_ROW_CHAIN(64, 1, 256)
HCAMD_ROW_CHAIN(64, 2, 256)
HCAMD_ROW_CHAIN(64, 4, 256)
HCAMD_ROW_CHAIN(128, 4, 256)
HCAMD_ROW_CHAIN(256, 4, 256)
HCAMD_ROW_CHAIN(512, 4, 512)
HCAMD_ROW_CHAIN(1024, 4, 1024)

// ---- the flat map for chains ---------------------------------------------------------
// A program that never holds two values at once (an operand or a constant, then
// operations that change the value in place) on dense arrays: one dispatch of
// the chain interpreter works on sixteen elements of a lane, and there is one
// level of dispatch instead of two (the general interpreter also branches on the
// stack depth), so an interpreted instruction costs a third of the scalar issue
// per element.  A workgroup owns 4096 consecutive elements; a lane's sixteen are
// four runs of four, 1024 elements apart (16-byte accesses to fp32 arrays, 8-byte
// ones to fp16 arrays, whole cache lines per wave either way), or, when every
// array is fp16 (ALLH), two runs of eight, 2048 elements apart (16-byte
// accesses).  The elements past the last whole region go through the general
// interpreter in one more workgroup, the first of the grid: it takes longer than
// the others and would otherwise finish alone after them.
namespace {
template <int NIN, bool ALLH>
__device__ __forceinline__ void map_chain(const MapArgs &a, const uint32_t n_in) {
  constexpr int NE = 16, P = 2;
  const size_t n = a.cols;
  const size_t regions = n / 4096;
  const uint32_t t = threadIdx.x;
  const bool out_f16 = (a.f16_mask >> 8) & 1;
  const uint32_t extra = n % 4096 ? 1u : 0u;
  if (extra && blockIdx.x == 0) {
    Raw raw;
    Stack r;
#pragma nounroll
    for (size_t first = regions * 4096 + (size_t)t * 8; first < n; first += 256 * 8) {
      gather(a, n_in, raw, [&](int, int e, size_t &off) {
        off = first + e;
        return off < n;
      });
      run_program(a, raw, 0, r);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (first + e < n && !((r.bad >> e) & 1u))
          store_elem(a.out, out_f16, first + e, r.st[0][e]);
    }
    return;
  }
  const size_t base = (size_t)(blockIdx.x - extra) * 4096;
  u32x4 w[NIN][P][2];
#pragma unroll
  for (int i = 0; i < NIN; ++i)
    if (i < (int)n_in) {
      if constexpr (ALLH) {
        const u32x4 *q = static_cast<const u32x4 *>(a.in[i]) + base / 8 + t;
#pragma unroll
        for (int p = 0; p < P; ++p)
          w[i][p][0] = ldg<true>(q + p * 256);
      } else if ((a.f16_mask >> i) & 1) {
        const u32x2 *q = static_cast<const u32x2 *>(a.in[i]) + base / 4 + t;
#pragma unroll
        for (int p = 0; p < P; ++p) {
          const u32x2 lo = ldg<true>(q + (2 * p) * 256), hi = ldg<true>(q + (2 * p + 1) * 256);
          w[i][p][0] = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
      } else {
        const u32x4 *q = static_cast<const u32x4 *>(a.in[i]) + base / 4 + t;
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            w[i][p][j] = ldg<true>(q + (2 * p + j) * 256);
      }
    }
  float v[NE];
  uint32_t bad = 0;
#pragma unroll
  for (int e = 0; e < NE; ++e)
    v[e] = 0.0f;
  Instr next = a.prog[0];
#pragma nounroll
  for (uint32_t pc = 0; pc < a.n_instr; ++pc) {
    const Instr cur = next;
    next = a.prog[(pc + 1) & (kMaxProg - 1)];
    const uint32_t op = cur.op, arg = cur.arg;
    const float imm = cur.imm;
    const bool half = (arg & 0x100u) != 0;
    if (chain_reads(op)) {
      auto use = [&](auto number) {
        constexpr int I = decltype(number)::value;
        if constexpr (I < NIN)
          chain_operand<NE>(op, v, bad, half,
                            chain_words([&](int p, int j, int c) { return w[I][p][j][c]; },
                                        ALLH || ((a.f16_mask >> I) & 1)));
      };
      switch (arg & 3u) {
      case 0: use(std::integral_constant<int, 0>{}); break;
      case 1: use(std::integral_constant<int, 1>{}); break;
      case 2: use(std::integral_constant<int, 2>{}); break;
      default: use(std::integral_constant<int, 3>{}); break;
      }
    } else {
      chain_plain<NE>(op, v, bad, imm, half);
    }
  }
  if constexpr (ALLH) {
    _Float16 *o = static_cast<_Float16 *>(a.out) + base + (size_t)t * 8;
#pragma unroll
    for (int p = 0; p < P; ++p) {
      if ((bad >> (8 * p)) & 0xffu) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (!((bad >> (8 * p + e)) & 1u))
            o[p * 2048 + e] = (_Float16)v[8 * p + e];
      } else {
        f16x8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          h[e] = (_Float16)v[8 * p + e];
        stg<true>(reinterpret_cast<f16x8 *>(o + p * 2048), h);
      }
    }
  } else {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const size_t at = base + (size_t)g * 1024 + (size_t)t * 4;
      const uint32_t bits = (bad >> (4 * g)) & 0xfu;
      if (bits) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (!((bits >> e) & 1u))
            store_elem(a.out, out_f16, at + e, v[4 * g + e]);
      } else if (out_f16) {
        f16x4 h;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          h[e] = (_Float16)v[4 * g + e];
        stg<true>(reinterpret_cast<f16x4 *>(static_cast<_Float16 *>(a.out) + at), h);
      } else {
        stg<true>(reinterpret_cast<f32x4 *>(static_cast<float *>(a.out) + at),
                  f32x4{v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]});
      }
    }
  }
}
} // namespace
#define HCAMD_MAP_CHAIN(NAME, NIN, ALLH)                                                  \
  extern "C" __global__ __launch_bounds__(256) void NAME(const MapArgs a, const uint32_t n_in) { \
    map_chain<NIN, ALLH>(a, n_in);                                                        \
  }
HCAMD_MAP_CHAIN(hcamd_map_chain_n2, 2, false)
HCAMD_MAP_CHAIN(hcamd_map_chain_n4, 4, false)
HCAMD_MAP_CHAIN(hcamd_map_chain_n2h, 2, true)
HCAMD_MAP_CHAIN(hcamd_map_chain_n4h, 4, true)

// ---- layer normalisation without the interpreter -----------------------------------
// The six-stage row program  mean = sum(x) / n;  var = sum((x - mean) *
// (x - mean)) / n;  s = sqrt(var + eps);  out = (x - mean) / s * w + b  (the
// mean's division and the last one numpy.ma's, as the front-end emits it for a
// body written with mean and var along axis 1) on dense fp32 rows, with the same operations in the same order
// per element as the interpreter performs them (every product and sum rounded
// on its own, a true division, elements whose quotient is not finite left
// unstored); only the order in which a row's terms are added differs.  LPR lanes
// share a row, each with E chunks of four elements LPR chunks apart, the row
// stays in registers between its three passes, the waves of a row meet in LDS.
// The same for the three-stage root-mean-square normalisation  s = sqrt(sum(x *
// x) / n + eps);  out = x / s * w  (hcamd_rms_norm_f32_*: no mean, no bias).
namespace {
// HALF: x and out are fp16 (a chunk is then eight elements, computed in fp32
// and rounded once when stored, which is what the trailing R16 of such a
// program does); w and b stay fp32.
template <int LPR, int E, bool RMS, bool HALF>
__device__ __forceinline__ void layer_norm_rows(const void *__restrict__ x, size_t ld,
                                                const float *__restrict__ w,
                                                const float *__restrict__ b,
                                                void *__restrict__ out, size_t ldo,
                                                uint32_t rows, uint32_t cols, float n, float eps,
                                                uint32_t frozen) {
  constexpr int T = LPR < 256 ? 256 : LPR, RPW = T / LPR, W = LPR / kWave;
  constexpr int C = HALF ? 8 : 4; // elements of a 16-byte chunk
  __shared__ float slots[2][RPW][W];
  const uint32_t lane = threadIdx.x % LPR, sub = threadIdx.x / LPR;
  const uint32_t row = blockIdx.x * RPW + sub, chunks = cols / C;
  const bool live = row < rows;
  const char *xr = static_cast<const char *>(x) + (size_t)row * ld * (HALF ? 2 : 4);
  float v[E][C];
  float acc = -0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const uint32_t c = e * LPR + lane;
#pragma unroll
    for (int k = 0; k < C; ++k)
      v[e][k] = -0.0f;
    if (live && c < chunks) {
      if constexpr (HALF) {
        const f16x8 h = ldg<true>(reinterpret_cast<const f16x8 *>(xr) + c);
#pragma unroll
        for (int k = 0; k < C; ++k)
          v[e][k] = (float)h[k];
      } else {
        const f32x4 f = ldg<true>(reinterpret_cast<const f32x4 *>(xr) + c);
#pragma unroll
        for (int k = 0; k < C; ++k)
          v[e][k] = f[k];
      }
    }
  }
  // (RMS: no mean is taken off; the mean of the squares, no bias)
  float mean = 0.0f;
  if constexpr (!RMS) {
#pragma unroll
    for (int e = 0; e < E; ++e)
#pragma unroll
      for (int k = 0; k < C; ++k)
        acc = __fadd_rn(acc, v[e][k]);
    mean = group_reduce<SumOp, W>(acc, slots[0][sub]) / n;
  }
  acc = -0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const uint32_t c = e * LPR + lane;
    if (live && c < chunks) {
#pragma unroll
      for (int k = 0; k < C; ++k) {
        const float d = RMS ? v[e][k] : __fsub_rn(v[e][k], mean);
        acc = __fadd_rn(acc, __fmul_rn(d, d));
      }
    }
  }
  const float mean_sq = group_reduce<SumOp, W>(acc, slots[1][sub]) / n;
  const float s = __builtin_sqrtf(__fadd_rn(mean_sq, eps));
  // The mean is numpy.ma's quotient: one that is not finite is deactivated, and
  // with it every element computed from it (the variance of such a row is an
  // active 0, but the row's x - mean are all inactive).  `frozen` (the stored
  // expression is a bare numpy.ma array, written in full): deactivated
  // elements are stored too, with what numpy.ma leaves in them, the dividend.
  const bool row_gone = !is_finite(RMS ? mean_sq : mean);
  if (!live || (row_gone && !frozen))
    return;
  // Dividing a whole row by one scalar: s_inv = 1.0 / (double)s is formed once
  // and a quotient is float(double(y) * s_inv).  That is the correctly rounded
  // fp32 quotient whenever it is a normal number: the product is within 2^-52
  // (relative) of y / s, and a quotient of two 24-bit significands that is not
  // itself representable lies at least 2^-49 (relative) from every fp32 value and
  // from every midpoint between two, so both round the same way.  A chunk whose
  // quotients are all normal numbers, or zeros that come from zero dividends
  // (s > 0: the quotient keeps the dividend's sign, and numpy.ma's 0 * dividend
  // added to it changes nothing), has nothing deactivated and takes the short
  // way; any other chunk (a quotient that is not finite, or below the normal
  // range, where fp32 values lie further apart and an exact tie is possible) is
  // divided the long way with numpy.ma's bookkeeping.
  const double s_inv = 1.0 / (double)s;
  const bool s_plain = s > 0.0f && !row_gone;
  char *orow = static_cast<char *>(out) + (size_t)row * ldo * (HALF ? 2 : 4);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const uint32_t c = e * LPR + lane;
    if (c < chunks) {
      float wv[C], bv[C], y[C];
#pragma unroll
      for (int q = 0; q < C / 4; ++q) {
        const f32x4 w4 = reinterpret_cast<const f32x4 *>(w)[c * (C / 4) + q];
        f32x4 b4 = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (!RMS)
          b4 = reinterpret_cast<const f32x4 *>(b)[c * (C / 4) + q];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          wv[4 * q + k] = w4[k];
          bv[4 * q + k] = b4[k];
        }
      }
#pragma unroll
      for (int k = 0; k < C; ++k)
        y[k] = RMS ? v[e][k] : __fsub_rn(v[e][k], mean);
      float quo[C];
      uint32_t lo = 255u, hi = 0u;
#pragma unroll
      for (int k = 0; k < C; ++k) {
        quo[k] = (float)((double)y[k] * s_inv);
        const uint32_t ex = (__builtin_bit_cast(uint32_t, quo[k]) >> 23) & 255u;
        lo = ex < lo ? ex : lo;
        hi = ex > hi ? ex : hi;
      }
      bool plain = s_plain && hi != 255u;
      if (plain && lo == 0u) {
#pragma unroll
        for (int k = 0; k < C; ++k)
          plain = plain && (((__builtin_bit_cast(uint32_t, quo[k]) >> 23) & 255u) != 0u || y[k] == 0.0f);
      }
      if (plain) {
#pragma unroll
        for (int k = 0; k < C; ++k)
          y[k] = RMS ? __fmul_rn(quo[k], wv[k]) : __fadd_rn(__fmul_rn(quo[k], wv[k]), bv[k]);
        if constexpr (HALF) {
          f16x8 h;
#pragma unroll
          for (int k = 0; k < C; ++k)
            h[k] = (_Float16)y[k];
          stg<true>(reinterpret_cast<f16x8 *>(orow) + c, h);
        } else {
          stg<true>(reinterpret_cast<f32x4 *>(orow) + c, f32x4{y[0], y[1], y[2], y[3]});
        }
        continue;
      }
      uint32_t bad = 0;
      float kept[C];
#pragma unroll
      for (int k = 0; k < C; ++k)
        kept[k] = 0.0f + y[k];
      masked_div_scalar<C, false>(bad, y, s, false);
      bad = row_gone ? ~0u : bad;
#pragma unroll
      for (int k = 0; k < C; ++k) {
        y[k] = RMS ? __fmul_rn(y[k], wv[k]) : __fadd_rn(__fmul_rn(y[k], wv[k]), bv[k]);
        y[k] = frozen && ((bad >> k) & 1u) ? kept[k] : y[k];
      }
      bad = frozen ? 0u : bad;
      if constexpr (HALF) {
        _Float16 *oh = reinterpret_cast<_Float16 *>(orow);
        if (bad == 0) {
          f16x8 h;
#pragma unroll
          for (int k = 0; k < C; ++k)
            h[k] = (_Float16)y[k];
          stg<true>(reinterpret_cast<f16x8 *>(orow) + c, h);
        } else {
#pragma unroll
          for (int k = 0; k < C; ++k)
            if (!((bad >> k) & 1u))
              oh[C * c + k] = (_Float16)y[k];
        }
      } else {
        float *of = reinterpret_cast<float *>(orow);
        if (bad == 0) {
          stg<true>(reinterpret_cast<f32x4 *>(orow) + c, f32x4{y[0], y[1], y[2], y[3]});
        } else {
#pragma unroll
          for (int k = 0; k < C; ++k)
            if (!((bad >> k) & 1u))
              of[C * c + k] = y[k];
        }
      }
    }
  }
}
} // namespace
#define HCAMD_NORM_KERNEL(NAME, LPR, E, RMS, HALF)                                        \
  extern "C" __global__ __launch_bounds__(LPR < 256 ? 256 : LPR) void NAME(               \
      const void *x, size_t ld, const float *w, const float *b, void *out, size_t ldo,    \
      uint32_t rows, uint32_t cols, float n, float eps, uint32_t frozen) {                \
    layer_norm_rows<LPR, E, RMS, HALF>(x, ld, w, b, out, ldo, rows, cols, n, eps, frozen); \
  }
#define HCAMD_LAYER_NORM(LPR, E)                                                          \
  HCAMD_NORM_KERNEL(hcamd_layer_norm_f32_w##LPR##_e##E, LPR, E, false, false)             \
  HCAMD_NORM_KERNEL(hcamd_rms_norm_f32_w##LPR##_e##E, LPR, E, true, false)                \
  HCAMD_NORM_KERNEL(hcamd_rms_norm_f16_w##LPR##_e##E, LPR, E, true, true)
// (a row of 8192 on 512 lanes with four chunks each: 48.3 us for 4096 rows; on
// 1024 lanes with two 50.1, on 256 with eight 51.1; with the weights and biases
// requested behind the row instead of where they are used 50.8: the registers
// that hold them cost a workgroup per compute unit)
HCAMD_LAYER_NORM(64, 1)
HCAMD_LAYER_NORM(64, 2)
HCAMD_LAYER_NORM(128, 4)
HCAMD_LAYER_NORM(512, 1)
HCAMD_LAYER_NORM(128, 2)
HCAMD_LAYER_NORM(256, 2)
HCAMD_LAYER_NORM(512, 2)
HCAMD_LAYER_NORM(512, 4)
HCAMD_LAYER_NORM(256, 8)
HCAMD_LAYER_NORM(1024, 2)
HCAMD_LAYER_NORM(1024, 4)
HCAMD_LAYER_NORM(1024, 8)
