// Shared device helpers for the gfx950 kernels: 128-bit vector types, streaming
// loads/stores, and wave64 reductions built on DPP with an LDS cross-wave step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hcamd {

constexpr int kWave = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// 128-bit global access.  NT selects the non-temporal hint: data that is
// touched once should not displace lines in L2 / the memory-side cache.
template <bool NT, class V> __device__ __forceinline__ V ldg(const V *p) {
  if constexpr (NT)
    return __builtin_nontemporal_load(p);
  else
    return *p;
}
template <bool NT, class V> __device__ __forceinline__ void stg(V *p, V v) {
  if constexpr (NT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// ---- tanh, shared by the map kernels ---------------------------------------
// tanh without a branch.  The library routine chooses between its two formulas
// with a per-lane branch, and one per-lane branch inside the interpreter is
// enough for the compiler to linearise an interpreter's whole dispatch around it (every arm
// becomes a block that is stepped over, and all stack registers are copied at
// every join).  Both formulas are evaluated here and one is selected:
// |x| < 1: x + x^3 P(x^2), P fitted to (tanh(t)/t - 1)/t^2 (1.1 ulp);
// otherwise 1 - 2/(exp(2|x|) + 1) (1.1 ulp); the sign is copied from x, and a
// NaN comes out of the second formula as a NaN.
__device__ __forceinline__ float tanh_selects(float x) {
  const float t = __builtin_fabsf(x);
  const float z = t * t;
  float p = -0.00035845194361172616f;
  p = __builtin_fmaf(p, z, 0.0023013644386082888f);
  p = __builtin_fmaf(p, z, -0.007946105673909187f);
  p = __builtin_fmaf(p, z, 0.021486656740307808f);
  p = __builtin_fmaf(p, z, -0.05387980118393898f);
  p = __builtin_fmaf(p, z, 0.13332344591617584f);
  p = __builtin_fmaf(p, z, -0.33333295583724976f);
  const float small = __builtin_fmaf(t * z, p, t);
  const float big = 1.0f - 2.0f / (expf(2.0f * t) + 1.0f);
  return __builtin_copysignf(t < 1.0f ? small : big, x);
}

// ---- wave64 reductions -----------------------------------------------------
// DPP moves data between lanes inside the VALU without touching LDS.  The
// sequence below reduces 16-lane rows with quad permutes and mirrors, then
// folds the four rows with row broadcasts; lane 63 ends up holding the result
// and readlane makes it wave-uniform.
template <int CTRL, int ROW_MASK = 0xF, class T>
__device__ __forceinline__ T dpp(T identity, T v) {
  static_assert(sizeof(T) == 4, "DPP moves 32-bit lanes");
  return __builtin_bit_cast(
      T, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity),
                                     __builtin_bit_cast(int, v), CTRL,
                                     ROW_MASK, 0xF, false));
}

struct MaxOp {
  using T = float;
  static __device__ __forceinline__ float identity() { return -INFINITY; }
  static __device__ __forceinline__ float apply(float a, float b) {
    return fmaxf(a, b);
  }
};
struct SumOp {
  using T = float;
  static __device__ __forceinline__ float identity() { return 0.0f; }
  static __device__ __forceinline__ float apply(float a, float b) {
    return a + b;
  }
};
struct UMaxOp {
  using T = uint32_t;
  static __device__ __forceinline__ uint32_t identity() { return 0u; }
  static __device__ __forceinline__ uint32_t apply(uint32_t a, uint32_t b) {
    return a > b ? a : b;
  }
};

template <class Op>
__device__ __forceinline__ typename Op::T wave_reduce(typename Op::T v) {
  using T = typename Op::T;
  const T id = Op::identity();
  v = Op::apply(v, dpp<0xB1>(id, v));  // quad_perm [1,0,3,2]
  v = Op::apply(v, dpp<0x4E>(id, v));  // quad_perm [2,3,0,1]
  v = Op::apply(v, dpp<0x141>(id, v)); // row_half_mirror
  v = Op::apply(v, dpp<0x140>(id, v)); // row_mirror: rows of 16 reduced
  v = Op::apply(v, dpp<0x142, 0xA>(id, v)); // row_bcast15 into rows 1,3
  v = Op::apply(v, dpp<0x143, 0xC>(id, v)); // row_bcast31 into rows 2,3
  return __builtin_bit_cast(
      T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Reduction over the WAVES consecutive waves that share one row: one LDS slot
// per wave, one barrier.  `slots` must hold WAVES values, belong to this row
// only, and must not be reused for another reduction without a barrier in
// between (callers pass a different slot array per step).  Every thread of the
// workgroup must call it (the barrier is workgroup-wide).
template <class Op, int WAVES>
__device__ __forceinline__ typename Op::T group_reduce(typename Op::T v,
                                                       typename Op::T *slots) {
  v = wave_reduce<Op>(v);
  if constexpr (WAVES == 1)
    return v;
  const int wave = (threadIdx.x / kWave) % WAVES;
  if ((threadIdx.x & (kWave - 1)) == 0)
    slots[wave] = v;
  __syncthreads();
  typename Op::T r = slots[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w)
    r = Op::apply(r, slots[w]);
  return r;
}

} // namespace hcamd
