// Elementwise maps: c = a + b (fp32) and d = a * b + c (fp16 storage, fp32
// arithmetic).  HBM-bound: every element is read once and written once.
//
// Flat kernels treat a contiguous tensor as one vector of 16-byte words.  A
// workgroup owns VPT * 256 consecutive words; thread t takes words t, t+256,
// ... so every wave-level access covers 1 KiB of consecutive bytes.  Workgroups
// that lie wholly inside the array run without any bounds test (a scalar
// branch); only the last workgroup predicates per word and finishes the
// sub-word tail per element, so tail masking costs nothing on the bulk.
#include "common.h"

using namespace hcamd;

namespace {
constexpr int kThreads = 256;

struct AddF32 {
  using Vec = f32x4;
  using Elem = float;
  static constexpr int kElems = 4;
  static constexpr int kInputs = 2;
  static __device__ __forceinline__ Vec apply(const Vec *in) {
    return in[0] + in[1];
  }
  static __device__ __forceinline__ Elem apply1(const Elem *in) {
    return in[0] + in[1];
  }
};

struct FmaF16 {
  using Vec = f16x8;
  using Elem = _Float16;
  static constexpr int kElems = 8;
  static constexpr int kInputs = 3;
  static __device__ __forceinline__ Elem apply1(const Elem *in) {
    // fp16 x fp16 is exact in fp32 (11+11 significand bits), so the rounding
    // of the separate multiply never happens and mul+add equals a fused
    // multiply-add.  Two roundings remain and both are required: the fp32 sum
    // (nearest even) and then the fp32->fp16 conversion (nearest even).  The
    // one-instruction form v_fma_mixlo_f16 rounds the exact sum straight to
    // fp16 and differs from that in about one element in 70,000 (an fp32
    // result that lands on an fp16 tie), so the fp32 value is pinned in a
    // register before it is converted.
    float r = __builtin_fmaf((float)in[0], (float)in[1], (float)in[2]);
    asm volatile("" : "+v"(r));
    return (_Float16)r;
  }
  static __device__ __forceinline__ Vec apply(const Vec *in) {
    Vec r;
#pragma unroll
    for (int i = 0; i < kElems; ++i) {
      Elem e[3] = {in[0][i], in[1][i], in[2][i]};
      r[i] = apply1(e);
    }
    return r;
  }
};

struct Ptrs3 {
  const void *in[3];
  void *out;
};

// DELAY: the wave sleeps DELAY * 64 clocks between the arrival of its operands
// and its stores (see the paced kernels below).
template <class Op, int VPT, bool NT, int DELAY = 0>
__device__ __forceinline__ void flat_map(const Ptrs3 &p, size_t n) {
  using Vec = typename Op::Vec;
  using Elem = typename Op::Elem;
  const size_t nvec = n / Op::kElems;
  const size_t first = (size_t)blockIdx.x * (kThreads * VPT) + threadIdx.x;
  const Vec *in[Op::kInputs];
#pragma unroll
  for (int a = 0; a < Op::kInputs; ++a)
    in[a] = static_cast<const Vec *>(p.in[a]);
  Vec *out = static_cast<Vec *>(p.out);

  if (((size_t)blockIdx.x + 1) * (kThreads * VPT) <= nvec) {
    Vec v[VPT][Op::kInputs];
#pragma unroll
    for (int a = 0; a < Op::kInputs; ++a)
#pragma unroll
      for (int j = 0; j < VPT; ++j)
        v[j][a] = ldg<NT>(in[a] + first + (size_t)j * kThreads);
    if constexpr (DELAY > 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_sleep(DELAY);
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      stg<NT>(out + first + (size_t)j * kThreads, Op::apply(v[j]));
    return;
  }

  // Last workgroup: per-word predicate, then the elements past the last
  // whole word, one per thread.
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const size_t w = first + (size_t)j * kThreads;
    if (w < nvec) {
      Vec v[Op::kInputs];
#pragma unroll
      for (int a = 0; a < Op::kInputs; ++a)
        v[a] = in[a][w];
      out[w] = Op::apply(v);
    }
  }
  const size_t e = nvec * Op::kElems + threadIdx.x;
  if (threadIdx.x < Op::kElems && e < n) {
    Elem s[Op::kInputs];
#pragma unroll
    for (int a = 0; a < Op::kInputs; ++a)
      s[a] = static_cast<const Elem *>(p.in[a])[e];
    static_cast<Elem *>(p.out)[e] = Op::apply1(s);
  }
}
} // namespace

#define HCAMD_FLAT_ADD(NAME, VPT, NT)                                          \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *a, const float *b, float *c, size_t n) {                    \
    Ptrs3 p{{a, b, nullptr}, c};                                               \
    flat_map<AddF32, VPT, NT>(p, n);                                           \
  }

#define HCAMD_FLAT_FMA(NAME, VPT, NT)                                          \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const _Float16 *a, const _Float16 *b, const _Float16 *c, _Float16 *d,    \
      size_t n) {                                                              \
    Ptrs3 p{{a, b, c}, d};                                                     \
    flat_map<FmaF16, VPT, NT>(p, n);                                           \
  }

HCAMD_FLAT_ADD(hcamd_add_f32_v1, 1, false)
HCAMD_FLAT_ADD(hcamd_add_f32_v2, 2, false)
HCAMD_FLAT_ADD(hcamd_add_f32_v4, 4, false)
HCAMD_FLAT_ADD(hcamd_add_f32_v8, 8, false)
HCAMD_FLAT_ADD(hcamd_add_f32_v1_nt, 1, true)
HCAMD_FLAT_ADD(hcamd_add_f32_v2_nt, 2, true)
HCAMD_FLAT_ADD(hcamd_add_f32_v4_nt, 4, true)
HCAMD_FLAT_ADD(hcamd_add_f32_v8_nt, 8, true)

// Paced kernels: one word per lane, the number of resident waves held down by
// holding registers the kernel does not need (REG = highest register touched:
// 127 -> 4 waves per SIMD, 95 -> 5), and a pause between the arrival of a wave's
// operands and its store.  With three read streams and one write stream every
// wave that stores the moment its loads are back keeps reads and writes finely
// mixed at the memory; four waves per SIMD and 6 * 64 clocks of pause measured
// best (8191 x 8193 fp16: 85.9 -> 80.4 us, 0.78 -> 0.83 of the HBM peak).  The
// same treatment of the two-stream fp32 sum measured no better than v4_nt.
#define HCAMD_FLAT_FMA_PACED(NAME, REG, DELAY)                                 \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const _Float16 *a, const _Float16 *b, const _Float16 *c, _Float16 *d,    \
      size_t n) {                                                              \
    asm volatile("v_mov_b32 v" #REG ", 0" ::: "v" #REG);                       \
    Ptrs3 p{{a, b, c}, d};                                                     \
    flat_map<FmaF16, 1, true, DELAY>(p, n);                                    \
  }
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w4_d6, 127, 6)
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w4_d0, 127, 0)
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w4_d3, 127, 3)
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w4_d12, 127, 12)
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w5_d12, 95, 12)
HCAMD_FLAT_FMA_PACED(hcamd_fma_f16_v1_nt_w6_d8, 79, 8)
HCAMD_FLAT_FMA(hcamd_fma_f16_v1, 1, false)
HCAMD_FLAT_FMA(hcamd_fma_f16_v2, 2, false)
HCAMD_FLAT_FMA(hcamd_fma_f16_v4, 4, false)
HCAMD_FLAT_FMA(hcamd_fma_f16_v1_nt, 1, true)
HCAMD_FLAT_FMA(hcamd_fma_f16_v2_nt, 2, true)
HCAMD_FLAT_FMA(hcamd_fma_f16_v4_nt, 4, true)

// General path: any base alignment, any leading dimensions.  One element per
// work-item; x runs along the row so a wave reads consecutive elements.
extern "C" __global__ __launch_bounds__(256) void hcamd_add_f32_scalar(
    const float *a, const float *b, float *c, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    c[i] = a[i] + b[i];
}

// Windows of larger arrays (leading dimension != columns): a row is walked in
// groups of V elements, V = 8, 4 or 2 as the common alignment of the four
// arrays' rows allows (16-, 8- or 4-byte accesses), the cols % V elements at
// the end of the row one by one.  blockIdx.y walks rows, x the groups of a row.
template <int V>
__device__ __forceinline__ void fma_rows(const _Float16 *a, size_t lda, const _Float16 *b,
                                         size_t ldb, const _Float16 *c, size_t ldc,
                                         _Float16 *d, size_t ldd, size_t cols) {
  typedef _Float16 hv __attribute__((ext_vector_type(V)));
  const size_t row = blockIdx.y;
  const size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t whole = cols / V;
  const _Float16 *ar = a + row * lda, *br = b + row * ldb, *cr = c + row * ldc;
  _Float16 *dr = d + row * ldd;
  if (g < whole) {
    const hv x = __builtin_nontemporal_load(reinterpret_cast<const hv *>(ar) + g);
    const hv y = __builtin_nontemporal_load(reinterpret_cast<const hv *>(br) + g);
    const hv z = __builtin_nontemporal_load(reinterpret_cast<const hv *>(cr) + g);
    hv r;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      _Float16 e[3] = {x[i], y[i], z[i]};
      r[i] = FmaF16::apply1(e);
    }
    __builtin_nontemporal_store(r, reinterpret_cast<hv *>(dr) + g);
  } else if (g - whole < cols % V) {
    const size_t col = whole * V + (g - whole);
    _Float16 e[3] = {ar[col], br[col], cr[col]};
    dr[col] = FmaF16::apply1(e);
  }
}
#define HCAMD_FMA_ROWS(NAME, V)                                                \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const _Float16 *a, size_t lda, const _Float16 *b, size_t ldb,            \
      const _Float16 *c, size_t ldc, _Float16 *d, size_t ldd, size_t rows,     \
      size_t cols) {                                                           \
    fma_rows<V>(a, lda, b, ldb, c, ldc, d, ldd, cols);                         \
  }
HCAMD_FMA_ROWS(hcamd_fma_f16_rows_v8, 8)
HCAMD_FMA_ROWS(hcamd_fma_f16_rows_v4, 4)
HCAMD_FMA_ROWS(hcamd_fma_f16_rows_v2, 2)

extern "C" __global__ __launch_bounds__(256) void hcamd_fma_f16_2d(
    const _Float16 *a, size_t lda, const _Float16 *b, size_t ldb,
    const _Float16 *c, size_t ldc, _Float16 *d, size_t ldd, size_t rows,
    size_t cols) {
  const size_t col = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t row = blockIdx.y;
  if (col < cols && row < rows) {
    _Float16 e[3] = {a[row * lda + col], b[row * ldb + col],
                     c[row * ldc + col]};
    d[row * ldd + col] = FmaF16::apply1(e);
  }
}
