// Matrix product of gathered tiles (fp32, fp16 or bf16 storage; products and sums
// in fp32, one rounding on the way out):
//
//   out[map_o(i, j)] = sum_k a[map_a(i, k)] * b[map_b(k, j)]      per group
//
// The operation behind a kernel body that loads its operands through index
// mappings (python/hckernel/kernel_api.py:297-345 with mapping=..., as in the
// implicit-GEMM convolution of python/hckernel/tests/test_examples.py:168-258)
// and multiplies them with numpy.dot.  Every group has its own window into each
// buffer (a start per dimension); inside the window the tile element (r, c)
// sits at index row[r][d] + col[c][d] along dimension d, and each dimension is
// driven by the tile row or by the tile column, never by both.  An element is
// active if every index is inside the window, exactly the reference's bounds
// test; inactive operand elements count as zero and inactive output elements
// are not written.
//
// Tables (built and bounds-checked on the host):
//   groups[g]  16 ints: {base, extent[4]} for a, b and out (base = element
//              offset of the window, extent = buffer size - start per dim),
//              then one word: bit 0 = the set's out windows are neighbours,
//              bit 1 = its a windows are neighbours and every a element is
//              active, bits 2.. = index of the packed b tile
//   *_rows[r], *_cols[c]  8 ints: {offset, index[4], unused[3]} (offset = sum
//              of index * stride; dimensions the other coordinate drives hold 0)
//
// The b tile of a group depends only on its b window, and many groups share one
// (every output position of a convolution reads the same filters).  A first
// kernel gathers each distinct b tile once into a dense K_pad x TN_pad array
// (inactive elements and padding are zero); the product kernel then reads its b
// panels with plain 16-byte loads and spends its gathers on a alone.
//
// One workgroup per group; the TM x TN tile is walked in T x T blocks, R x R
// outputs per lane, K in steps of 32 through LDS panels stored k-major so that
// a lane's R operands are one LDS read.  Four shapes are built: T = 64 (R = 4,
// 256 lanes) for large tiles and T = 32, 16, 8 (R = 4, 2, 1, one wave) so that
// small tiles do not pay for a 64 x 64 block of mostly inactive lanes.  The
// gathers of the next K step are issued before the multiply-adds of the current
// one.  The host lays the group records out by window address, and consecutive
// records go to the same XCD, so that groups that run together share cache lines
// in that XCD's L2.
//
// Fusion (G = 2, 4 or 16): a workgroup takes G consecutive records that read the
// same b window and treats them as one tile of G * TM rows, row v belonging to
// record v % G and tile row v / G.  The b panel is then gathered once for G
// groups, and because neighbouring records are neighbouring windows of a (the
// next output position of a convolution), the G lanes that gather one tile row
// for the G groups read adjacent addresses: one cache line serves them all.
#include "common.h"
#include <type_traits>

using namespace hcamd;

namespace {
constexpr int kXcds = 8;

struct GatherGemmArgs {
  const void *a;
  const float *bpack; // b tiles packed by hcamd_gather_pack_b (always fp32)
  void *out;
  const int32_t *groups;
  const int32_t *a_rows, *a_cols, *o_rows, *o_cols;
  uint32_t tm, tn, k, n_groups, per_xcd;
  uint32_t k_pad, tn_pad; // rows / row length of a packed b tile
};

struct PackBArgs {
  const void *b;
  float *bpack;
  const int32_t *windows; // [n_windows][8]: base, extent[4]
  const int32_t *b_rows, *b_cols;
  uint32_t k, tn, k_pad, tn_pad, n_windows;
};

struct Window {
  uint32_t base;
  uint32_t ext[4];
};

// offset of a table entry if all of its indices are inside the window, else -1
__device__ __forceinline__ int resolve(const int32_t *entry, const Window &w) {
  const u32x4 lo = *reinterpret_cast<const u32x4 *>(entry);
  const uint32_t i3 = static_cast<uint32_t>(entry[4]);
  const bool ok = lo.y < w.ext[0] && lo.z < w.ext[1] && lo.w < w.ext[2] &&
                  i3 < w.ext[3];
  return ok ? static_cast<int>(lo.x) : -1;
}

__device__ __forceinline__ Window window_of(const int32_t *rec) {
  Window w;
  w.base = static_cast<uint32_t>(rec[0]);
#pragma unroll
  for (int d = 0; d < 4; ++d)
    w.ext[d] = static_cast<uint32_t>(rec[1 + d]);
  return w;
}
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ bool inside(u32x4 lo, uint32_t i3, const Window &w) {
  return lo.y < w.ext[0] && lo.z < w.ext[1] && lo.w < w.ext[2] && i3 < w.ext[3];
}

// MFMA = false: R x R outputs per lane, fp32 FMAs on the vector ALUs.
// MFMA = true (T = 32 or 64, R = 4): every wave owns a 32 x 32 sub-block and
// accumulates it with v_mfma_f32_32x32x2_f32, two K values per instruction:
// lane l supplies a[l % 32][l / 32] and b[l / 32][l % 32] and holds
// c[8*g + 4*(l/32) + e][l % 32] in accumulator element 4*g + e.
template <class E, int T, int R, bool MFMA, int G, int kStep>
__device__ __forceinline__ void gather_gemm(const GatherGemmArgs &p) {
  // four elements that are only aligned like one
  typedef E ex4u __attribute__((ext_vector_type(4), aligned(sizeof(E))));
  constexpr int kSide = T / R;            // lanes per block edge
  constexpr int kThreads = kSide * kSide;
  static_assert(!MFMA || (R == 4 && (T == 32 || T == 64)), "MFMA block shapes");
  constexpr int kPitch = T + 4;
  constexpr int kRowsPerPass = kThreads / kStep;
  constexpr int kPasses = T / kRowsPerPass; // gathers per lane, operand and K step
  static_assert(kThreads % kStep == 0 && T % kRowsPerPass == 0, "panel split");
  constexpr bool kPackA = G >= 4 && G % 4 == 0 && 8 % (G / 4) == 0 && T == 64 &&
                          kThreads == 256 && kStep == 32;
  static_assert(kPackA || kRowsPerPass % G == 0, "a pass gathers whole sets of G rows");
  constexpr int kBLoads = kStep * (T / 4) / kThreads; // 16-byte b loads per lane and K step
  static_assert(kStep * (T / 4) % kThreads == 0, "b panel split");
  // 16-bit storage on the matrix cores: the panels hold the stored type, row by
  // row (32 K values + 8 of padding, so that the 16-byte operand reads of eight
  // consecutive rows cover all banks), and feed v_mfma_f32_32x32x16 directly;
  // lane l supplies K values 16*s + 8*(l/32) .. +8 of row l % 32 in sub-step s.
  constexpr bool kLow = MFMA && sizeof(E) == 2;
  static_assert(!kLow || kStep == 32, "16-bit panels are 32 K values wide");
  constexpr int kLowPitch = kStep + 8;
  typedef E ex8 __attribute__((ext_vector_type(8)));
  __shared__ __attribute__((aligned(16))) float as[kLow ? 1 : kStep][kLow ? 4 : kPitch];
  __shared__ __attribute__((aligned(16))) float bs[kLow ? 1 : kStep][kLow ? 4 : kPitch];
  __shared__ __attribute__((aligned(16))) E as16[kLow ? T : 1][kLow ? kLowPitch : 8];
  __shared__ __attribute__((aligned(16))) E bs16[kLow ? T : 1][kLow ? kLowPitch : 8];
  // 16-byte b loads per lane and K step: rows of the packed tile are K-major
  // [k][column] fp32, or, for kLow, column-major [column][k] in the stored type
  constexpr int kBLoads16 = kLow ? T * (kStep / 8) / kThreads : 1;
  // row_a / row_o: absolute element offset of the row's first element, or -1;
  // col_o: offset inside the window; col_ok: bit g set if the column is inside
  // the out window of record g
  __shared__ __attribute__((aligned(16))) int row_a[T], row_o[T], col_o[T], col_ok[T];

  // n_groups counts sets of G records here
  const uint32_t set = (blockIdx.x % kXcds) * p.per_xcd + blockIdx.x / kXcds;
  if (set >= p.n_groups)
    return;
  const int32_t *rec = p.groups + static_cast<size_t>(set) * 16 * G;
  // the a / out window of record g of the set (the records are read where
  // they are needed: a few cached loads per block)
  auto win_a = [&](int g) { return window_of(rec + 16 * g); };
  auto win_o = [&](int g) { return window_of(rec + 16 * g + 10); };
  // set by the host in the first record of a set: the out windows of its
  // records are one element apart, in record order
  const bool run_o = kPackA && (rec[15] & 1);
  const E *a = static_cast<const E *>(p.a);
  // word 15 of the set's first record: bit 0 flags neighbouring out windows,
  // bit 1 a windows that are neighbours and fully active, the rest says which
  // packed b tile the set reads
  const float *bp = p.bpack + (size_t)((uint32_t)rec[15] >> 2) * p.k_pad * p.tn_pad;
  E *out = static_cast<E *>(p.out);
  const uint32_t rows = p.tm * G;

  const int t = threadIdx.x;
  const int tx = t % kSide, ty = t / kSide;
  // gathers: G adjacent lanes take the G records of one tile row (or, for b,
  // G adjacent columns), the next 32 lanes step through K
  const int ld_g = t % G, ld_k = (t / G) % kStep, ld_r = t / (G * kStep);
  const Window my_wa = win_a(kPackA ? 0 : ld_g);
  // MFMA: sub-block of this wave and the lane's place in it
  const int lane = t % kWave, wave = t / kWave;
  constexpr int kSubs = T >= 32 ? T / 32 : 1; // 32 x 32 sub-blocks per edge
  const int sub_m = 32 * (wave / kSubs), sub_n = 32 * (wave % kSubs);
  const int l_lo = lane % 32, l_hi = lane / 32;

  // the T x T blocks of the tile are spread over blockIdx.y
  const uint32_t n_blocks = (p.tn + T - 1) / T;
  const uint32_t blocks = ((rows + T - 1) / T) * n_blocks;
  for (uint32_t block = blockIdx.y; block < blocks; block += gridDim.y) {
    const uint32_t m0 = block / n_blocks * T, n0 = block % n_blocks * T;
    {
      for (int e = t; e < 2 * T; e += kThreads) {
        if (e < T) {
          const uint32_t v = m0 + e, i = v / G;
          const int g = v % G;
          int oa = -1, oo = -1;
          if (i < p.tm) {
            const int32_t *ea = p.a_rows + 8 * (size_t)i;
            const int32_t *eo = p.o_rows + 8 * (size_t)i;
            const u32x4 la = *reinterpret_cast<const u32x4 *>(ea);
            const u32x4 lo = *reinterpret_cast<const u32x4 *>(eo);
            const uint32_t a3 = ea[4], o3 = eo[4];
            const Window wa = win_a(g), wo = win_o(g);
            if (inside(la, a3, wa))
              oa = (int)(wa.base + la.x);
            if (inside(lo, o3, wo))
              oo = (int)(wo.base + lo.x);
          }
          row_a[e] = oa;
          row_o[e] = oo;
        } else {
          const uint32_t c = n0 + e - T;
          int oo = 0, ok = 0;
          if (c < p.tn) {
            const int32_t *eo = p.o_cols + 8 * (size_t)c;
            const u32x4 lo = *reinterpret_cast<const u32x4 *>(eo);
            const uint32_t o3 = eo[4];
            oo = (int)lo.x;
            for (int h = 0; h < G; ++h)
              ok |= inside(lo, o3, win_o(h)) ? 1 << h : 0;
          }
          col_o[e - T] = oo;
          col_ok[e - T] = ok;
        }
      }
      __syncthreads();

      int ra[kPasses];
#pragma unroll
      for (int i = 0; i < kPasses; ++i)
        ra[i] = row_a[(ld_r + kRowsPerPass / G * i) * G + ld_g];
      float acc[R][R];
#pragma unroll
      for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j)
          acc[i][j] = 0.0f;
      f32x16 macc;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        macc[i] = 0.0f;

      // Four fused records (kPackA): a lane gathers one tile row of a for all
      // four records at once.  When their windows follow each other element by
      // element the four values are one 16-byte load; they land next to each
      // other in the panel either way.
      [[maybe_unused]] int ra4[2][4];
      [[maybe_unused]] bool run4[2];
      // kPackA: K value and row quad of the lane; quads pi and pi + 8 hold the
      // same four records, 4 * (pi % (G / 4)) .. + 3
      const int pk = t % kStep, pi = t / kStep;
      [[maybe_unused]] Window wa4[4];
      if constexpr (kPackA) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          wa4[e] = win_a(4 * (pi % (G / 4)) + e);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int v0 = 4 * (pi + 8 * j);
          bool run = true;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ra4[j][e] = row_a[v0 + e];
            run = run && ra4[j][e] >= 0 && ra4[j][e] == ra4[j][0] + e;
          }
          run4[j] = run;
        }
      }
      // Staging registers of one K step.  Every load below is unconditional: an
      // inactive element is read from element 0 of its buffer (always there) and
      // replaced by zero when the step is stored to LDS, so nothing between the
      // loads and that store waits on memory and the loads of a step overlap
      // each other and the multiply-adds of the step before.
      [[maybe_unused]] E raw[kPackA ? 1 : kPasses];      // a, one element per pass
      [[maybe_unused]] uint32_t raw_ok = 0;               // bit i: raw[i] is active
      [[maybe_unused]] ex4u raw4[2];                      // a, kPackA with neighbouring windows
      [[maybe_unused]] E raw1[2][4];                      // a, kPackA in general
      f32x4 vb[kLow ? 1 : kBLoads];
      [[maybe_unused]] ex8 vb16[kBLoads16];
      uint32_t vb_ok = 0;                                 // bit j: b load j is inside the tile
      [[maybe_unused]] int next_off = 0;                  // kFast: a column offset of the next step
      const E *bp16 = reinterpret_cast<const E *>(p.bpack) +
                      (size_t)((uint32_t)rec[15] >> 2) * p.k_pad * p.tn_pad;
      auto gather = [&](uint32_t k0, auto fast) {
        constexpr bool kFast = decltype(fast)::value;
        // b: the next kStep rows of the packed tile, columns n0 .. n0 + T
        vb_ok = 0;
        if constexpr (kLow) {
#pragma unroll
          for (int j = 0; j < kBLoads16; ++j) {
            const int id = t + j * kThreads, part = id % (kStep / 8);
            const uint32_t c = n0 + id / (kStep / 8);
            const bool ok = c < p.tn_pad;
            vb_ok |= ok ? 1u << j : 0u;
            vb16[j] = *reinterpret_cast<const ex8 *>(bp16 + (size_t)(ok ? c : 0) * p.k_pad + k0 +
                                                     8 * part);
          }
        } else {
#pragma unroll
          for (int j = 0; j < kBLoads; ++j) {
            const int id = t + j * kThreads, kr = id / (T / 4);
            const uint32_t c = n0 + 4 * (id % (T / 4));
            const bool ok = c < p.tn_pad;
            vb_ok |= ok ? 1u << j : 0u;
            vb[j] = *reinterpret_cast<const f32x4 *>(bp + (size_t)(k0 + kr) * p.tn_pad +
                                                     (ok ? c : 0));
          }
        }
        if constexpr (!kPackA) {
          const uint32_t kk = k0 + ld_k;
          const int oa = resolve(p.a_cols + 8 * (size_t)(kk < p.k ? kk : 0), my_wa);
          raw_ok = 0;
#pragma unroll
          for (int i = 0; i < kPasses; ++i) {
            // both offsets are non-negative when valid: the sign of the OR says
            // whether either is the -1 marker
            const bool ok = kk < p.k && (oa | ra[i]) >= 0;
            raw_ok |= ok ? 1u << i : 0u;
            raw[i] = a[ok ? oa + ra[i] : 0];
          }
        } else {
          const uint32_t ka = k0 + pk;
          const int32_t *pa = p.a_cols + 8 * (size_t)(ka < p.k ? ka : 0);
          if constexpr (kFast) {
            // every element of the set is active and the four windows of a quad
            // are neighbours: one 16-byte (8-byte) load per quad.  The column
            // offset was requested one step ago; the next one is requested now.
            const int off = next_off;
            const uint32_t kn = ka + kStep;
            next_off = p.a_cols[8 * (size_t)(kn < p.k ? kn : 0)];
            raw_ok = ka < p.k ? 1u : 0u;
#pragma unroll
            for (int j = 0; j < 2; ++j)
              raw4[j] = *reinterpret_cast<const ex4u *>(a + off + ra4[j][0]);
          } else {
            const u32x4 ea = *reinterpret_cast<const u32x4 *>(pa);
            const uint32_t ea3 = pa[4];
            const int off = (int)ea.x;
            raw_ok = 0;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const bool ok = ka < p.k && inside(ea, ea3, wa4[e]) && ra4[j][e] >= 0;
                raw_ok |= ok ? 1u << (4 * j + e) : 0u;
                raw1[j][e] = a[ok ? off + ra4[j][e] : 0];
              }
          }
        }
      };
      auto commit = [&](auto fast) {
        constexpr bool kFast = decltype(fast)::value;
        if constexpr (kLow) {
#pragma unroll
          for (int j = 0; j < kBLoads16; ++j) {
            const int id = t + j * kThreads;
            ex8 v = vb16[j];
            if (!((vb_ok >> j) & 1))
#pragma unroll
              for (int e = 0; e < 8; ++e)
                v[e] = (E)0.0f;
            *reinterpret_cast<ex8 *>(&bs16[id / (kStep / 8)][8 * (id % (kStep / 8))]) = v;
          }
        } else {
#pragma unroll
          for (int j = 0; j < kBLoads; ++j) {
            const int id = t + j * kThreads;
            const f32x4 v = ((vb_ok >> j) & 1) ? vb[j] : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            *reinterpret_cast<f32x4 *>(&bs[id / (T / 4)][4 * (id % (T / 4))]) = v;
          }
        }
        if constexpr (!kPackA) {
#pragma unroll
          for (int i = 0; i < kPasses; ++i) {
            const int v = (ld_r + kRowsPerPass / G * i) * G + ld_g;
            const E x = ((raw_ok >> i) & 1) ? raw[i] : (E)0.0f;
            if constexpr (kLow)
              as16[v][ld_k] = x;
            else
              as[ld_k][v] = (float)x;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            E x[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if constexpr (kFast)
                x[e] = (raw_ok & 1) ? (E)raw4[j][e] : (E)0.0f;
              else
                x[e] = ((raw_ok >> (4 * j + e)) & 1) ? raw1[j][e] : (E)0.0f;
            }
            if constexpr (kLow) {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                as16[4 * (pi + 8 * j) + e][pk] = x[e];
            } else {
              *reinterpret_cast<f32x4 *>(&as[pk][4 * (pi + 8 * j)]) =
                  f32x4{(float)x[0], (float)x[1], (float)x[2], (float)x[3]};
            }
          }
        }
      };
      auto multiply = [&]() {
        if constexpr (kLow) {
#pragma unroll
          for (int sub = 0; sub < kStep / 16; ++sub) {
            const ex8 x = *reinterpret_cast<const ex8 *>(&as16[sub_m + l_lo][16 * sub + 8 * l_hi]);
            const ex8 y = *reinterpret_cast<const ex8 *>(&bs16[sub_n + l_lo][16 * sub + 8 * l_hi]);
            if constexpr (std::is_same<E, __bf16>::value)
              macc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, macc, 0, 0, 0);
            else
              macc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, macc, 0, 0, 0);
          }
        } else if constexpr (MFMA) {
#pragma unroll
          for (int kk = 0; kk < kStep; kk += 2)
            macc = __builtin_amdgcn_mfma_f32_32x32x2f32(
                as[kk + l_hi][sub_m + l_lo], bs[kk + l_hi][sub_n + l_lo], macc,
                0, 0, 0);
        } else {
#pragma unroll 8
          for (int kk = 0; kk < kStep; ++kk) {
            float av[R], bv[R];
            if constexpr (R == 4) {
              const f32x4 x = *reinterpret_cast<const f32x4 *>(&as[kk][R * ty]);
              const f32x4 y = *reinterpret_cast<const f32x4 *>(&bs[kk][R * tx]);
#pragma unroll
              for (int i = 0; i < R; ++i) {
                av[i] = x[i];
                bv[i] = y[i];
              }
            } else {
#pragma unroll
              for (int i = 0; i < R; ++i) {
                av[i] = as[kk][R * ty + i];
                bv[i] = bs[kk][R * tx + i];
              }
            }
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
              for (int j = 0; j < R; ++j)
                acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
          }
        }
      };
      auto k_loop = [&](auto fast) {
        if constexpr (decltype(fast)::value)
          next_off = p.a_cols[8 * (size_t)((uint32_t)pk < p.k ? pk : 0)];
        if (p.k > 0)
          gather(0, fast);
        for (uint32_t k0 = 0; k0 < p.k; k0 += kStep) {
          commit(fast);
          __syncthreads();
          if (k0 + kStep < p.k)
            gather(k0 + kStep, fast);
          multiply();
          __syncthreads();
        }
      };
      // bit 1 of the flag word: every a element of the set is active and its a
      // windows are neighbours (host-checked), so the quads of this block can be
      // read as vectors if their rows are neighbours too.  The choice is made per
      // wave: both loops store the same panels and pass the same barriers.
      bool fast_a = false;
      if constexpr (kPackA)
        fast_a = (rec[15] & 2) && __builtin_amdgcn_ballot_w64(!(run4[0] && run4[1])) == 0;
      if (fast_a)
        k_loop(std::true_type{});
      else
        k_loop(std::false_type{});

      // block row v belongs to record v % G (m0 is a multiple of G)
      if constexpr (MFMA) {
        const int co = col_o[sub_n + l_lo], ok = col_ok[sub_n + l_lo];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // accumulator elements 4q .. 4q+3 are four consecutive block rows:
          // with fused records one tile row for four records of the set.  When
          // their out windows follow each other element by element
          // (run_o) the four values are one 16-byte store.
          const int v0 = sub_m + 8 * q + 4 * l_hi;
          int ro[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            ro[e] = row_o[v0 + e];
          bool packed = false;
          if constexpr (kPackA)
            packed = run_o && ((ok >> (v0 % G)) & 0xF) == 0xF &&
                     (ro[0] | ro[1] | ro[2] | ro[3]) >= 0;
          if (packed) {
            ex4u val;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              val[e] = (E)macc[4 * q + e];
            *reinterpret_cast<ex4u *>(out + ro[0] + co) = val;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (ro[e] >= 0 && ((ok >> ((v0 + e) % G)) & 1))
                out[ro[e] + co] = (E)macc[4 * q + e];
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < R; ++i) {
          const int v = R * ty + i;
          const int ro = row_o[v];
#pragma unroll
          for (int j = 0; j < R; ++j) {
            const int co = col_o[R * tx + j], ok = col_ok[R * tx + j];
            if (ro >= 0 && ((ok >> (v % G)) & 1))
              out[ro + co] = (E)acc[i][j];
          }
        }
      }
      __syncthreads();
    }
  }
}
} // namespace

// bpack[w][k][c] = b element (k, c) of window w, zero where inactive or padding
template <class E> __device__ __forceinline__ void pack_b(const PackBArgs &p) {
  const uint32_t w = blockIdx.y;
  const int32_t *rec = p.windows + 8 * (size_t)w;
  const Window wb = window_of(rec);
  const E *b = static_cast<const E *>(p.b);
  const size_t per = (size_t)p.k_pad * p.tn_pad;
  for (size_t id = (size_t)blockIdx.x * 256 + threadIdx.x; id < per;
       id += (size_t)gridDim.x * 256) {
    const uint32_t k = (uint32_t)(id / p.tn_pad), c = (uint32_t)(id % p.tn_pad);
    float v = 0.0f;
    if (k < p.k && c < p.tn) {
      const int ok = resolve(p.b_rows + 8 * (size_t)k, wb);
      const int oc = resolve(p.b_cols + 8 * (size_t)c, wb);
      if ((ok | oc) >= 0)
        v = (float)b[wb.base + ok + oc];
    }
    p.bpack[(size_t)w * per + id] = v;
  }
}
// the same in the stored 16-bit type and column by column: bpack[w][c][k]
template <class E> __device__ __forceinline__ void pack_b_low(const PackBArgs &p) {
  const uint32_t w = blockIdx.y;
  const Window wb = window_of(p.windows + 8 * (size_t)w);
  const E *b = static_cast<const E *>(p.b);
  E *dst = reinterpret_cast<E *>(p.bpack);
  const size_t per = (size_t)p.k_pad * p.tn_pad;
  for (size_t id = (size_t)blockIdx.x * 256 + threadIdx.x; id < per;
       id += (size_t)gridDim.x * 256) {
    const uint32_t c = (uint32_t)(id / p.k_pad), k = (uint32_t)(id % p.k_pad);
    E v = (E)0.0f;
    if (k < p.k && c < p.tn) {
      const int ok = resolve(p.b_rows + 8 * (size_t)k, wb);
      const int oc = resolve(p.b_cols + 8 * (size_t)c, wb);
      if ((ok | oc) >= 0)
        v = b[wb.base + ok + oc];
    }
    dst[(size_t)w * per + id] = v;
  }
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gather_pack_b_low_f16(PackBArgs p) {
  pack_b_low<_Float16>(p);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gather_pack_b_low_bf16(PackBArgs p) {
  pack_b_low<__bf16>(p);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gather_pack_b_f32(PackBArgs p) {
  pack_b<float>(p);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gather_pack_b_f16(PackBArgs p) {
  pack_b<_Float16>(p);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gather_pack_b_bf16(PackBArgs p) {
  pack_b<__bf16>(p);
}

#define HCAMD_GATHER_GEMM(NAME, E, T, R, MFMA, G, KS)                          \
  extern "C" __global__ __launch_bounds__((T / R) * (T / R)) void NAME(        \
      GatherGemmArgs p) {                                                      \
    gather_gemm<E, T, R, MFMA, G, KS>(p);                                      \
  }
// block shape (m = matrix cores, t = vector ALUs) and records per workgroup
#define HCAMD_GATHER_SET(TY, E)                                                \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m64_g1, E, 64, 4, true, 1, 32)    \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m64_g2, E, 64, 4, true, 2, 32)    \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m64_g4, E, 64, 4, true, 4, 32)    \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m64_g16, E, 64, 4, true, 16, 32)  \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m32_g1, E, 32, 4, true, 1, 32)    \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_m32_g2, E, 32, 4, true, 2, 32)    \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_t16_g1, E, 16, 2, false, 1, 32)   \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_t16_g2, E, 16, 2, false, 2, 32)   \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_t8_g1, E, 8, 1, false, 1, 32)     \
  HCAMD_GATHER_GEMM(hcamd_gather_gemm_##TY##_t8_g2, E, 8, 1, false, 2, 32)
HCAMD_GATHER_SET(f32, float)
HCAMD_GATHER_SET(f16, _Float16)
HCAMD_GATHER_SET(bf16, __bf16)
// the 64- and 32-wide blocks on the vector ALUs, kept for comparison (fp32 only)
HCAMD_GATHER_GEMM(hcamd_gather_gemm_f32_t64_g1, float, 64, 4, false, 1, 32)
HCAMD_GATHER_GEMM(hcamd_gather_gemm_f32_t32_g1, float, 32, 4, false, 1, 32)
