// C[M,N] = A[M,K] * B[K,N], bf16 inputs, fp32 accumulation on MFMA, bf16
// output (round to nearest even).  A is row-major; B is column-major and is
// passed as Bt[N,K] row-major, so both operands are K-contiguous.
//
// Tiled kernel.  A workgroup of WM x WN waves owns a BM x BN tile of C and walks
// K in steps of 64.  Each step's A and B panels (BM x 64 and BN x 64 bf16) live
// in LDS, double buffered: while the MFMAs consume buffer b, the global loads
// for the next step are in flight into registers and are written to buffer b^1
// afterwards; one barrier per step.
//
// LDS layout: a panel row is 64 bf16 = 128 bytes = eight 16-byte chunks.  Chunk
// c of row r is stored at chunk position c ^ swz(r), so that the sixteen lanes
// of an MFMA operand read (sixteen consecutive rows, same logical chunk) fall
// into different banks, and so do the eight lanes that write one row.
//
// MFMA: v_mfma_f32_16x16x32_bf16.  Lane l supplies row (l % 16) and the eight
// K values 8*(l/16)..8*(l/16)+7 of each 16 x 32 operand block, i.e. exactly
// one 16-byte chunk of a panel row.  The Bt block is given as the first
// operand and the A block as the second, which yields the transposed product:
// lane l then holds C[m = l % 16][n = 4*(l/16) .. 4*(l/16)+3], four consecutive
// columns that are stored as one 8-byte word.
//
// Workgroup order: consecutive workgroup ids go to different XCDs (each with a
// private L2), so ids are first regrouped to give each XCD a contiguous range
// and the range is then walked in GROUP_M-row bands; an XCD's concurrent tiles
// form a compact block that shares A and B panels in its L2.
#include "common.h"

#include <type_traits>

using namespace hcamd;

namespace {

constexpr int kBK = 64;         // K step (bf16 elements)
constexpr int kRowBytes = 128;  // kBK * 2
constexpr int kChunks = 8;      // 16-byte chunks per panel row
constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// s_waitcnt immediates (gfx9 encoding: vmcnt[3:0] at 3:0 and [5:4] at 15:14,
// expcnt at 6:4, lgkmcnt at 11:8).  Issued through the builtin so that the
// compiler's own wait insertion sees them and counts from there.
constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) {
  return (vmcnt & 0xf) | ((vmcnt >> 4) << 14) | (7 << 4) | ((lgkmcnt & 0xf) << 8);
}
constexpr int kNoVm = 63, kNoLgkm = 15;

template <int SH> __device__ __forceinline__ int swz(int row) {
  return (row >> SH) & 7;
}

__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n,
                                                  int &tm, int &tn) {
  const int n_wg = tiles_m * tiles_n;
  int wg = blockIdx.x;
  if (n_wg % kXcds == 0)
    wg = (wg % kXcds) * (n_wg / kXcds) + wg / kXcds;
  const int band = kGroupM * tiles_n;
  const int first_m = (wg / band) * kGroupM;
  const int rows = min(tiles_m - first_m, kGroupM);
  const int in_band = wg % band;
  tm = first_m + in_band % rows;
  tn = in_band / rows;
}

template <int BM, int BN, int WM, int WN, int SH>
__device__ __forceinline__ void gemm_tile(const __bf16 *__restrict__ A,
                                          size_t lda,
                                          const __bf16 *__restrict__ Bt,
                                          size_t ldb, __bf16 *__restrict__ C,
                                          size_t ldc, int M, int N, int K) {
  constexpr int kThreads = WM * WN * kWave;
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int kMI = kWaveM / 16;
  constexpr int kNI = kWaveN / 16;
  constexpr int kALoads = BM * kChunks / kThreads;
  constexpr int kBLoads = BN * kChunks / kThreads;
  static_assert(BM * kChunks % kThreads == 0 && BN * kChunks % kThreads == 0,
                "panel chunks must divide evenly over the threads");
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;

  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  // ---- global -> register -> LDS staging ---------------------------------
  // chunk id = tid + i * kThreads: row = id / 8, chunk = id % 8
  const __bf16 *a_src[kALoads];
  const __bf16 *b_src[kBLoads];
  int a_dst[kALoads], b_dst[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int id = tid + i * kThreads;
    const int r = id / kChunks, c = id % kChunks;
    a_src[i] = A + (size_t)(tm * BM + r) * lda + c * 8;
    a_dst[i] = r * kRowBytes + ((c ^ swz<SH>(r)) * 16);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int id = tid + i * kThreads;
    const int r = id / kChunks, c = id % kChunks;
    b_src[i] = Bt + (size_t)(tn * BN + r) * ldb + c * 8;
    b_dst[i] = kABytes + r * kRowBytes + ((c ^ swz<SH>(r)) * 16);
  }

  // ---- LDS -> operand registers -------------------------------------------
  // operand block row = base + lane % 16, logical chunk = 4*ks + lane / 16
  int a_off[kMI], b_off[kNI];
  const int lrow = lane % 16, lchunk = lane / 16;
#pragma unroll
  for (int i = 0; i < kMI; ++i)
    a_off[i] = (wave_m + i * 16 + lrow) * kRowBytes;
#pragma unroll
  for (int i = 0; i < kNI; ++i)
    b_off[i] = kABytes + (wave_n + i * 16 + lrow) * kRowBytes;
  // rows base+lrow with base % 16 == 0: swz depends on lrow only
  const int lswz = swz<SH>(lrow);

  f32x4 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 a_reg[kALoads], b_reg[kBLoads];
  auto load_global = [&](int kt) {
    const size_t k0 = (size_t)kt * kBK;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      a_reg[i] = *reinterpret_cast<const u32x4 *>(a_src[i] + k0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      b_reg[i] = *reinterpret_cast<const u32x4 *>(b_src[i] + k0);
  };
  auto store_lds = [&](int buf) {
    unsigned char *base = lds + buf * kStageBytes;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      *reinterpret_cast<u32x4 *>(base + a_dst[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      *reinterpret_cast<u32x4 *>(base + b_dst[i]) = b_reg[i];
  };
  auto compute = [&](int buf) {
    const unsigned char *base = lds + buf * kStageBytes;
#pragma unroll
    for (int ks = 0; ks < kBK / 32; ++ks) {
      const int coff = ((ks * 4 + lchunk) ^ lswz) * 16;
      bf16x8 af[kMI], bfr[kNI];
#pragma unroll
      for (int i = 0; i < kMI; ++i)
        af[i] = *reinterpret_cast<const bf16x8 *>(base + a_off[i] + coff);
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8 *>(base + b_off[j] + coff);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
#pragma unroll
        for (int j = 0; j < kNI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              bfr[j], af[i], acc[i][j], 0, 0, 0);
    }
  };

  const int KT = K / kBK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT)
      load_global(kt + 1);
    compute(buf);
    if (kt + 1 < KT)
      store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: fp32 -> bf16 (nearest even), 8-byte stores ---------------
  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lchunk * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * 16) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
      bf16x4 o;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        o[r] = (__bf16)acc[i][j][r];
      *reinterpret_cast<bf16x4 *>(crow + j * 16) = o;
    }
  }
}
// ---------------------------------------------------------------------------
// Pipelined kernel.  Same tiling and LDS layout as gemm_tile, but
//   * panels go from global memory straight into LDS (global_load_lds, 16
//     bytes per lane): a wave-level load fills 1 KiB of consecutive LDS, i.e.
//     eight panel rows, and the swizzle is applied on the global side (lane l
//     fetches logical chunk (l % 8) ^ swz(row) so that it lands in physical
//     chunk l % 8).  No staging registers, no ds_write.
//   * K is walked in half-steps of 32.  While the MFMAs of half-step h run, the
//     operand fragments of h+1 are read from LDS into a second register set, and
//     the panels of the tile after next are in flight from global memory.
//   * One barrier per 64-wide K tile, at the start of the odd half-step: by
//     then this wave's loads of the next tile have landed (vmcnt) and its
//     reads of the current tile are complete (lgkmcnt), so after the barrier
//     the next tile may be read and the current tile's buffer overwritten.
//   * The MFMA block size is a parameter.  MF = 16: v_mfma_f32_16x16x32_bf16,
//     one instruction per block and half-step; lane l supplies row l % 16 and
//     chunk l / 16, and holds C[l % 16][4*(l/16) + e].  MF = 32:
//     v_mfma_f32_32x32x16_bf16, two K sub-steps of 16 per half-step; lane l
//     supplies row l % 32 and chunk 2*u + l / 32 of sub-step u, and holds
//     C[l % 32][8*g + 4*(l/32) + e] in accumulator element 4*g + e.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void *global_cptr;
typedef __attribute__((address_space(3))) void *lds_ptr;
// E is the storage type of A, Bt and C: __bf16 or _Float16 (same tiling, the
// MFMA of the matching type, round-to-nearest-even on the way out).
template <class E, int MF, class V, class Acc>
__device__ __forceinline__ Acc mfma_block(V b, V a, Acc c) {
  if constexpr (std::is_same<E, __bf16>::value) {
    if constexpr (MF == 16)
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, a, c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c, 0, 0, 0);
  } else {
    if constexpr (MF == 16)
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(b, a, c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c, 0, 0, 0);
  }
}

// EDGE = true: M and N need not be multiples of the tile and K only a multiple
// of 8.  Panel rows past the last row are read from the last row (their results
// are never stored); in the last K tile the 16-byte chunks past K are read from
// the start of their row instead and overwritten with zeros in LDS by the lane
// that fetched them, before the barrier that releases the tile; stores are
// masked.  Everything else, and the speed on whole tiles, is the same.
// EPI selects the epilogue of whole-tile builds: 0 stores each lane's four
// consecutive columns as they lie in the accumulators (8-byte stores, 32 bytes
// per row and instruction); 1 and 2 pass the tile through LDS, which the main
// loop no longer needs, so that eight lanes write one whole 128-byte row
// segment with 16-byte stores (2: non-temporal).  PRIO raises the wave's issue
// priority for the duration of each MFMA burst.  PROBE != 0 is a measurement
// build whose output is not the product: the loop with one part taken out
// (1: the MFMAs alone on the first K tile's fragments, no loads, LDS reads,
// waits or barriers; 2: no wait for the loads at the barrier; 3: no barrier;
// 4: no LDS operand reads; 5: no loads; 6: the loads fetch into a register
// instead of LDS; 7: the Bt operand blocks are fetched in MFMA layout straight
// into registers; 8: the tile is not stored; 9: two K tiles only, i.e. launch,
// prologue and epilogue without the loop between them).  STAGE sends a panel through registers (buffer load, then
// ds_write) instead of the load that writes LDS itself.  RS != 0 writes each
// half-step out in hand order, one fenced slot per MFMA: the LDS reads of the
// next half-step's operands over the first RS MFMAs, load v of the next tile
// but one before MFMA LF + v * LS; RS == 0 leaves the order to the compiler
// under sched_group_barrier hints.
template <class E, int BM, int BN, int WM, int WN, int MF, bool EDGE = false, int EPI = 0,
          bool PRIO = false, int PROBE = 0, int STAGE = 0, int RS = 0, int LF = 1, int LS = 2, int ORDER = 2>
__device__ __forceinline__ void gemm_tile_pipelined(
    const E *__restrict__ A, size_t lda, const E *__restrict__ Bt, size_t ldb,
    E *__restrict__ C, size_t ldc, int M, int N, int K) {
  typedef E ex8 __attribute__((ext_vector_type(8)));
  typedef E ex4 __attribute__((ext_vector_type(4)));
  constexpr int kWaves = WM * WN;
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int SH = 0;
  constexpr int kMI = kWaveM / MF;
  constexpr int kNI = kWaveN / MF;
  constexpr int kSub = MF == 16 ? 1 : 2;      // K sub-steps per half-step
  constexpr int kAccRegs = MF == 16 ? 4 : 16;
  typedef float acc_t __attribute__((ext_vector_type(kAccRegs)));
  constexpr int kALoads = BM / (8 * kWaves); // wave-level loads per panel
  constexpr int kBLoads = BN / (8 * kWaves);
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "panel rows");
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;
  constexpr int kMfma = kMI * kNI * kSub;  // MFMAs per half-step
  constexpr int kReads = (kMI + kNI) * kSub; // ds_read_b128 per half-step

  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  if constexpr (EDGE)
    tile_of_workgroup((M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
  else
    tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;
  const int KT = PROBE == 9 ? 2 : EDGE ? (K + kBK - 1) / kBK : K / kBK; // host guarantees KT >= 2
  // EDGE: whole 16-byte chunks of the last K tile that hold data (8 = all)
  const int tail_chunks = EDGE && K % kBK ? (K % kBK) / 8 : 8;

  // ---- global -> LDS ---------------------------------------------------------
  // load i of this wave fills panel rows (i*kWaves + wave)*8 .. +8
  const int ld_row = lane / 8, ld_pchunk = lane % 8;
  const E *a_src[kALoads];
  const E *b_src[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    const int row = EDGE ? min(tm * BM + r, M - 1) : tm * BM + r;
    a_src[i] = A + (size_t)row * lda + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    const int row = EDGE ? min(tn * BN + r, N - 1) : tn * BN + r;
    b_src[i] = Bt + (size_t)row * ldb + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
  // Whole-tile builds address the panels through buffer descriptors: the lane's
  // part of the address (its row among the eight of a wave-level load, its
  // swizzled chunk) is one 32-bit register per panel for the whole kernel, and
  // what changes from load to load and from K tile to K tile is a scalar
  // offset, so the loop spends no vector instruction on addresses (the 64-bit
  // pointer form needs two per load, sixteen per K tile, on the port the MFMAs
  // issue through).  Offsets stay below 2^31: the host checks 256 * ld * 2.
  constexpr bool BUF = !EDGE;
  u32x4 probe_sink = {0u, 0u, 0u, 0u};
  __amdgpu_buffer_rsrc_t a_rsrc, b_rsrc;
  int a_voff = 0, b_voff = 0;
  if constexpr (BUF) {
    a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<E *>(A + (size_t)tm * BM * lda), 0, (int)(((size_t)(BM - 1) * lda + K) * sizeof(E)),
        0x00020000);
    b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<E *>(Bt + (size_t)tn * BN * ldb), 0, (int)(((size_t)(BN - 1) * ldb + K) * sizeof(E)),
        0x00020000);
    const int chunk = ld_pchunk ^ swz<SH>(ld_row); // rows advance in eights: the swizzle is the lane's
    a_voff = (int)((ld_row * lda + chunk * 8) * sizeof(E));
    b_voff = (int)((ld_row * ldb + chunk * 8) * sizeof(E));
  }
  const int a_step = (int)(kWaves * 8 * lda * sizeof(E)), b_step = (int)(kWaves * 8 * ldb * sizeof(E));
  const int a_first = (int)(wave * 8 * lda * sizeof(E)), b_first = (int)(wave * 8 * ldb * sizeof(E));
  // logical chunk the lane fetches in load i (the swizzle depends on the row)
  auto chunk_of = [&](int i) { return ld_pchunk ^ swz<SH>((i * kWaves + wave) * 8 + ld_row); };
  // STAGE: bit 0 sends the A panel, bit 1 the B panel through registers (a
  // buffer load into a register quad, a 16-byte LDS write half a K tile later)
  // instead of the load that writes LDS by itself.
  constexpr bool kStageA = BUF && (STAGE & 1), kStageB = BUF && (STAGE & 2);
  constexpr int kStaged = (kStageA ? kALoads : 0) + (kStageB ? kBLoads : 0);
  constexpr int kDirect = kALoads + kBLoads - kStaged;
  u32x4 stage_a[kALoads], stage_b[kBLoads];
  auto write_staged = [&](int buf) {
    unsigned char *base = lds + buf * kStageBytes + wave * 1024 + lane * 16;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      if constexpr (kStageA)
        *reinterpret_cast<u32x4 *>(base + i * kWaves * 1024) = stage_a[i];
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      if constexpr (kStageB)
        *reinterpret_cast<u32x4 *>(base + kABytes + i * kWaves * 1024) = stage_b[i];
  };
  bool in_loop = false;  // PROBE 7 only
  auto issue_loads = [&](int kt, int buf) {
    const size_t k0 = (size_t)kt * kBK;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024;
    if constexpr (BUF && PROBE == 7) {
      // measurement build: inside the loop the A panel goes to LDS as always,
      // the B operand blocks are fetched in the layout the MFMA takes them
      // (sixteen rows of 64 bytes per load) into a register that nothing reads
      if (in_loop) {
        const int kbytes = (int)(k0 * sizeof(E));
#pragma unroll
        for (int i = 0; i < kALoads; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(base + i * kWaves * 1024), 16,
                                                   a_voff, a_first + i * a_step + kbytes, 0, 0);
        const uint64_t p = reinterpret_cast<uint64_t>(Bt + (size_t)tn * BN * ldb);
        const u32x4 rb = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu,
                          (uint32_t)(((size_t)(BN - 1) * ldb + K) * sizeof(E)), 0x00020000u};
        const int voff = (int)(((lane % 16) * ldb + (lane / 16) * 8) * sizeof(E));
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int j = 0; j < kNI; ++j) {
            const int so = (int)((wave_n + j * 16) * ldb * sizeof(E)) + h * 64 + kbytes;
            asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(probe_sink) : "v"(voff), "s"(rb), "s"(so));
          }
        return;
      }
    }
    if constexpr (BUF) {
      const int kbytes = (int)(k0 * sizeof(E));
      // panels that pass through registers first: their loads are the oldest
      // of the tile, so a wait that leaves the direct ones out covers them
#pragma unroll
      for (int i = 0; i < kALoads; ++i)
        if constexpr (kStageA)
          stage_a[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_voff, a_first + i * a_step + kbytes, 0);
#pragma unroll
      for (int i = 0; i < kBLoads; ++i)
        if constexpr (kStageB)
          stage_b[i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_voff, b_first + i * b_step + kbytes, 0);
#pragma unroll
      for (int i = 0; i < kALoads; ++i)
        if constexpr (!kStageA)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(base + i * kWaves * 1024), 16,
                                                   a_voff, a_first + i * a_step + kbytes, 0, 0);
#pragma unroll
      for (int i = 0; i < kBLoads; ++i)
        if constexpr (!kStageB)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc,
                                                   (lds_ptr)(base + kABytes + i * kWaves * 1024), 16,
                                                   b_voff, b_first + i * b_step + kbytes, 0, 0);
      return;
    }
    const bool tail = EDGE && kt == KT - 1 && tail_chunks < 8;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const E *src = a_src[i] + k0;
      if (tail && chunk_of(i) >= tail_chunks)
        src -= chunk_of(i) * 8;          // chunk 0 of the row: valid, zeroed later
      __builtin_amdgcn_global_load_lds((global_cptr)src,
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const E *src = b_src[i] + k0;
      if (tail && chunk_of(i) >= tail_chunks)
        src -= chunk_of(i) * 8;
      __builtin_amdgcn_global_load_lds(
          (global_cptr)src, (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0,
          0);
    }
  };
  // one wave-level load of K tile kt (A panel first, then B), whole-tile builds
  auto load_one = [&](int kt, int buf, int v) {
    if constexpr (BUF) {
      unsigned char *base = lds + buf * kStageBytes + wave * 1024;
      const int kbytes = (int)((size_t)kt * kBK * sizeof(E));
      if constexpr (PROBE == 6) {
        // measurement build: the same fetch into a register instead of LDS
        const bool isa = v < kALoads;
        const uint64_t p = reinterpret_cast<uint64_t>(isa ? A + (size_t)tm * BM * lda : Bt + (size_t)tn * BN * ldb);
        const size_t bytes = ((size_t)((isa ? BM : BN) - 1) * (isa ? lda : ldb) + K) * sizeof(E);
        const u32x4 r = {(uint32_t)p, (uint32_t)(p >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
        const int so = isa ? a_first + v * a_step + kbytes : b_first + (v - kALoads) * b_step + kbytes;
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(probe_sink) : "v"(isa ? a_voff : b_voff), "s"(r), "s"(so));
        return;
      }
      if (v < kALoads)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(base + v * kWaves * 1024), 16, a_voff,
                                                 a_first + v * a_step + kbytes, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr)(base + kABytes + (v - kALoads) * kWaves * 1024),
                                                 16, b_voff, b_first + (v - kALoads) * b_step + kbytes, 0, 0);
    }
  };
  // EDGE: after the last K tile has landed, the chunks past K become zeros
  auto zero_tail = [&](int buf) {
    if (!(EDGE && tail_chunks < 8))
      return;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024 + lane * 16;
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      if (chunk_of(i) >= tail_chunks)
        *reinterpret_cast<u32x4 *>(base + i * kWaves * 1024) = zero;
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      if (chunk_of(i) >= tail_chunks)
        *reinterpret_cast<u32x4 *>(base + kABytes + i * kWaves * 1024) = zero;
  };

  // ---- LDS -> operand registers ------------------------------------------------
  // lane l supplies row l % MF; its chunk in half-step h, sub-step u is
  // 4*h + (kSub == 1 ? l / 16 : 2*u + l / 32)
  const int lrow = lane % MF, lchunk = lane / MF;
  const int lswz = swz<SH>(lrow);
  int a_off[kMI], b_off[kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
    a_off[i] = (wave_m + i * MF + lrow) * kRowBytes;
#pragma unroll
  for (int i = 0; i < kNI; ++i)
    b_off[i] = kABytes + (wave_n + i * MF + lrow) * kRowBytes;
  int coff[2][kSub];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int u = 0; u < kSub; ++u)
      coff[h][u] = ((4 * h + (kSub == 1 ? lchunk : 2 * u + lchunk)) ^ lswz) * 16;

  ex8 fa[2][kSub][kMI], fb[2][kSub][kNI];
  auto read_frags = [&](int buf, int ks, auto slot) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int u = 0; u < kSub; ++u) {
      const unsigned char *base = lds + buf * kStageBytes + (ks ? coff[1][u] : coff[0][u]);
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        if (!(PROBE == 7 && in_loop))
          fb[S][u][j] = *reinterpret_cast<const ex8 *>(base + b_off[j]);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
        fa[S][u][i] = *reinterpret_cast<const ex8 *>(base + a_off[i]);
    }
  };

  acc_t acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int e = 0; e < kAccRegs; ++e)
        acc[i][j][e] = 0.f;
  auto mma = [&](auto slot) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int u = 0; u < kSub; ++u)
#pragma unroll
      for (int i = 0; i < kMI; ++i)
#pragma unroll
        for (int j = 0; j < kNI; ++j) {
          acc[i][j] = mfma_block<E, MF>(fb[S][u][j], fa[S][u][i], acc[i][j]);
        }
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;
  // RS builds write the order of a half-step out by hand, one fenced slot per
  // MFMA: LDS read r of the next half-step's operands goes before MFMA
  // r * S / kReads (S = number of MFMAs the reads are spread over), the loads
  // of K tile kt before the odd MFMAs from the second on.  Fragments are read
  // in the order the MFMAs take them (Bt blocks, then A blocks), so the waits
  // the compiler puts in front of each MFMA are for its own operands only.
  auto half_step = [&](auto use, auto fill, auto spread, auto rfirst, auto lfirst, int rbuf, int rks, bool do_read,
                       bool do_load, int kt, int lbuf) {
    constexpr int U = decltype(use)::value;
    constexpr int F = decltype(fill)::value;
    constexpr int S = decltype(spread)::value;
    constexpr int RF = decltype(rfirst)::value;
    constexpr int LFv = decltype(lfirst)::value;
    static_assert(kSub == 1, "written for the 16 x 16 x 32 blocks");
    static_assert(LFv + (kALoads + kBLoads - 1) * LS < kMfma, "every load has its MFMA");
    static_assert(RF + (kReads - 1) * S / kReads < kMfma, "every LDS read has its MFMA");
    const unsigned char *rbase = lds + rbuf * kStageBytes + (rks ? coff[1][0] : coff[0][0]);
#pragma unroll
    for (int slot = 0; slot < kMI * kNI; ++slot) {
      {
        // ORDER 0: the four Bt blocks under one A block, then the next A block;
        // 1: the eight A blocks under one Bt block; 2: as 0 in a serpentine (every
        // other A block takes the Bt blocks in reverse: consecutive MFMAs then
        // always share an operand; 1 % faster than 0, measured)
        const int i = ORDER == 1 ? slot % kMI
                      : ORDER == 3 ? ((slot / kMI) % 2 ? kMI - 1 - slot % kMI : slot % kMI)
                                   : slot / kNI;
        const int j = (ORDER == 1 || ORDER == 3) ? slot / kMI
                      : ORDER == 2 && (slot / kNI) % 2 ? kNI - 1 - slot % kNI
                                                       : slot % kNI;
        if (do_read) {
#pragma unroll
          for (int r = 0; r < kReads; ++r)
            if (RF + r * S / kReads == slot) {
              if (r < kNI)
                fb[F][0][r] = *reinterpret_cast<const ex8 *>(rbase + b_off[r]);
              else
                fa[F][0][r - kNI] = *reinterpret_cast<const ex8 *>(rbase + a_off[r - kNI]);
            }
        }
        if (do_load && slot >= LFv && (slot - LFv) % LS == 0 && (slot - LFv) / LS < kALoads + kBLoads)
          load_one(kt, lbuf, (slot - LFv) / LS);
        acc[i][j] = mfma_block<E, MF>(fb[U][0][j], fa[U][0][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // Order inside a half-step: one LDS read per MFMA from the start, so the last
  // read is out after kReads MFMAs and has the rest of the sequence to land;
  // the global->LDS loads follow, one per MFMA.
  auto interleave = [&](auto vmem, auto dswrites, auto spread) {
    constexpr int V = decltype(vmem)::value;
    constexpr int D = decltype(dswrites)::value;
    constexpr int S = decltype(spread)::value;
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      if constexpr (S == 0) {
        constexpr int kVFirst = kMfma >= kReads + V + D ? kReads : 0;
        if (i < kReads)
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
        if (i >= kVFirst && i - kVFirst < V)
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
        if (i >= kVFirst + V && i - kVFirst - V < D)
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // DS write
      } else {
        // LDS reads evenly over the first S MFMAs (read r before MFMA
        // r * S / kReads), the loads before the odd MFMAs from the second on
#pragma unroll
        for (int r = 0; r < kReads; ++r)
          if (r * S / kReads == i)
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (i % 2 == 1 && i / 2 < V)
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        if (i % 2 == 0 && i / 2 < D)
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
    }
  };
  using NoVmem = std::integral_constant<int, 0>;
  using WithVmem = std::integral_constant<int, PROBE == 7 ? kALoads + 2 * kNI : kALoads + kBLoads>;
  using NoWrites = std::integral_constant<int, 0>;
  using WithWrites = std::integral_constant<int, kStaged>;
  // reads of the even half-step are the last of their buffer and have to be
  // back before the barrier: they stop a quarter of the MFMAs earlier
  using SpreadEven = std::integral_constant<int, RS == 0 ? 0 : (RS < kMfma * 3 / 4 ? RS : kMfma * 3 / 4)>;
  using SpreadOdd = std::integral_constant<int, RS>;

  issue_loads(0, 0);
  if constexpr (kStaged != 0) {
    write_staged(0);  // the compiler waits for the registers
    issue_loads(1, 1);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kALoads + kBLoads, 0));
  } else {
    issue_loads(1, 1);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kALoads + kBLoads, kNoLgkm));
  }
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, Slot0{});

  auto tile_step = [&](int t, auto load_next2, auto read_next) {
    constexpr bool LOAD = decltype(load_next2)::value;
    constexpr bool READ = decltype(read_next)::value;
    using RFirst = std::integral_constant<int, 0>;
    using LFirst = std::integral_constant<int, LF>;
    static_assert(RS == 0 || kStaged == 0, "the hand-ordered half-steps have no register-staged panels");
    // the step before the last: the last tile has landed at its barrier
    constexpr bool ZERO = EDGE && !LOAD && READ;
    const int buf = t & 1;
    if constexpr (RS != 0) {
      // every read was out a quarter of a half-step ago or earlier
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
      __builtin_amdgcn_sched_barrier(0);
      half_step(Slot0{}, Slot1{}, SpreadEven{}, RFirst{}, LFirst{}, buf, 1, PROBE != 4, false, 0, 0);
      __builtin_amdgcn_s_waitcnt(PROBE == 2 ? waitcnt_imm(kNoVm, 0) : waitcnt_imm(0, 0));
      if constexpr (PROBE != 3)
        __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      half_step(Slot1{}, Slot0{}, SpreadOdd{}, RFirst{}, LFirst{}, buf ^ 1, 0, READ && PROBE != 4,
                LOAD && PROBE != 5, t + 2, buf);
      return;
    }
    // even half-step: consume slot 0 (requested a whole half-step ago, so the
    // wait is free and makes the later waits exact), fetch slot 1
    if constexpr (RS == 0)
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PROBE != 4)
      read_frags(buf, 1, Slot1{});
    if constexpr (PRIO)
      __builtin_amdgcn_s_setprio(1);
    // staged panels of tile t + 1 (requested a K tile ago) go to the buffer
    // that the barrier of the previous step released
    if constexpr (READ && kStaged != 0)
      write_staged(buf ^ 1);
    mma(Slot0{});
    if constexpr (READ)
      interleave(NoVmem{}, WithWrites{}, SpreadEven{});
    else
      interleave(NoVmem{}, NoWrites{}, SpreadEven{});
    if constexpr (PRIO)
      __builtin_amdgcn_s_setprio(0);
    // odd half-step; the fences keep the MFMAs above on this side of the wait
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PROBE == 2)
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    if constexpr (ZERO) {
      zero_tail(buf ^ 1);
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    }
    if constexpr (PROBE != 3)
      __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (LOAD && PROBE != 5)
      issue_loads(t + 2, buf);
    if constexpr (READ && PROBE != 4)
      read_frags(buf ^ 1, 0, Slot0{});
    if constexpr (PRIO)
      __builtin_amdgcn_s_setprio(1);
    mma(Slot1{});
    if constexpr (LOAD && READ)
      interleave(WithVmem{}, NoWrites{}, SpreadOdd{});
    else if constexpr (READ)
      interleave(NoVmem{}, NoWrites{}, SpreadOdd{});
    if constexpr (PRIO)
      __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (PROBE == 7) {
    read_frags(0, 1, Slot1{});
    in_loop = true;
  }
  if constexpr (PROBE == 1) {
    read_frags(0, 1, Slot1{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    for (int t = 0; t < KT; ++t) {
      mma(Slot0{});
      mma(Slot1{});
    }
  } else {
    if constexpr (PROBE == 4)
      read_frags(0, 1, Slot1{});
    int t = 0;
    for (; t < KT - 2; ++t)
      tile_step(t, std::true_type{}, std::true_type{});
    tile_step(t, std::false_type{}, std::true_type{});
    tile_step(t + 1, std::false_type{}, std::false_type{});
  }

  if constexpr (PROBE == 6 || PROBE == 7) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("" ::"v"(probe_sink));
  }
  // ---- epilogue ------------------------------------------------------------------
  if constexpr (EPI != 0 && !EDGE && MF == 16) {
    // Through LDS: the wave's kWaveM x kWaveN tile as rows of kWaveN elements,
    // 16-byte chunk c of row r kept at chunk c ^ (r & 7) (the writes of sixteen
    // rows at one column then spread over the banks); read back eight lanes to
    // a row.  Every wave uses a region of its own, but the stage buffers it
    // lies in may still be read by slower waves: one barrier first.
    constexpr int kRowB = kWaveN * (int)sizeof(E);   // bytes of a wave's row of C: 128 or 256
    constexpr int kCPR = kRowB / 16;                  // 16-byte chunks per row
    static_assert(kCPR == 8 || kCPR == 16, "a wave row is eight or sixteen 16-byte chunks");
    static_assert(kWaves * kWaveM * kRowB <= 2 * kStageBytes, "the tile fits the stage buffers");
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_s_barrier();
    unsigned char *mine = lds + wave * (kWaveM * kRowB);
#pragma unroll
    for (int i = 0; i < kMI; ++i)
#pragma unroll
      for (int j = 0; j < kNI; ++j) {
        ex4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (E)acc[i][j][e];
        const int r = i * 16 + lrow;
        const int chunk = 2 * j + lchunk / 2;
        *reinterpret_cast<ex4 *>(mine + r * kRowB + ((chunk ^ (r & (kCPR - 1))) * 16) + (lchunk % 2) * 8) = o;
      }
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    const int rr = lane / kCPR, pc = lane % kCPR;
#pragma unroll
    for (int r0 = 0; r0 < kWaveM; r0 += kWave / kCPR) {
      const int r = r0 + rr;
      const u32x4 v = *reinterpret_cast<const u32x4 *>(mine + r * kRowB + pc * 16);
      E *dst = C + (size_t)(tm * BM + wave_m + r) * ldc + tn * BN + wave_n + ((pc ^ (r & (kCPR - 1))) * 8);
      if constexpr (PROBE == 8) {
        if (v[0] == 0x7fc07fc1u) // (never: keeps the read of the tile alive)
          *reinterpret_cast<u32x4 *>(dst) = v;
      } else if constexpr (EPI == 2)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst));
      else
        *reinterpret_cast<u32x4 *>(dst) = v;
    }
    return;
  }
  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lchunk * 4;
  const bool vec_c = !EDGE || (ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 7) == 0);
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    E *crow = C + (size_t)(m_base + i * MF) * ldc + n_base;
    if (EDGE && m_base + i * MF >= M)
      continue;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < kAccRegs / 4; ++g) {
        ex4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (E)acc[i][j][4 * g + e];
        const int n = n_base + j * MF + g * 8;
        if (!EDGE || (vec_c && n + 3 < N)) {
          *reinterpret_cast<ex4 *>(crow + j * MF + g * 8) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N)
              crow[j * MF + g * 8 + e] = o[e];
        }
      }
    }
  }
}
} // namespace

#define HCAMD_GEMM_P(NAME, E, BM, BN, WM, WN, MF)                              \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const E *A, size_t lda, const E *Bt, size_t ldb, E *C, size_t ldc,       \
      int M, int N, int K) {                                                   \
    gemm_tile_pipelined<E, BM, BN, WM, WN, MF>(A, lda, Bt, ldb, C, ldc, M, N,  \
                                               K);                             \
  }
#define HCAMD_GEMM_PE(NAME, E, BM, BN, WM, WN, MF)                             \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const E *A, size_t lda, const E *Bt, size_t ldb, E *C, size_t ldc,       \
      int M, int N, int K) {                                                   \
    gemm_tile_pipelined<E, BM, BN, WM, WN, MF, true>(A, lda, Bt, ldb, C, ldc,  \
                                                     M, N, K);                 \
  }
#define HCAMD_GEMM_PX(NAME, E, BM, BN, WM, WN, MF, EPI, PRIO, PROBE)             \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const E *A, size_t lda, const E *Bt, size_t ldb, E *C, size_t ldc,       \
      int M, int N, int K) {                                                   \
    gemm_tile_pipelined<E, BM, BN, WM, WN, MF, false, EPI, PRIO, PROBE>(       \
        A, lda, Bt, ldb, C, ldc, M, N, K);                                     \
  }
#define HCAMD_GEMM_PS(NAME, E, BM, BN, WM, WN, MF, STAGE, RS, LF, LS)          \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const E *A, size_t lda, const E *Bt, size_t ldb, E *C, size_t ldc,       \
      int M, int N, int K) {                                                   \
    gemm_tile_pipelined<E, BM, BN, WM, WN, MF, false, 2, false, 0, STAGE, RS,  \
                        LF, LS>(A, lda, Bt, ldb, C, ldc, M, N, K);             \
  }
// the default 256 x 256 kernel's loop with one part taken out (PROBE)
#define HCAMD_GEMM_PZ(NAME, PROBE)                                             \
  extern "C" __global__ __launch_bounds__(512) void NAME(                      \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_pipelined<__bf16, 256, 256, 2, 4, 16, false, 2, false, PROBE, 0, \
                        16, 1, 4>(A, lda, Bt, ldb, C, ldc, M, N, K);           \
  }
// the default whole-tile kernels: LDS-staged epilogue with non-temporal stores,
// hand-ordered half-steps (LDS reads over the first half of the MFMAs, the loads
// evenly over all of them)
HCAMD_GEMM_PS(hcamd_gemm_bf16_p256x256_w2x4, __bf16, 256, 256, 2, 4, 16, 0, 16, 1, 4)
HCAMD_GEMM_PS(hcamd_gemm_bf16_p128x128_w2x2, __bf16, 128, 128, 2, 2, 16, 0, 8, 1, 2)
HCAMD_GEMM_PS(hcamd_gemm_f16_p256x256_w2x4, _Float16, 256, 256, 2, 4, 16, 0, 16, 1, 4)
HCAMD_GEMM_PS(hcamd_gemm_f16_p128x128_w2x2, _Float16, 128, 128, 2, 2, 16, 0, 8, 1, 2)
// for measurement: the order of a half-step left to the compiler under
// sched_group_barrier hints (one LDS read per MFMA from the start, the loads
// bunched behind them), with each epilogue / with raised priority; the loads
// early in hand-written order; the A panel staged through registers
HCAMD_GEMM_PX(hcamd_gemm_bf16_p256x256_w2x4_hinted, __bf16, 256, 256, 2, 4, 16, 2, false, 0)
HCAMD_GEMM_PX(hcamd_gemm_bf16_p256x256_w2x4_direct, __bf16, 256, 256, 2, 4, 16, 0, false, 0)
HCAMD_GEMM_PX(hcamd_gemm_bf16_p256x256_w2x4_lds, __bf16, 256, 256, 2, 4, 16, 1, false, 0)
HCAMD_GEMM_PX(hcamd_gemm_bf16_p256x256_w2x4_prio, __bf16, 256, 256, 2, 4, 16, 2, true, 0)
HCAMD_GEMM_PS(hcamd_gemm_bf16_p256x256_w2x4_loads_early, __bf16, 256, 256, 2, 4, 16, 0, 16, 1, 2)
HCAMD_GEMM_PS(hcamd_gemm_bf16_p256x256_w2x4_stage_a, __bf16, 256, 256, 2, 4, 16, 1, 0, 1, 2)
// four waves with 128 x 128 each (one wave per SIMD, the accumulators in the
// 256 AGPRs): a third less LDS operand traffic, the same speed within noise
// (plain MFMA order: the serpentine costs this build 30 %)
extern "C" __global__ __launch_bounds__(256) void hcamd_gemm_bf16_p256x256_w2x2(
    const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C, size_t ldc, int M, int N, int K) {
  gemm_tile_pipelined<__bf16, 256, 256, 2, 2, 16, false, 2, false, 0, 0, 24, 1, 4, 0>(A, lda, Bt, ldb, C, ldc, M,
                                                                                    N, K);
}
// measurement builds whose output is not the product: compiled only into a
// library built with `python -m hc_amd.build --probes`
#ifdef HCAMD_PROBES
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_mfma_only, 1)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_no_vmwait, 2)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_no_barrier, 3)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_no_ldsread, 4)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_no_loads, 5)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_loads_to_regs, 6)
HCAMD_GEMM_PX(hcamd_gemm_bf16_probe_b_direct, __bf16, 256, 256, 2, 4, 16, 2, false, 7)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_no_stores, 8)
HCAMD_GEMM_PZ(hcamd_gemm_bf16_probe_two_tiles, 9)
// other hand orders of the four-wave shape (these do compute the product; they are
// here because only measurements select them): LDS reads over the first 48 MFMAs
// of a half-step's 64; a load every second MFMA; the eight A blocks under one Bt block
#define HCAMD_GEMM_W2X2(NAME, RS, LF, LS, ORDER)                                \
  extern "C" __global__ __launch_bounds__(256) void NAME(                       \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,     \
      size_t ldc, int M, int N, int K) {                                        \
    gemm_tile_pipelined<__bf16, 256, 256, 2, 2, 16, false, 2, false, 0, 0, RS,  \
                        LF, LS, ORDER>(A, lda, Bt, ldb, C, ldc, M, N, K);       \
  }
HCAMD_GEMM_W2X2(hcamd_gemm_bf16_probe_w2x2_reads48, 48, 1, 4, 0)
HCAMD_GEMM_W2X2(hcamd_gemm_bf16_probe_w2x2_loads2, 24, 1, 2, 0)
HCAMD_GEMM_W2X2(hcamd_gemm_bf16_probe_w2x2_a_inner, 24, 1, 4, 1)
// the bare MFMA stream with the accumulators stored straight from registers, in
// 16 x 16 x 32 and in 32 x 32 x 16 blocks (half the operand registers read per
// multiply-add): what the block shape alone does to the clock
HCAMD_GEMM_PX(hcamd_gemm_bf16_probe_mfma16_direct, __bf16, 256, 256, 2, 4, 16, 0, false, 1)
HCAMD_GEMM_PX(hcamd_gemm_bf16_probe_mfma32_direct, __bf16, 256, 256, 2, 4, 32, 0, false, 1)
#endif
HCAMD_GEMM_PE(hcamd_gemm_bf16_p256x256_w2x4_edge, __bf16, 256, 256, 2, 4, 16)
HCAMD_GEMM_PE(hcamd_gemm_f16_p256x256_w2x4_edge, _Float16, 256, 256, 2, 4, 16)
HCAMD_GEMM_PE(hcamd_gemm_bf16_p128x128_w2x2_edge, __bf16, 128, 128, 2, 2, 16)
HCAMD_GEMM_PE(hcamd_gemm_f16_p128x128_w2x2_edge, _Float16, 128, 128, 2, 2, 16)
HCAMD_GEMM_P(hcamd_gemm_bf16_p256x256_w4x2, __bf16, 256, 256, 4, 2, 16)
HCAMD_GEMM_P(hcamd_gemm_bf16_p256x128_w2x2, __bf16, 256, 128, 2, 2, 16)
HCAMD_GEMM_P(hcamd_gemm_bf16_p32_256x256_w2x4, __bf16, 256, 256, 2, 4, 32)
HCAMD_GEMM_P(hcamd_gemm_bf16_p32_256x256_w4x2, __bf16, 256, 256, 4, 2, 32)

#define HCAMD_GEMM(NAME, BM, BN, WM, WN, SH)                                   \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(             \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile<BM, BN, WM, WN, SH>(A, lda, Bt, ldb, C, ldc, M, N, K);           \
  }

HCAMD_GEMM(hcamd_gemm_bf16_256x256_w2x4_s0, 256, 256, 2, 4, 0)
HCAMD_GEMM(hcamd_gemm_bf16_256x256_w2x4_s1, 256, 256, 2, 4, 1)
HCAMD_GEMM(hcamd_gemm_bf16_256x256_w4x2_s0, 256, 256, 4, 2, 0)
HCAMD_GEMM(hcamd_gemm_bf16_128x128_w2x2_s0, 128, 128, 2, 2, 0)
HCAMD_GEMM(hcamd_gemm_bf16_256x128_w2x2_s0, 256, 128, 2, 2, 0)

// General kernel: any M, N, K, any leading dimensions and alignment.  A
// 64 x 64 tile of C per workgroup, a 4 x 4 block per thread, fp32 FMAs on
// LDS-staged 64 x 16 panels, every access bounds-checked.  Correct everywhere,
// fast nowhere; it exists for the shapes the tiled kernel does not take.
template <class E>
__device__ __forceinline__ void gemm_general(const E *A, size_t lda, const E *Bt,
                                             size_t ldb, E *C, size_t ldc, int M,
                                             int N, int K) {
  constexpr int T = 64, KB = 16;
  __shared__ float sa[KB][T + 1];
  __shared__ float sb[KB][T + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += KB) {
    for (int e = threadIdx.x; e < T * KB; e += 256) {
      const int r = e / KB, k = e % KB;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + k;
      sa[k][r] = (gm < M && gk < K) ? (float)A[(size_t)gm * lda + gk] : 0.f;
      sb[k][r] = (gn < N && gk < K) ? (float)Bt[(size_t)gn * ldb + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < KB; ++k) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = sa[k][ty * 4 + i];
        bv[i] = sb[k][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gm = m0 + ty * 4 + i, gn = n0 + tx * 4 + j;
      if (gm < M && gn < N)
        C[(size_t)gm * ldc + gn] = (E)acc[i][j];
    }
}

extern "C" __global__ __launch_bounds__(256) void hcamd_gemm_bf16_general(
    const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,
    size_t ldc, int M, int N, int K) {
  gemm_general<__bf16>(A, lda, Bt, ldb, C, ldc, M, N, K);
}
extern "C" __global__ __launch_bounds__(256) void hcamd_gemm_f16_general(
    const _Float16 *A, size_t lda, const _Float16 *Bt, size_t ldb, _Float16 *C,
    size_t ldc, int M, int N, int K) {
  gemm_general<_Float16>(A, lda, Bt, ldb, C, ldc, M, N, K);
}
