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
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void *global_cptr;
typedef __attribute__((address_space(3))) void *lds_ptr;

template <int BM, int BN, int WM, int WN, int SH>
__device__ __forceinline__ void gemm_tile_pipelined(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
  constexpr int kWaves = WM * WN;
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int kMI = kWaveM / 16;
  constexpr int kNI = kWaveN / 16;
  constexpr int kALoads = BM / (8 * kWaves); // wave-level loads per panel
  constexpr int kBLoads = BN / (8 * kWaves);
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "panel rows");
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;
  constexpr int kMfma = kMI * kNI;     // MFMAs per half-step
  constexpr int kReads = kMI + kNI;    // ds_read_b128 per half-step

  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  // ---- global -> LDS ---------------------------------------------------------
  // load i of this wave fills panel rows (i*kWaves + wave)*8 .. +8
  const int ld_row = lane / 8, ld_pchunk = lane % 8;
  const __bf16 *a_src[kALoads];
  const __bf16 *b_src[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    a_src[i] = A + (size_t)(tm * BM + r) * lda + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    b_src[i] = Bt + (size_t)(tn * BN + r) * ldb + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
  auto issue_loads = [&](int kt, int buf) {
    const size_t k0 = (size_t)kt * kBK;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      __builtin_amdgcn_global_load_lds((global_cptr)(a_src[i] + k0),
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_cptr)(b_src[i] + k0),
          (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0, 0);
  };

  // ---- LDS -> operand registers ------------------------------------------------
  const int lrow = lane % 16, lchunk = lane / 16;
  const int lswz = swz<SH>(lrow);
  int a_off[kMI], b_off[kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
    a_off[i] = (wave_m + i * 16 + lrow) * kRowBytes;
#pragma unroll
  for (int i = 0; i < kNI; ++i)
    b_off[i] = kABytes + (wave_n + i * 16 + lrow) * kRowBytes;
  const int coff0 = ((0 + lchunk) ^ lswz) * 16;
  const int coff1 = ((4 + lchunk) ^ lswz) * 16;

  bf16x8 fa[2][kMI], fb[2][kNI];
  auto read_frags = [&](int buf, int ks, auto slot) {
    constexpr int S = decltype(slot)::value;
    const unsigned char *base = lds + buf * kStageBytes + (ks ? coff1 : coff0);
#pragma unroll
    for (int j = 0; j < kNI; ++j)
      fb[S][j] = *reinterpret_cast<const bf16x8 *>(base + b_off[j]);
#pragma unroll
    for (int i = 0; i < kMI; ++i)
      fa[S][i] = *reinterpret_cast<const bf16x8 *>(base + a_off[i]);
  };

  f32x4 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto mma = [&](auto slot) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int i = 0; i < kMI; ++i)
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            fb[S][j], fa[S][i], acc[i][j], 0, 0, 0);
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;

  // Order inside a half-step: one LDS read per MFMA from the start, so the last
  // read is out after kReads MFMAs and has the rest of the sequence to land;
  // the global->LDS loads follow, one per MFMA.
  auto interleave = [&](auto vmem) {
    constexpr int V = decltype(vmem)::value;
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      if (i < kReads)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
      else if (i - kReads < V)
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
    }
  };
  using NoVmem = std::integral_constant<int, 0>;
  using WithVmem = std::integral_constant<int, kALoads + kBLoads>;

  const int KT = K / kBK; // host guarantees KT >= 2
  issue_loads(0, 0);
  issue_loads(1, 1);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(kALoads + kBLoads, kNoLgkm));
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, Slot0{});

  auto tile_step = [&](int t, auto load_next2, auto read_next) {
    constexpr bool LOAD = decltype(load_next2)::value;
    constexpr bool READ = decltype(read_next)::value;
    const int buf = t & 1;
    // even half-step: consume slot 0 (requested a whole half-step ago, so the
    // wait is free and makes the later waits exact), fetch slot 1
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 1, Slot1{});
    mma(Slot0{});
    interleave(NoVmem{});
    // odd half-step; the fences keep the MFMAs above on this side of the wait
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (LOAD)
      issue_loads(t + 2, buf);
    if constexpr (READ)
      read_frags(buf ^ 1, 0, Slot0{});
    mma(Slot1{});
    if constexpr (LOAD && READ)
      interleave(WithVmem{});
    else if constexpr (READ)
      interleave(NoVmem{});
    __builtin_amdgcn_sched_barrier(0);
  };
  int t = 0;
  for (; t < KT - 2; ++t)
    tile_step(t, std::true_type{}, std::true_type{});
  tile_step(t, std::false_type{}, std::true_type{});
  tile_step(t + 1, std::false_type{}, std::false_type{});

  // ---- epilogue ------------------------------------------------------------------
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
// The pipelined kernel again, with the MFMA block size as a parameter: MF = 32
// uses v_mfma_f32_32x32x16_bf16 (two K sub-steps of 16 per half-step), half as
// many matrix instructions for the same operand reads.  Same barriers, same
// load schedule as gemm_tile_pipelined.
// ---------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN, int MF, int ABL = 0>
__device__ __forceinline__ void gemm_tile_pipelined_mf(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
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
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  // ---- global -> LDS ---------------------------------------------------------
  // load i of this wave fills panel rows (i*kWaves + wave)*8 .. +8
  const int ld_row = lane / 8, ld_pchunk = lane % 8;
  const __bf16 *a_src[kALoads];
  const __bf16 *b_src[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    a_src[i] = A + (size_t)(tm * BM + r) * lda + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    b_src[i] = Bt + (size_t)(tn * BN + r) * ldb + ((ld_pchunk ^ swz<SH>(r)) * 8);
  }
  auto issue_loads = [&](int kt, int buf) {
    const size_t k0 = (size_t)kt * kBK;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      __builtin_amdgcn_global_load_lds((global_cptr)(a_src[i] + k0),
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_cptr)(b_src[i] + k0),
          (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0, 0);
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

  bf16x8 fa[2][kSub][kMI], fb[2][kSub][kNI];
  auto read_frags = [&](int buf, int ks, auto slot) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int u = 0; u < kSub; ++u) {
      const unsigned char *base = lds + buf * kStageBytes + (ks ? coff[1][u] : coff[0][u]);
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        fb[S][u][j] = *reinterpret_cast<const bf16x8 *>(base + b_off[j]);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
        fa[S][u][i] = *reinterpret_cast<const bf16x8 *>(base + a_off[i]);
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
          if constexpr (MF == 16)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                fb[S][u][j], fa[S][u][i], acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                fb[S][u][j], fa[S][u][i], acc[i][j], 0, 0, 0);
        }
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;

  // Order inside a half-step: one LDS read per MFMA from the start, so the last
  // read is out after kReads MFMAs and has the rest of the sequence to land;
  // the global->LDS loads follow, one per MFMA.
  auto interleave = [&](auto vmem) {
    constexpr int V = decltype(vmem)::value;
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      constexpr int kVFirst = kMfma >= kReads + V ? kReads : 0;
      if (i < kReads)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
      if (i >= kVFirst && i - kVFirst < V)
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
    }
  };
  using NoVmem = std::integral_constant<int, 0>;
  using WithVmem = std::integral_constant<int, kALoads + kBLoads>;

  const int KT = K / kBK; // host guarantees KT >= 2
  issue_loads(0, 0);
  issue_loads(1, 1);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(kALoads + kBLoads, kNoLgkm));
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, Slot0{});

  auto tile_step = [&](int t, auto load_next2, auto read_next) {
    constexpr bool LOAD = decltype(load_next2)::value;
    constexpr bool READ = decltype(read_next)::value;
    const int buf = t & 1;
    // even half-step: consume slot 0 (requested a whole half-step ago, so the
    // wait is free and makes the later waits exact), fetch slot 1
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 1, Slot1{});
    mma(Slot0{});
    interleave(NoVmem{});
    // odd half-step; the fences keep the MFMAs above on this side of the wait
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (LOAD)
      issue_loads(t + 2, buf);
    if constexpr (READ)
      read_frags(buf ^ 1, 0, Slot0{});
    mma(Slot1{});
    if constexpr (LOAD && READ)
      interleave(WithVmem{});
    else if constexpr (READ)
      interleave(NoVmem{});
    __builtin_amdgcn_sched_barrier(0);
  };
  int t = 0;
  for (; t < KT - 2; ++t)
    tile_step(t, std::true_type{}, std::true_type{});
  tile_step(t, std::false_type{}, std::true_type{});
  tile_step(t + 1, std::false_type{}, std::false_type{});

  // ---- epilogue ------------------------------------------------------------------
  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lchunk * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * MF) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < kAccRegs / 4; ++g) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (__bf16)acc[i][j][4 * g + e];
        if constexpr (ABL & 16) // measurement only: no stores
          asm volatile("" ::"v"(o));
        else
          *reinterpret_cast<bf16x4 *>(crow + j * MF + g * 8) = o;
      }
    }
  }
}
// ---------------------------------------------------------------------------
// Pipelined kernel on v_mfma_f32_32x32x16_bf16.  A 32 x 32 output block per
// instruction halves the number of MFMA issues and of operand reads per flop
// compared with 16 x 16 x 32, and two independent accumulators already keep the
// matrix pipe full.  Operand layout: lane l supplies row l % 32 and the eight K
// values 8*(l/32) .. +7 of a 32 x 16 block, again one 16-byte chunk of a panel
// row.  With Bt first and A second, lane l holds C[m = l % 32][n = 8*g +
// 4*(l/32) + e] for accumulator element 4*g + e: four consecutive columns per
// group g.  K is walked in quarter-steps of 16; fragments of quarter-step q+1
// are fetched while the MFMAs of q run; the barrier sits at the start of the
// last quarter-step of each 64-wide tile.
// ---------------------------------------------------------------------------
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int BM, int BN, int WM, int WN>
__device__ __forceinline__ void gemm_tile_p32(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
  constexpr int kWaves = WM * WN;
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int kMI = kWaveM / 32;
  constexpr int kNI = kWaveN / 32;
  constexpr int kALoads = BM / (8 * kWaves);
  constexpr int kBLoads = BN / (8 * kWaves);
  static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "panel rows");
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;
  constexpr int kMfma = kMI * kNI;  // per quarter-step
  constexpr int kReads = kMI + kNI; // per quarter-step

  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  const int ld_row = lane / 8, ld_pchunk = lane % 8;
  const __bf16 *a_src[kALoads];
  const __bf16 *b_src[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    a_src[i] = A + (size_t)(tm * BM + r) * lda + ((ld_pchunk ^ swz<0>(r)) * 8);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    b_src[i] = Bt + (size_t)(tn * BN + r) * ldb + ((ld_pchunk ^ swz<0>(r)) * 8);
  }
  auto issue_loads = [&](int kt, int buf) {
    const size_t k0 = (size_t)kt * kBK;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      __builtin_amdgcn_global_load_lds((global_cptr)(a_src[i] + k0),
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_cptr)(b_src[i] + k0),
          (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0, 0);
  };

  const int lrow = lane % 32, lhalf = lane / 32;
  const int lswz = swz<0>(lrow);
  int a_off[kMI], b_off[kNI], coff[4];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
    a_off[i] = (wave_m + i * 32 + lrow) * kRowBytes;
#pragma unroll
  for (int i = 0; i < kNI; ++i)
    b_off[i] = kABytes + (wave_n + i * 32 + lrow) * kRowBytes;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    coff[q] = ((2 * q + lhalf) ^ lswz) * 16;

  bf16x8 fa[2][kMI], fb[2][kNI];
  auto read_frags = [&](int buf, int q, auto slot) {
    constexpr int S = decltype(slot)::value;
    const unsigned char *base = lds + buf * kStageBytes + coff[q];
#pragma unroll
    for (int j = 0; j < kNI; ++j)
      fb[S][j] = *reinterpret_cast<const bf16x8 *>(base + b_off[j]);
#pragma unroll
    for (int i = 0; i < kMI; ++i)
      fa[S][i] = *reinterpret_cast<const bf16x8 *>(base + a_off[i]);
  };

  f32x16 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        acc[i][j][e] = 0.f;
  auto mma = [&](auto slot) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int i = 0; i < kMI; ++i)
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            fb[S][j], fa[S][i], acc[i][j], 0, 0, 0);
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;

  // Order inside a quarter-step: all LDS reads for the next quarter-step go out
  // first, in one burst, so that they have the whole MFMA sequence (kMfma x 32
  // cycles) to land; the global->LDS loads are then spread between the MFMAs.
  auto interleave = [&](auto vmem, auto reads) {
    constexpr int V = decltype(vmem)::value;
    constexpr int R = decltype(reads)::value;
    constexpr int vper = (V + kMfma - 1) / kMfma;
    if (R > 0)
      __builtin_amdgcn_sched_group_barrier(0x100, R, 0);
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (i * vper < V)
        __builtin_amdgcn_sched_group_barrier(0x020, vper, 0);
    }
  };
  using None = std::integral_constant<int, 0>;
  using Reads = std::integral_constant<int, kReads>;
  using Vmem = std::integral_constant<int, kALoads + kBLoads>;

  const int KT = K / kBK; // host guarantees KT >= 2
  issue_loads(0, 0);
  issue_loads(1, 1);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(kALoads + kBLoads, kNoLgkm));
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, Slot0{});

  auto tile_step = [&](int t, auto load_next2, auto read_next) {
    constexpr bool LOAD = decltype(load_next2)::value;
    constexpr bool READ = decltype(read_next)::value;
    const int buf = t & 1;
    // The fragments of quarter-step 0 were requested a whole MFMA sequence
    // ago; stating that they have landed lets every later wait be counted
    // exactly instead of draining the queue.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 1, Slot1{});
    mma(Slot0{});
    interleave(None{}, Reads{});
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 2, Slot0{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, kReads)); // slot 1 landed
    __builtin_amdgcn_sched_barrier(0);
    mma(Slot1{});
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 3, Slot1{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, kReads)); // slot 0 landed
    __builtin_amdgcn_sched_barrier(0);
    mma(Slot0{});
    // Last quarter-step: the next tile must have landed, and this wave must be
    // done reading the current one, before anybody crosses the barrier.  The
    // scheduling fences keep the MFMAs above on this side of the wait, so the
    // reads just issued have had their full sequence to complete.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (READ)
      read_frags(buf ^ 1, 0, Slot0{});
    if constexpr (LOAD)
      issue_loads(t + 2, buf);
    mma(Slot1{});
    if constexpr (LOAD && READ)
      interleave(Vmem{}, Reads{});
    else if constexpr (READ)
      interleave(None{}, Reads{});
    __builtin_amdgcn_sched_barrier(0);
  };
  int t = 0;
  for (; t < KT - 2; ++t)
    tile_step(t, std::true_type{}, std::true_type{});
  tile_step(t, std::false_type{}, std::true_type{});
  tile_step(t + 1, std::false_type{}, std::false_type{});

  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lhalf * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * 32) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (__bf16)acc[i][j][4 * g + e];
        *reinterpret_cast<bf16x4 *>(crow + j * 32 + g * 8) = o;
      }
    }
  }
}
// ---------------------------------------------------------------------------
// Ping-pong kernel (32x32x16 MFMA).  The eight waves of a workgroup form two
// groups of four, one wave of each group on every SIMD.  Time is cut into
// phases that end in a workgroup barrier; a wave alternates between
//   M  memory phase:  fetch the operand fragments of one 32-wide K half-tile
//                     from LDS (and, in the first half, start the global->LDS
//                     loads of the next 64-wide tile), wait for the fragments;
//   C  compute phase: sixteen MFMAs on those fragments, nothing else.
// Group 1 passes one extra barrier at the start, so it always runs the phase
// that group 0 ran a barrier ago: on every SIMD one wave feeds the matrix pipe
// while the other uses the LDS and vector-memory pipes, instead of both
// competing for the same unit at the same moment.
//
// Tile t lives in LDS stage t & 1.  Its loads are issued in the M phases of
// the first half of tile t-1 - after the barrier that ends the last read of
// tile t-2 from the same stage - and are awaited (vmcnt(0)) before the barrier
// that ends each wave's last two phases of tile t-1, i.e. at least a full phase
// after they were issued.
// ---------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN>
__device__ __forceinline__ void gemm_tile_pingpong(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
  constexpr int kWaves = WM * WN;
  static_assert(kWaves == 8, "two groups of four waves");
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int kMI = kWaveM / 32;
  constexpr int kNI = kWaveN / 32;
  constexpr int kALoads = BM / (8 * kWaves);
  constexpr int kBLoads = BN / (8 * kWaves);
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;

  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  // waves w and w+4 share a SIMD: group = wave / 4
  const int group = wave / 4;
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  const int ld_row = lane / 8, ld_pchunk = lane % 8;
  const __bf16 *a_src[kALoads];
  const __bf16 *b_src[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    a_src[i] = A + (size_t)(tm * BM + r) * lda + ((ld_pchunk ^ swz<0>(r)) * 8);
  }
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int r = (i * kWaves + wave) * 8 + ld_row;
    b_src[i] = Bt + (size_t)(tn * BN + r) * ldb + ((ld_pchunk ^ swz<0>(r)) * 8);
  }
  auto issue_loads = [&](int kt, int buf) {
    const size_t k0 = (size_t)kt * kBK;
    unsigned char *base = lds + buf * kStageBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      __builtin_amdgcn_global_load_lds((global_cptr)(a_src[i] + k0),
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_cptr)(b_src[i] + k0),
          (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0, 0);
  };

  const int lrow = lane % 32, lhalf = lane / 32;
  const int lswz = swz<0>(lrow);
  int a_off[kMI], b_off[kNI], coff[4];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
    a_off[i] = (wave_m + i * 32 + lrow) * kRowBytes;
#pragma unroll
  for (int i = 0; i < kNI; ++i)
    b_off[i] = kABytes + (wave_n + i * 32 + lrow) * kRowBytes;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    coff[q] = ((2 * q + lhalf) ^ lswz) * 16;

  bf16x8 fa[2][kMI], fb[2][kNI]; // the two K quarter-steps of one half-tile
  auto read_half = [&](int buf, int h) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const unsigned char *base = lds + buf * kStageBytes + coff[2 * h + q];
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        fb[q][j] = *reinterpret_cast<const bf16x8 *>(base + b_off[j]);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
        fa[q][i] = *reinterpret_cast<const bf16x8 *>(base + a_off[i]);
    }
  };

  f32x16 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        acc[i][j][e] = 0.f;
  auto mma_half = [&]() {
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int i = 0; i < kMI; ++i)
#pragma unroll
        for (int j = 0; j < kNI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              fb[q][j], fa[q][i], acc[i][j], 0, 0, 0);
  };
  auto phase_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  const int KT = K / kBK;
  issue_loads(0, 0);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kNoLgkm));
  phase_end();
  if (group == 1)
    phase_end(); // group 1 runs one phase behind group 0

  for (int t = 0; t < KT; ++t) {
    const int buf = t & 1;
    // M, first half: start the next tile's loads, fetch fragments
    if (t + 1 < KT)
      issue_loads(t + 1, buf ^ 1);
    read_half(buf, 0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    phase_end();
    // C, first half
    __builtin_amdgcn_s_setprio(1);
    mma_half();
    __builtin_amdgcn_s_setprio(0);
    phase_end();
    // M, second half: fragments, then make sure this wave's loads have landed
    read_half(buf, 1);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    phase_end();
    // C, second half
    __builtin_amdgcn_s_setprio(1);
    mma_half();
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kNoLgkm));
    phase_end();
  }
  if (group == 0)
    phase_end(); // matches group 1's extra barrier

  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lhalf * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * 32) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (__bf16)acc[i][j][4 * g + e];
        *reinterpret_cast<bf16x4 *>(crow + j * 32 + g * 8) = o;
      }
    }
  }
}
// ---------------------------------------------------------------------------
// Register-staged kernel: four waves, one per SIMD, each owning a 128 x 128
// block of the 256 x 256 tile (sixteen 32 x 32 accumulators = 256 accumulation
// registers).  Compared with eight waves of 128 x 64 this reads a third less
// from LDS per flop, and no two waves ever compete for one SIMD's matrix pipe;
// all overlap comes from software pipelining inside the single instruction
// stream of a wave:
//   * K is walked in quarter-steps of 16 (sixteen MFMAs each).  The fragments of
//     quarter-step q+1 are read from LDS while the MFMAs of q run.
//   * The next tile's panels travel global -> registers during quarter-steps
//     0 and 1 (one 16-byte load per two MFMAs, never a burst), rest for a whole
//     quarter-step, and go registers -> LDS (other stage) in the first half of
//     quarter-step 3.
//   * One barrier per tile, in the middle of quarter-step 3: before it this
//     wave's LDS writes are complete and its reads of the current stage are
//     done; after it the next tile's first fragments are fetched under the
//     remaining eight MFMAs.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void gemm_tile_staged(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
  constexpr int BM = 256, BN = 256, WN = 2;
  constexpr int kThreads = 256;
  constexpr int kWaveM = 128, kWaveN = 128;
  constexpr int kMI = 4, kNI = 4;
  constexpr int kLoads = 8; // 16-byte chunks per thread per panel
  constexpr int kABytes = BM * kRowBytes;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;

  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  // global -> registers -> LDS: chunk id = tid + i*256: row = tid/8 + 32*i,
  // chunk = tid % 8; (row & 7) does not depend on i
  const int st_row = tid / 8, st_chunk = tid % 8;
  const __bf16 *a_src = A + (size_t)(tm * BM + st_row) * lda + st_chunk * 8;
  const __bf16 *b_src = Bt + (size_t)(tn * BN + st_row) * ldb + st_chunk * 8;
  const size_t a_step = 32 * lda, b_step = 32 * ldb;
  const int st_off = st_row * kRowBytes + ((st_chunk ^ swz<0>(st_row)) * 16);
  u32x4 a_reg[kLoads], b_reg[kLoads];

  // LDS -> fragments
  const int lrow = lane % 32, lhalf = lane / 32;
  const int lswz = swz<0>(lrow);
  const int a_off = (wave_m + lrow) * kRowBytes;
  const int b_off = kABytes + (wave_n + lrow) * kRowBytes;
  int coff[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    coff[q] = ((2 * q + lhalf) ^ lswz) * 16;

  bf16x8 fa[2][kMI], fb[2][kNI];
  auto read_frags = [&](int buf, int q, auto slot) {
    constexpr int S = decltype(slot)::value;
    const unsigned char *base = lds + buf * kStageBytes + coff[q];
#pragma unroll
    for (int j = 0; j < kNI; ++j)
      fb[S][j] = *reinterpret_cast<const bf16x8 *>(base + b_off + j * 32 * kRowBytes);
#pragma unroll
    for (int i = 0; i < kMI; ++i)
      fa[S][i] = *reinterpret_cast<const bf16x8 *>(base + a_off + i * 32 * kRowBytes);
  };

  f32x16 acc[kMI][kNI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kNI; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        acc[i][j][e] = 0.f;
  // rows [i0, i1) of the wave's accumulator grid
  auto mma_rows = [&](auto slot, int i0, int i1) {
    constexpr int S = decltype(slot)::value;
#pragma unroll
    for (int i = 0; i < kMI; ++i)
      if (i >= i0 && i < i1)
#pragma unroll
        for (int j = 0; j < kNI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              fb[S][j], fa[S][i], acc[i][j], 0, 0, 0);
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;

  auto load_a = [&](int kt) {
    const __bf16 *p = a_src + (size_t)kt * kBK;
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      a_reg[i] = *reinterpret_cast<const u32x4 *>(p + i * a_step);
  };
  auto load_b = [&](int kt) {
    const __bf16 *p = b_src + (size_t)kt * kBK;
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      b_reg[i] = *reinterpret_cast<const u32x4 *>(p + i * b_step);
  };
  auto store_stage = [&](int buf) {
    unsigned char *base = lds + buf * kStageBytes + st_off;
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      *reinterpret_cast<u32x4 *>(base + i * 32 * kRowBytes) = a_reg[i];
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      *reinterpret_cast<u32x4 *>(base + kABytes + i * 32 * kRowBytes) = b_reg[i];
  };
  const int KT = K / kBK; // host guarantees KT >= 2
  load_a(0);
  load_b(0);
  store_stage(0);
  load_a(1);
  load_b(1);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, Slot0{});

  auto tile_step = [&](int t, auto load_next2, auto has_next) {
    constexpr bool LOAD = decltype(load_next2)::value; // tile t+2 exists
    constexpr bool NEXT = decltype(has_next)::value;   // tile t+1 exists
    const int buf = t & 1;
    // ---- quarter-step 0: MFMAs on slot 0, fetch slot 1 -------------------
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_sched_barrier(0);
    read_frags(buf, 1, Slot1{});
    mma_rows(Slot0{}, 0, 4);
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- quarter-step 1 -------------------------------------------------------
    read_frags(buf, 2, Slot0{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 8));
    __builtin_amdgcn_sched_barrier(0);
    mma_rows(Slot1{}, 0, 4);
    __builtin_amdgcn_sched_barrier(0);
    // ---- quarter-step 2 -------------------------------------------------------
    read_frags(buf, 3, Slot1{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 8));
    __builtin_amdgcn_sched_barrier(0);
    mma_rows(Slot0{}, 0, 4);
    __builtin_amdgcn_sched_barrier(0);
    // ---- quarter-step 3, first half: registers -> LDS (other stage) ---------
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    if constexpr (NEXT)
      store_stage(buf ^ 1);
    mma_rows(Slot1{}, 0, 2);
    if constexpr (NEXT) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x200, 2, 0); // DS write
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(kNoVm, 0));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // ---- quarter-step 3, second half: next tile's first fragments, and the
    // first global loads of the tile after next ------------------------------
    if constexpr (NEXT)
      read_frags(buf ^ 1, 0, Slot0{});
    if constexpr (LOAD)
      load_a(t + 2);
    mma_rows(Slot1{}, 2, 4);
    if constexpr (NEXT)
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
    if constexpr (LOAD) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (LOAD)
      load_b(t + 2);
  };
  int t = 0;
  for (; t < KT - 2; ++t)
    tile_step(t, std::true_type{}, std::true_type{});
  tile_step(t, std::false_type{}, std::true_type{});
  tile_step(t + 1, std::false_type{}, std::false_type{});

  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lhalf * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * 32) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (__bf16)acc[i][j][4 * g + e];
        *reinterpret_cast<bf16x4 *>(crow + j * 32 + g * 8) = o;
      }
    }
  }
}
// ---------------------------------------------------------------------------
// Ring kernel.  256 x 256 tile, K walked in slices of 32, and a ring of SLOTS
// LDS slots of 32 KiB (A slice 256 x 32, then the B slice).  A slice is
// requested SLOTS-1 slices before its fragments are read, so a request that
// misses L2 has about three slices of MFMA time to come back instead of one;
// with only two 64-wide stages the slowest of a tile's 512 requests decides
// when the whole workgroup may go on.
//
//   step s:  wait until this wave's loads of slice s+1 have landed and its
//            fragment reads of slice s are complete; barrier; request slice
//            s+SLOTS into the slot slice s occupied; read the fragments of
//            slice s+1 into the other register set; MFMAs on slice s.
//
// A slice row is 32 bf16 = 64 bytes = four chunks; chunk c of row r sits at
// chunk position c ^ ((r >> 1) & 3), which makes the eight lanes served per
// clock by a 16-byte LDS read hit eight different 16-byte bank groups.  A
// wave-level direct load fills 1 KiB = 16 slice rows; lane l lands in row l/4,
// position l%4, and therefore fetches logical chunk (l%4) ^ ((l>>3) & 3).
// A 16 x 16 x 32 MFMA operand is exactly 16 slice rows.
// ---------------------------------------------------------------------------
template <int WM, int WN, int SLOTS, int MF, int ABL = 0, int SKEW = 0>
__device__ __forceinline__ void gemm_tile_ring(
    const __bf16 *__restrict__ A, size_t lda, const __bf16 *__restrict__ Bt,
    size_t ldb, __bf16 *__restrict__ C, size_t ldc, int M, int N, int K) {
  // MF = 16: v_mfma_f32_16x16x32_bf16, one K sub-step per slice.
  // MF = 32: v_mfma_f32_32x32x16_bf16, two K sub-steps of 16 per slice.
  // ABL (measurement only, results are wrong when non-zero) removes one part of
  // the steady-state loop: 1 global loads, 2 LDS reads, 4 MFMAs, 8 barriers.
  static_assert(MF == 16 || MF == 32, "MFMA block size");
  constexpr int BM = 256, BN = 256, BK = 32;
  constexpr int kRow = BK * 2; // bytes
  constexpr int kWaves = WM * WN;
  constexpr int kWaveM = BM / WM;
  constexpr int kWaveN = BN / WN;
  constexpr int kMI = kWaveM / MF;
  constexpr int kNI = kWaveN / MF;
  constexpr int kSub = MF == 16 ? 1 : 2;      // K sub-steps per slice
  constexpr int kAccRegs = MF == 16 ? 4 : 16; // fp32 per lane per block
  constexpr int kALoads = BM / (16 * kWaves); // wave-level loads per slice
  constexpr int kBLoads = BN / (16 * kWaves);
  constexpr int kLoads = kALoads + kBLoads;
  constexpr int kABytes = BM * kRow;
  constexpr int kSlotBytes = (BM + BN) * kRow;
  constexpr int kMfma = kMI * kNI * kSub;
  constexpr int kReads = (kMI + kNI) * kSub;
  static_assert((SLOTS & (SLOTS - 1)) == 0, "slot index is s & (SLOTS-1)");
  typedef float acc_t __attribute__((ext_vector_type(kAccRegs)));

  __shared__ __attribute__((aligned(1024))) unsigned char lds[SLOTS * kSlotBytes];

  int tm, tn;
  tile_of_workgroup(M / BM, N / BN, tm, tn);
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wave_m = (wave / WN) * kWaveM;
  const int wave_n = (wave % WN) * kWaveN;

  // ---- global -> LDS ---------------------------------------------------------
  // load i of this wave fills slice rows (i*kWaves + wave)*16 .. +16; the byte
  // offset of a lane inside the panel fits 32 bits (checked by the host)
  const int ld_row = lane / 4;
  const int ld_chunk = (lane % 4) ^ ((lane >> 3) & 3);
  const char *a_base = reinterpret_cast<const char *>(A + (size_t)tm * BM * lda);
  const char *b_base = reinterpret_cast<const char *>(Bt + (size_t)tn * BN * ldb);
  uint32_t a_off[kALoads], b_off[kBLoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i)
    a_off[i] = (uint32_t)(((i * kWaves + wave) * 16 + ld_row) * lda * 2 + ld_chunk * 16);
#pragma unroll
  for (int i = 0; i < kBLoads; ++i)
    b_off[i] = (uint32_t)(((i * kWaves + wave) * 16 + ld_row) * ldb * 2 + ld_chunk * 16);
  const int KS = K / BK; // host guarantees K % 64 == 0 and KS >= SLOTS
  // Workgroups of one XCD start their walk over K at different slices (the sum
  // over K is the same in any order): at a given moment they then fetch from
  // different 64-byte columns of A and Bt, i.e. from different L2 channels.
  const int skew = SKEW ? ((int)(blockIdx.x / kXcds) * SKEW) % KS : 0;
  auto issue_loads = [&](int s) {
    int sk = s + skew;
    sk = sk >= KS ? sk - KS : sk;
    const char *ga = a_base + (size_t)sk * kRow;
    const char *gb = b_base + (size_t)sk * kRow;
    unsigned char *base = lds + (s & (SLOTS - 1)) * kSlotBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kALoads; ++i)
      __builtin_amdgcn_global_load_lds((global_cptr)(ga + a_off[i]),
                                       (lds_ptr)(base + i * kWaves * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_cptr)(gb + b_off[i]),
          (lds_ptr)(base + kABytes + i * kWaves * 1024), 16, 0, 0);
  };

  // ---- LDS -> operand registers ------------------------------------------------
  // lane l supplies row l % MF; its logical chunk in sub-step u is
  // (kSub == 1 ? l / 16 : 2 * u + l / 32)
  const int lrow = lane % MF, lhi = lane / MF;
  const int lswz = (lrow >> 1) & 3;
  int coff[kSub];
#pragma unroll
  for (int u = 0; u < kSub; ++u)
    coff[u] = lrow * kRow + (((kSub == 1 ? lhi : 2 * u + lhi) ^ lswz) * 16);
  const int fa_off = wave_m * kRow;
  const int fb_off = kABytes + wave_n * kRow;
  bf16x8 fa[2][kSub][kMI], fb[2][kSub][kNI];
  auto read_frags = [&](int s, auto set) {
    constexpr int S = decltype(set)::value;
    const unsigned char *base = lds + (s & (SLOTS - 1)) * kSlotBytes;
#pragma unroll
    for (int u = 0; u < kSub; ++u) {
#pragma unroll
      for (int j = 0; j < kNI; ++j)
        fb[S][u][j] = *reinterpret_cast<const bf16x8 *>(base + fb_off + coff[u] +
                                                        j * MF * kRow);
#pragma unroll
      for (int i = 0; i < kMI; ++i)
        fa[S][u][i] = *reinterpret_cast<const bf16x8 *>(base + fa_off + coff[u] +
                                                        i * MF * kRow);
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
  auto mma = [&](auto set) {
    constexpr int S = decltype(set)::value;
#pragma unroll
    for (int u = 0; u < kSub; ++u)
#pragma unroll
      for (int i = 0; i < kMI; ++i)
#pragma unroll
        for (int j = 0; j < kNI; ++j) {
          if constexpr (MF == 16)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                fb[S][u][j], fa[S][u][i], acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                fb[S][u][j], fa[S][u][i], acc[i][j], 0, 0, 0);
        }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;

  // LDS reads go out at the start of a step, at most one per MFMA and all
  // within its first half; the global->LDS loads are spread over the rest.
  auto interleave = [&](auto reads, auto vmem) {
    constexpr int R = decltype(reads)::value;
    constexpr int V = decltype(vmem)::value;
    constexpr int kRStride = (kMfma / 2) / (R > 0 ? R : 1) > 0 ? (kMfma / 2) / (R > 0 ? R : 1) : 1;
    constexpr int kRPer = R > kMfma / 2 ? (R + kMfma / 2 - 1) / (kMfma / 2) : 1;
    constexpr int kVStride = V > 0 ? (kMfma - 2) / V : 1;
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      if (R > 0 && i % kRStride == 0 && (i / kRStride) * kRPer < R)
        __builtin_amdgcn_sched_group_barrier(0x100, kRPer, 0); // DS read
      if (V > 0 && i >= 1 && (i - 1) % kVStride == 0 && (i - 1) / kVStride < V)
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // VMEM read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
    }
  };

  // VM = loads of this wave that may still be in flight at the top of the step
  // (those of slices after s+1)
  auto step = [&](int s, auto cur, auto nxt, auto load, auto read, auto vm) {
    constexpr bool LOAD = decltype(load)::value;
    constexpr bool READ = decltype(read)::value;
    constexpr int VM = decltype(vm)::value;
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((ABL & 1) ? 0 : VM, 0));
    if constexpr (!(ABL & 8))
      __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (LOAD && !(ABL & 1))
      issue_loads(s + SLOTS);
    if constexpr (READ && !(ABL & 2))
      read_frags(s + 1, nxt);
    if constexpr (!(ABL & 4)) {
      mma(cur);
      interleave(std::integral_constant < int, READ && !(ABL & 2) ? kReads : 0 > {},
                 std::integral_constant < int, LOAD && !(ABL & 1) ? kLoads : 0 > {});
    } else {
      constexpr int C = decltype(cur)::value;
#pragma unroll
      for (int u = 0; u < kSub; ++u) {
#pragma unroll
        for (int j = 0; j < kNI; ++j)
          asm volatile("" ::"v"(fb[C][u][j]));
#pragma unroll
        for (int i = 0; i < kMI; ++i)
          asm volatile("" ::"v"(fa[C][u][i]));
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

#pragma unroll
  for (int s = 0; s < SLOTS; ++s)
    issue_loads(s);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm((SLOTS - 1) * kLoads, kNoLgkm));
  __builtin_amdgcn_s_barrier();
  read_frags(0, Set0{});

  using Yes = std::true_type;
  using No = std::false_type;
  constexpr int kSteady = (SLOTS - 2) * kLoads;
  int s = 0;
  for (; s < KS - SLOTS; s += 2) {
    step(s, Set0{}, Set1{}, Yes{}, Yes{}, std::integral_constant<int, kSteady>{});
    step(s + 1, Set1{}, Set0{}, Yes{}, Yes{}, std::integral_constant<int, kSteady>{});
  }
  // the last SLOTS slices: nothing left to request
  static_assert(SLOTS == 4, "tail below is written for four slots");
  step(s, Set0{}, Set1{}, No{}, Yes{}, std::integral_constant<int, 2 * kLoads>{});
  step(s + 1, Set1{}, Set0{}, No{}, Yes{}, std::integral_constant<int, 1 * kLoads>{});
  step(s + 2, Set0{}, Set1{}, No{}, Yes{}, std::integral_constant<int, 0>{});
  step(s + 3, Set1{}, Set0{}, No{}, No{}, std::integral_constant<int, 0>{});

  // ---- epilogue ------------------------------------------------------------------
  // MF = 16: lane holds C[l % 16][4*(l/16) + e];  MF = 32: C[l % 32][8*g +
  // 4*(l/32) + e] for accumulator element 4*g + e.
  const int m_base = tm * BM + wave_m + lrow;
  const int n_base = tn * BN + wave_n + lhi * 4;
#pragma unroll
  for (int i = 0; i < kMI; ++i) {
    __bf16 *crow = C + (size_t)(m_base + i * MF) * ldc + n_base;
#pragma unroll
    for (int j = 0; j < kNI; ++j) {
#pragma unroll
      for (int g = 0; g < kAccRegs / 4; ++g) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (__bf16)acc[i][j][4 * g + e];
        *reinterpret_cast<bf16x4 *>(crow + j * MF + g * 8) = o;
      }
    }
  }
}
} // namespace

#define HCAMD_GEMM_PM(NAME, WM, WN, MF)                                          \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_pipelined_mf<256, 256, WM, WN, MF>(A, lda, Bt, ldb, C, ldc, M,   \
                                                 N, K);                        \
  }
HCAMD_GEMM_PM(hcamd_gemm_bf16_pm32_256x256_w2x4, 2, 4, 32)
HCAMD_GEMM_PM(hcamd_gemm_bf16_pm32_256x256_w4x2, 4, 2, 32)
HCAMD_GEMM_PM(hcamd_gemm_bf16_pm16_256x256_w2x4, 2, 4, 16)

#define HCAMD_GEMM_N(NAME, WM, WN, MF)                                           \
  extern "C" __global__ __launch_bounds__(WM *WN * 64) void NAME(              \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_ring<WM, WN, 4, MF>(A, lda, Bt, ldb, C, ldc, M, N, K);           \
  }
HCAMD_GEMM_N(hcamd_gemm_bf16_n256x256_w2x2, 2, 2, 32)
HCAMD_GEMM_N(hcamd_gemm_bf16_n256x256_w2x4, 2, 4, 16)
HCAMD_GEMM_N(hcamd_gemm_bf16_n256x256_w4x2, 4, 2, 16)
HCAMD_GEMM_N(hcamd_gemm_bf16_n32_256x256_w2x4, 2, 4, 32)

#define HCAMD_GEMM_P(NAME, BM, BN, WM, WN, SH)                                 \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(             \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_pipelined<BM, BN, WM, WN, SH>(A, lda, Bt, ldb, C, ldc, M, N, K); \
  }

HCAMD_GEMM_P(hcamd_gemm_bf16_p256x256_w2x4, 256, 256, 2, 4, 0)
HCAMD_GEMM_P(hcamd_gemm_bf16_p256x256_w4x2, 256, 256, 4, 2, 0)
HCAMD_GEMM_P(hcamd_gemm_bf16_p256x256_w2x2, 256, 256, 2, 2, 0)
HCAMD_GEMM_P(hcamd_gemm_bf16_p128x128_w2x2, 128, 128, 2, 2, 0)
HCAMD_GEMM_P(hcamd_gemm_bf16_p256x128_w2x2, 256, 128, 2, 2, 0)

#define HCAMD_GEMM_Q(NAME, BM, BN, WM, WN)                                     \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(             \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_p32<BM, BN, WM, WN>(A, lda, Bt, ldb, C, ldc, M, N, K);           \
  }

HCAMD_GEMM_Q(hcamd_gemm_bf16_q256x256_w2x4, 256, 256, 2, 4)
HCAMD_GEMM_Q(hcamd_gemm_bf16_q256x256_w4x2, 256, 256, 4, 2)
HCAMD_GEMM_Q(hcamd_gemm_bf16_q256x256_w2x2, 256, 256, 2, 2)
HCAMD_GEMM_Q(hcamd_gemm_bf16_q128x128_w2x2, 128, 128, 2, 2)
HCAMD_GEMM_Q(hcamd_gemm_bf16_q256x128_w2x4, 256, 128, 2, 4)

#define HCAMD_GEMM_PP(NAME, BM, BN, WM, WN)                                    \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(             \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile_pingpong<BM, BN, WM, WN>(A, lda, Bt, ldb, C, ldc, M, N, K);      \
  }

HCAMD_GEMM_PP(hcamd_gemm_bf16_pp256x256_w2x4, 256, 256, 2, 4)
HCAMD_GEMM_PP(hcamd_gemm_bf16_pp256x256_w4x2, 256, 256, 4, 2)

extern "C" __global__ __launch_bounds__(256) void hcamd_gemm_bf16_r256x256(
    const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,
    size_t ldc, int M, int N, int K) {
  gemm_tile_staged(A, lda, Bt, ldb, C, ldc, M, N, K);
}


#define HCAMD_GEMM(NAME, BM, BN, WM, WN, SH)                                   \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(             \
      const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,    \
      size_t ldc, int M, int N, int K) {                                       \
    gemm_tile<BM, BN, WM, WN, SH>(A, lda, Bt, ldb, C, ldc, M, N, K);           \
  }

HCAMD_GEMM(hcamd_gemm_bf16_256x256_w2x4_s0, 256, 256, 2, 4, 0)
HCAMD_GEMM(hcamd_gemm_bf16_256x256_w2x4_s1, 256, 256, 2, 4, 1)
HCAMD_GEMM(hcamd_gemm_bf16_256x256_w4x2_s0, 256, 256, 4, 2, 0)
HCAMD_GEMM(hcamd_gemm_bf16_256x256_w2x2_s0, 256, 256, 2, 2, 0)
HCAMD_GEMM(hcamd_gemm_bf16_128x128_w2x2_s0, 128, 128, 2, 2, 0)
HCAMD_GEMM(hcamd_gemm_bf16_256x128_w2x2_s0, 256, 128, 2, 2, 0)

// General kernel: any M, N, K, any leading dimensions and alignment.  A
// 64 x 64 tile of C per workgroup, a 4 x 4 block per thread, fp32 FMAs on
// LDS-staged 64 x 16 panels, every access bounds-checked.  Correct everywhere,
// fast nowhere; it exists for the shapes the tiled kernel does not take.
extern "C" __global__ __launch_bounds__(256) void hcamd_gemm_bf16_general(
    const __bf16 *A, size_t lda, const __bf16 *Bt, size_t ldb, __bf16 *C,
    size_t ldc, int M, int N, int K) {
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
        C[(size_t)gm * ldc + gn] = (__bf16)acc[i][j];
    }
}
