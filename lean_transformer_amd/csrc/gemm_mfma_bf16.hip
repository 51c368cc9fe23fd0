// Tiled bf16 GEMM for gfx950 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulation) with the FFN epilogues fused.
//
// Tile: BM x BN outputs per workgroup, 64 k per step, WM x WN wavefronts each owning a (BM/WM) x (BN/WN) sub-tile as
// 32 x 32 MFMA blocks.  Operand tiles go global -> registers -> LDS (16-byte accesses) and are double-buffered in LDS:
// while the matrix cores work on one stage the global loads of the next are in flight, with one barrier per k-step.
//
// Either operand may be stored k-major (k contiguous: activations x weights^T) or mn-major (k strided: transposed
// activations in the weight-gradient GEMMs, weights in the input-gradient GEMMs):
//   k-major   LDS tile [rows][64]: 128-byte rows of eight 16-byte chunks; chunk c of row r sits in slot c ^ ((r >> 1) & 7),
//             so the 16 lanes of one LDS access phase (rows r..r+15, same logical chunk) cover all 64 banks.
//             A lane reads its 8 consecutive k values with one ds_read_b128.
//   mn-major  LDS tile [64][cols]: the MFMA operand needs 8 k values of one column per lane, i.e. a transpose; it is done by
//             the LDS itself with ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of 4 consecutive columns
//             (4 * (i % 4) ..) of k-row i / 4 and receives column i of the 4 k-rows.  16-byte chunks are swizzled by
//             (k & 3) << 2 | ((k >> 3) & 1) << 1 to spread the k-rows of one access over the banks.
// No transposed copy of an activation or weight is ever written to HBM.
//
// Workgroups are numbered so that each XCD (hardware dispatches workgroup i to XCD i % 8) walks a contiguous range of
// tiles, GROUP_M tile-rows at a time, keeping one XCD's 32 concurrent tiles on few distinct A / B panels in its own L2.
#include <type_traits>

#include "lt_gemm.h"

namespace {

constexpr int BK = 64;
constexpr int GROUP_M = 8;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4;

__device__ __forceinline__ int swz_km(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_mn(int k) { return ((k & 3) << 2) | (((k >> 3) & 1) << 1); }

// scheduling hint for one k-substep: spread READS LDS-read instructions evenly between MFMAS matrix instructions
template <int READS, int MFMAS, int G = 0> struct SchedInterleave {
  static __device__ __forceinline__ void run() {
    constexpr int n = READS * (G + 1) / MFMAS - READS * G / MFMAS;
    if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (G + 1 < MFMAS) SchedInterleave<READS, MFMAS, G + 1>::run();
  }
};

template <int BM, int BN, int WM, int WN, bool A_KM, bool B_KM, int KIND, typename TX>
__global__ __launch_bounds__(WM * WN * 64) void gemm_bf16_kernel(GemmProblem p, int tiles_m, int tiles_n) {
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int FM = WTM / 32, FN = WTN / 32;
  constexpr int A_CHUNKS = BM * BK / 8 / NT, B_CHUNKS = BN * BK / 8 / NT;  // 16-byte chunks per thread per stage
  static_assert(BM * BK / 8 % NT == 0 && BN * BK / 8 % NT == 0, "tile must divide over the threads");
  static_assert(FN % 2 == 0 || KIND != EPI_ACT_FWD, "gated pairing needs an even number of column blocks per wavefront");

  // two stages of both operand tiles; after the main loop the same memory stages accumulator strips for the epilogue
  constexpr int STAGE_LD = WTN + 8;  // floats per staged row: 4 rows apart land 32 banks apart
  constexpr int SMEM_BYTES = 2 * (BM + BN) * BK * 2 > WM * WN * 32 * STAGE_LD * 4 ? 2 * (BM + BN) * BK * 2
                                                                                   : WM * WN * 32 * STAGE_LD * 4;
  __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];
  bf16(*lds_a)[BM * BK] = reinterpret_cast<bf16(*)[BM * BK]>(smem);
  bf16(*lds_b)[BN * BK] = reinterpret_cast<bf16(*)[BN * BK]>(smem + 2 * BM * BK * 2);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const bool gated = (KIND == EPI_ACT_FWD) && p.epi.gated;

  // ---- tile assignment: XCD-contiguous, grouped along M
  int pid = blockIdx.x;
  const int num_pid = tiles_m * tiles_n;
  if ((num_pid & 7) == 0) pid = (pid & 7) * (num_pid >> 3) + (pid >> 3);
  const int group = GROUP_M * tiles_n;
  const int first_m = (pid / group) * GROUP_M;
  const int gsz = min(tiles_m - first_m, GROUP_M);
  const int tm = first_m + (pid % group) % gsz;
  const int tn = (pid % group) / gsz;
  const int64_t m0 = (int64_t)tm * BM;
  const int64_t n0 = (int64_t)tn * (gated ? BN / 2 : BN);  // gated: in gate columns

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  u32x4 ra[A_CHUNKS], rb[B_CHUNKS];

  const int kt_seg0 = (int)((p.K[0] + BK - 1) / BK);
  const int kt_total = kt_seg0 + (p.nseg > 1 ? (int)((p.K[1] + BK - 1) / BK) : 0);

  // global -> registers for k-step kt
  auto load_tiles = [&](int kt) {
    const int seg = kt >= kt_seg0;
    const int64_t k0 = (int64_t)(seg ? kt - kt_seg0 : kt) * BK;
    const int64_t K = p.K[seg];
    const bf16* A = reinterpret_cast<const bf16*>(p.A[seg].ptr);
    const bf16* B = reinterpret_cast<const bf16*>(p.B[seg].ptr);
    const int64_t lda = p.A[seg].ld, ldb = p.B[seg].ld;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (A_KM) {
        const int row = q >> 3, c = q & 7;
        const int64_t gm = min(m0 + row, p.M - 1);  // rows past M are clamped (their results are never stored)
        ra[i] = *reinterpret_cast<const u32x4*>(A + gm * lda + k0 + c * 8);
      } else {
        const int kr = q / (BM / 8), c = q % (BM / 8);
        const int64_t gk = k0 + kr;
        ra[i] = gk < K ? *reinterpret_cast<const u32x4*>(A + gk * lda + m0 + c * 8) : u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (B_KM) {
        const int row = q >> 3, c = q & 7;
        int64_t gn;
        if (gated) {
          const int rr = row % WTN;
          gn = (rr / (WTN / 2)) * p.N + n0 + (row / WTN) * (WTN / 2) + rr % (WTN / 2);
        } else {
          gn = n0 + row;
        }
        rb[i] = *reinterpret_cast<const u32x4*>(B + gn * ldb + k0 + c * 8);
      } else {
        const int kr = q / (BN / 8), c = q % (BN / 8);
        const int64_t gk = k0 + kr;
        rb[i] = gk < K ? *reinterpret_cast<const u32x4*>(B + gk * ldb + n0 + c * 8) : u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  // registers -> LDS stage s
  auto store_tiles = [&](int s) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (A_KM) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<u32x4*>(&lds_a[s][(row * 8 + (c ^ swz_km(row))) * 8]) = ra[i];
      } else {
        const int kr = q / (BM / 8), c = q % (BM / 8);
        *reinterpret_cast<u32x4*>(&lds_a[s][kr * BM + ((c ^ swz_mn(kr)) << 3)]) = ra[i];
      }
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (B_KM) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<u32x4*>(&lds_b[s][(row * 8 + (c ^ swz_km(row))) * 8]) = rb[i];
      } else {
        const int kr = q / (BN / 8), c = q % (BN / 8);
        *reinterpret_cast<u32x4*>(&lds_b[s][kr * BN + ((c ^ swz_mn(kr)) << 3)]) = rb[i];
      }
    }
  };
  // one MFMA operand fragment (8 k values of row/column `lane & 31` of 32-wide block starting at `base`) for k-substep kk
  auto frag_km = [&](const bf16* tile, int base, int kk) -> bf16x8 {
    const int row = base + (lane & 31);
    const int c = kk * 2 + (lane >> 5);
    return *reinterpret_cast<const bf16x8*>(&tile[(row * 8 + (c ^ swz_km(row))) * 8]);
  };
  auto frag_mn = [&](const bf16* tile, int cols, int base, int kk) -> bf16x8 {
    union { bf16x8 v; s16x4 h[2]; } u;
    const int i16 = lane & 15;
    const int col = base + ((lane >> 4) & 1) * 16 + 4 * (i16 & 3);
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int kr = kk * 16 + 8 * (lane >> 5) + 4 * s + (i16 >> 2);
      const bf16* src = &tile[kr * cols + ((((col >> 3) ^ swz_mn(kr)) << 3) | (col & 7))];
      u.h[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(src));
    }
    return u.v;
  };

  auto load_frags = [&](int s, int kk, bf16x8 (&a)[FM], bf16x8 (&b)[FN]) {
#pragma unroll
    for (int i = 0; i < FM; i++) {
      if constexpr (A_KM) a[i] = frag_km(lds_a[s], wm * WTM + i * 32, kk);
      else a[i] = frag_mn(lds_a[s], BM, wm * WTM + i * 32, kk);
    }
#pragma unroll
    for (int j = 0; j < FN; j++) {
      if constexpr (B_KM) b[j] = frag_km(lds_b[s], wn * WTN + j * 32, kk);
      else b[j] = frag_mn(lds_b[s], BN, wn * WTN + j * 32, kk);
    }
  };
  constexpr int FRAG_READS = FM * (A_KM ? 1 : 2) + FN * (B_KM ? 1 : 2);  // LDS read instructions per k-substep

  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  for (int kt = 0; kt < kt_total; kt++) {
    const int s = kt & 1;
    const bool has_next = kt + 1 < kt_total;
    if (has_next) load_tiles(kt + 1);
    // fragments are double-buffered in registers: the LDS reads of k-substep kk + 1 are issued before, and interleaved
    // with, the MFMAs of k-substep kk
    bf16x8 af[2][FM], bfr[2][FN];
    load_frags(s, 0, af[0], bfr[0]);
#pragma unroll
    for (int kk = 0; kk < BK / 16; kk++) {
      if (kk + 1 < BK / 16) load_frags(s, kk + 1, af[(kk + 1) & 1], bfr[(kk + 1) & 1]);
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j], 0, 0, 0);
      if (kk + 1 < BK / 16) SchedInterleave<FRAG_READS, FM * FN>::run();
    }
    if (has_next) store_tiles(s ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  The accumulators of a 32 x 32 block sit column-per-lane (register r = row 8 * (r / 4) + 4 * (lane / 32)
  //      + r % 4, column lane % 32); each wavefront transposes one 32-row strip of its sub-tile at a time through its own
  //      LDS region and reads it back row-major, 8 consecutive columns per lane, so that the fused epilogue reads and
  //      writes HBM in 16-byte pieces of contiguous rows.  (The main loop ended with a barrier: the stages are free.)
  float* stage = reinterpret_cast<float*>(smem) + wave * (32 * STAGE_LD);
  const bool pair = (KIND == EPI_ACT_FWD) && gated;
#pragma unroll
  for (int i = 0; i < FM; i++) {
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * STAGE_LD + j * 32 + (lane & 31)] = acc[i][j][r];
    __builtin_amdgcn_wave_barrier();
    const int64_t mrow0 = m0 + wm * WTM + i * 32;
    if (pair) {
      // columns [0, WTN/2) of the sub-tile are gate columns, [WTN/2, WTN) the matching linear columns
      constexpr int LANES_PER_ROW = WTN / 2 / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        float vg[8], vl[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          vg[e] = stage[row * STAGE_LD + c + e];
          vl[e] = stage[row * STAGE_LD + WTN / 2 + c + e];
        }
        if (m < p.M) epi_act_fwd_gated8(p.epi, m, n0 + wn * (WTN / 2) + c, vg, vl);
      }
    } else {
      constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        const int64_t n = n0 + wn * WTN + c;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = stage[row * STAGE_LD + c + e];
        if (m < p.M) {
          if constexpr (KIND == EPI_STORE) epi_store8(p.epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_FWD) epi_act_fwd8(p.epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_BWD) epi_act_bwd8(p.epi, m, n, v);
          else epi_out8<TX>(p.epi, m, n, v);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// =====================================================================================================================
// Variant with asynchronous global -> LDS copies (global_load_lds_dwordx4): operand tiles never pass through registers.
// A wavefront's copy instruction deposits the 64 lanes' 16-byte pieces at consecutive LDS addresses (lane i at base + 16 i),
// so the swizzled LDS layouts are produced by choosing which global chunk each lane fetches.
//
// Tile 256 x 256, 4 wavefronts (2 x 2, 128 x 128 each), k-steps of 32, a ring of 4 LDS stages (each one array holding the
// A and the B tile of a k-step, so that copies into one stage provably do not alias reads of another), k-loop unrolled by 4.
// Pipeline of k-step kt:
//     matrix instructions on the first 16 k (fragments already in registers)
//         interleaved with: LDS reads of the second 16 k, copies of k-step kt + 3 into the stage freed one barrier ago
//     wait until this wavefront's copies of k-step kt + 1 have landed and its LDS reads are done; workgroup barrier
//     matrix instructions on the second 16 k
//         interleaved with: LDS reads of the first 16 k of k-step kt + 1
// Copies therefore have three k-steps to arrive, and no LDS read latency is exposed after the barrier.
// =====================================================================================================================
__device__ const u32x4 lt_zero_chunk = {0u, 0u, 0u, 0u};  // source of the lanes past the end of a ragged reduction

constexpr int DK = 32;  // k per step of the copy-based kernel

// scheduling hint for one half k-step: READS LDS reads and COPIES global->LDS copies spread evenly over MFMAS matrix
// instructions (packing the reads into the first half of the matrix instructions measured slower)
template <int READS, int COPIES, int MFMAS, int G = 0> struct SchedInterleave3 {
  static __device__ __forceinline__ void run() {
    constexpr int nr = READS * (G + 1) / MFMAS - READS * G / MFMAS;
    constexpr int nc = COPIES * (G + 1) / MFMAS - COPIES * G / MFMAS;
    if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
    if constexpr (nc > 0) __builtin_amdgcn_sched_group_barrier(0x020, nc, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (G + 1 < MFMAS) SchedInterleave3<READS, COPIES, MFMAS, G + 1>::run();
  }
};

// k-major tile with 64-byte rows (32 k): four 16-byte chunks per row, four rows per 256-byte bank line
__device__ __forceinline__ int swz_km32(int row) { return (row >> 2) & 3; }

// wait until at most N of this wavefront's copies are in flight and all its LDS reads have returned, then barrier.
// The wait is a real s_waitcnt instruction (not inline assembly) so that the compiler's own wait-count bookkeeping sees
// that older copies have landed; the empty asm statements only keep it from moving LDS accesses across the barrier.
template <int N> __device__ __forceinline__ void wait_copies_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));  // vmcnt(N) expcnt(7: none) lgkmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <bool A_KM, bool B_KM, int KIND, typename TX, bool K_TAIL>
__global__ __launch_bounds__(256) void gemm_bf16_dma_kernel(GemmProblem p, int tiles_m, int tiles_n) {
  constexpr int BM = 256, BN = 256, WN = 2, WTM = 128, WTN = 128, FM = 4, FN = 4;
  constexpr int LOADS = 4;                       // copy instructions per wavefront per operand per k-step (16 KiB / 4 / 1 KiB)
  constexpr int STAGE_ELEMS = (BM + BN) * DK;    // one stage: A tile then B tile
  __shared__ __attribute__((aligned(1024))) bf16 stage0[STAGE_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 stage1[STAGE_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 stage2[STAGE_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 stage3[STAGE_ELEMS];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const bool gated = (KIND == EPI_ACT_FWD) && p.epi.gated;

  int pid = blockIdx.x;
  const int num_pid = tiles_m * tiles_n;
  if ((num_pid & 7) == 0) pid = (pid & 7) * (num_pid >> 3) + (pid >> 3);
  const int group = GROUP_M * tiles_n;
  const int first_m = (pid / group) * GROUP_M;
  const int gsz = min(tiles_m - first_m, GROUP_M);
  const int tm = first_m + (pid % group) % gsz;
  const int tn = (pid % group) / gsz;
  const int64_t m0 = (int64_t)tm * BM;
  const int64_t n0 = (int64_t)tn * (gated ? BN / 2 : BN);

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int kt_seg0 = (int)((p.K[0] + DK - 1) / DK);
  const int kt_total = kt_seg0 + (p.nseg > 1 ? (int)((p.K[1] + DK - 1) / DK) : 0);

  // ---- per-lane byte offsets of this wavefront's copies, relative to a wavefront-uniform base that advances with k
  uint32_t off_a[LOADS], off_b[LOADS];
  int krow_a[LOADS], krow_b[LOADS];  // mn-major: k-row inside the k-step (for the ragged-reduction test)
  const char* base_a = nullptr;
  const char* base_b = nullptr;
  int64_t step_a = 0, step_b = 0;  // bytes per k-step
  auto setup_segment = [&](int seg) {
    const int64_t lda = p.A[seg].ld, ldb = p.B[seg].ld;
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
      const int q = (wave * LOADS + j) * 64 + lane;  // 16-byte slot of the LDS tile this lane fills
      if constexpr (A_KM) {
        const int row = q >> 2, c = (q & 3) ^ swz_km32(row);
        const int64_t gm = min(m0 + row, p.M - 1) - m0;
        off_a[j] = (uint32_t)((gm * lda + c * 8) * 2);
        krow_a[j] = 0;
      } else {
        const int kr = q / (BM / 8), c = (q % (BM / 8)) ^ swz_mn(kr);
        off_a[j] = (uint32_t)((kr * lda + c * 8) * 2);
        krow_a[j] = kr;
      }
      if constexpr (B_KM) {
        const int row = q >> 2, c = (q & 3) ^ swz_km32(row);
        int64_t gn;
        if (gated) {
          const int rr = row % WTN;
          gn = (rr / (WTN / 2)) * p.N + (row / WTN) * (WTN / 2) + rr % (WTN / 2);
        } else {
          gn = row;
        }
        off_b[j] = (uint32_t)((gn * ldb + c * 8) * 2);
        krow_b[j] = 0;
      } else {
        const int kr = q / (BN / 8), c = (q % (BN / 8)) ^ swz_mn(kr);
        off_b[j] = (uint32_t)((kr * ldb + c * 8) * 2);
        krow_b[j] = kr;
      }
    }
    const char* a = reinterpret_cast<const char*>(p.A[seg].ptr);
    const char* b = reinterpret_cast<const char*>(p.B[seg].ptr);
    base_a = A_KM ? a + m0 * lda * 2 : a + m0 * 2;
    base_b = B_KM ? b + n0 * ldb * 2 : b + n0 * 2;
    step_a = A_KM ? DK * 2 : DK * lda * 2;
    step_b = B_KM ? DK * 2 : DK * ldb * 2;
  };
  setup_segment(0);
  int copy_seg = 0;  // segment the offsets above belong to

  // all copies of k-step kt (2 * LOADS instructions) into stage `st`
  auto issue_copies = [&](auto steady, int kt, bf16* st) {
    int seg = copy_seg;
    if constexpr (!decltype(steady)::value) {  // the steady loop never crosses a segment boundary
      seg = kt >= kt_seg0;
      if (seg != copy_seg) {
        setup_segment(seg);
        copy_seg = seg;
      }
    }
    const int ks = seg ? kt - kt_seg0 : kt;
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
      const char* ga = base_a + ks * step_a + off_a[j];
      const char* gb = base_b + ks * step_b + off_b[j];
      if constexpr (K_TAIL) {
        const int64_t K = p.K[seg];
        if (!A_KM && (int64_t)ks * DK + krow_a[j] >= K) ga = reinterpret_cast<const char*>(&lt_zero_chunk);
        if (!B_KM && (int64_t)ks * DK + krow_b[j] >= K) gb = reinterpret_cast<const char*>(&lt_zero_chunk);
      }
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)ga,
                                       (__attribute__((address_space(3))) void*)(st + (wave * LOADS + j) * 512), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gb,
                                       (__attribute__((address_space(3))) void*)(st + BM * DK + (wave * LOADS + j) * 512), 16,
                                       0, 0);
    }
  };
  auto frag_km = [&](const bf16* tile, int base, int kk) -> bf16x8 {
    const int row = base + (lane & 31);
    const int c = kk * 2 + (lane >> 5);
    return *reinterpret_cast<const bf16x8*>(&tile[(row * 4 + (c ^ swz_km32(row))) * 8]);
  };
  auto frag_mn = [&](const bf16* tile, int cols, int base, int kk) -> bf16x8 {
    union { bf16x8 v; s16x4 h[2]; } u;
    const int i16 = lane & 15;
    const int col = base + ((lane >> 4) & 1) * 16 + 4 * (i16 & 3);
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int kr = kk * 16 + 8 * (lane >> 5) + 4 * s + (i16 >> 2);
      const bf16* src = &tile[kr * cols + ((((col >> 3) ^ swz_mn(kr)) << 3) | (col & 7))];
      u.h[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(src));
    }
    return u.v;
  };
  auto load_frags = [&](const bf16* st, int kk, bf16x8 (&a)[FM], bf16x8 (&b)[FN]) {
#pragma unroll
    for (int i = 0; i < FM; i++) {
      if constexpr (A_KM) a[i] = frag_km(st, wm * WTM + i * 32, kk);
      else a[i] = frag_mn(st, BM, wm * WTM + i * 32, kk);
    }
#pragma unroll
    for (int j = 0; j < FN; j++) {
      if constexpr (B_KM) b[j] = frag_km(st + BM * DK, wn * WTN + j * 32, kk);
      else b[j] = frag_mn(st + BM * DK, BN, wn * WTN + j * 32, kk);
    }
  };
  constexpr int FRAG_READS = FM * (A_KM ? 1 : 2) + FN * (B_KM ? 1 : 2);

  bf16x8 af[2][FM], bfr[2][FN];  // [0]: first 16 k of the current k-step, [1]: second 16 k

  // A k-step is issued as two halves so that the loop body can start at the barrier:
  //   first_half(kt)   LDS reads of the second 16 k of k-step kt (stage `cur`), copies of k-step kt + 3 into `cpy`,
  //                    matrix instructions on the first 16 k
  //   second_half(kt)  wait for the copies of k-step kt + 1 + barrier, LDS reads of the first 16 k of k-step kt + 1 (stage
  //                    `nxt`), matrix instructions on the second 16 k
  // steady == true: straight-line code for k-steps far enough from the end of their k-segment.
  auto first_half = [&](auto steady, int kt, const bf16* cur, bf16* cpy) {
    constexpr bool STEADY = decltype(steady)::value;
    load_frags(cur, 1, af[1], bfr[1]);
    if (STEADY || kt + 3 < kt_total) issue_copies(steady, kt + 3, cpy);
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[0][i], bfr[0][j], acc[i][j], 0, 0, 0);
    SchedInterleave3<FRAG_READS, 2 * LOADS, FM * FN>::run();
  };
  auto second_half = [&](auto steady, int kt, const bf16* nxt) {
    constexpr bool STEADY = decltype(steady)::value;
    const int remaining = kt_total - 1 - kt;  // k-steps after this one
    // copies still allowed in flight: those of k-steps kt + 2 and kt + 3 (issued after the ones of kt + 1)
    if (STEADY || remaining >= 3) wait_copies_and_barrier<4 * LOADS>();
    else if (remaining == 2) wait_copies_and_barrier<2 * LOADS>();
    else wait_copies_and_barrier<0>();
    if (STEADY || remaining >= 1) load_frags(nxt, 0, af[0], bfr[0]);
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[1][i], bfr[1][j], acc[i][j], 0, 0, 0);
    SchedInterleave3<FRAG_READS, 0, FM * FN>::run();
  };
  using Steady = std::integral_constant<bool, true>;
  using Ragged = std::integral_constant<bool, false>;

  // ---- prologue: first three k-steps in flight, the first one landed, first half of k-step 0 issued
  issue_copies(Ragged{}, 0, stage0);
  if (kt_total > 1) issue_copies(Ragged{}, 1, stage1);
  if (kt_total > 2) issue_copies(Ragged{}, 2, stage2);
  if (kt_total > 2) wait_copies_and_barrier<4 * LOADS>();
  else if (kt_total == 2) wait_copies_and_barrier<2 * LOADS>();
  else wait_copies_and_barrier<0>();
  load_frags(stage0, 0, af[0], bfr[0]);
  first_half(Ragged{}, 0, stage0, stage3);

  // loop body i of a group of four: second half of k-step kt + i, first half of k-step kt + i + 1
  int kt = 0;
  for (;;) {
    // copies issued by the steady loop (k-steps up to kt + 7) must stay inside the k-segment the offsets are set up for
    const int bound = (copy_seg == 0 && p.nseg > 1) ? kt_seg0 : kt_total;
    for (; kt + 7 < bound; kt += 4) {
      second_half(Steady{}, kt, stage1);
      first_half(Steady{}, kt + 1, stage1, stage0);
      second_half(Steady{}, kt + 1, stage2);
      first_half(Steady{}, kt + 2, stage2, stage1);
      second_half(Steady{}, kt + 2, stage3);
      first_half(Steady{}, kt + 3, stage3, stage2);
      second_half(Steady{}, kt + 3, stage0);
      first_half(Steady{}, kt + 4, stage0, stage3);
    }
    if (kt >= kt_total) break;
    second_half(Ragged{}, kt, stage1);
    if (kt + 1 < kt_total) { first_half(Ragged{}, kt + 1, stage1, stage0); second_half(Ragged{}, kt + 1, stage2); }
    if (kt + 2 < kt_total) { first_half(Ragged{}, kt + 2, stage2, stage1); second_half(Ragged{}, kt + 2, stage3); }
    if (kt + 3 < kt_total) { first_half(Ragged{}, kt + 3, stage3, stage2); second_half(Ragged{}, kt + 3, stage0); }
    if (kt + 4 < kt_total) first_half(Ragged{}, kt + 4, stage0, stage3);
    kt += 4;
    if (kt >= kt_total) break;
  }
  __syncthreads();  // every wavefront is done with the stages: they become epilogue staging space

  // ---- epilogue: as in the register-staged kernel; each wavefront stages its strips in a stage array of its own
  constexpr int STAGE_LD = WTN + 8;
  static_assert(32 * STAGE_LD * 4 <= STAGE_ELEMS * 2, "a 32-row strip must fit one stage array");
  float* stage = reinterpret_cast<float*>(wave == 0 ? stage0 : wave == 1 ? stage1 : wave == 2 ? stage2 : stage3);
  const bool pair = (KIND == EPI_ACT_FWD) && gated;
#pragma unroll
  for (int i = 0; i < FM; i++) {
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * STAGE_LD + j * 32 + (lane & 31)] = acc[i][j][r];
    __builtin_amdgcn_wave_barrier();
    const int64_t mrow0 = m0 + wm * WTM + i * 32;
    if (pair) {
      constexpr int LANES_PER_ROW = WTN / 2 / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        float vg[8], vl[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          vg[e] = stage[row * STAGE_LD + c + e];
          vl[e] = stage[row * STAGE_LD + WTN / 2 + c + e];
        }
        if (m < p.M) epi_act_fwd_gated8(p.epi, m, n0 + wn * (WTN / 2) + c, vg, vl);
      }
    } else {
      constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        const int64_t n = n0 + wn * WTN + c;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = stage[row * STAGE_LD + c + e];
        if (m < p.M) {
          if constexpr (KIND == EPI_STORE) epi_store8(p.epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_FWD) epi_act_fwd8(p.epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_BWD) epi_act_bwd8(p.epi, m, n, v);
          else epi_out8<TX>(p.epi, m, n, v);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <bool A_KM, bool B_KM, int KIND>
int launch_dma(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  const bool gated = KIND == EPI_ACT_FWD && p.epi.gated;
  const int tiles_m = (int)((p.M + 255) / 256);
  const int tiles_n = (int)(p.N / (gated ? 128 : 256));
  bool k_tail = false;
  for (int s = 0; s < p.nseg; s++) k_tail = k_tail || (p.K[s] % DK != 0);
  dim3 grid((unsigned)(tiles_m * tiles_n)), block(256);
  const bool bf16_io = KIND == EPI_OUT && io_dtype == LT_BF16;
  if constexpr (!A_KM && !B_KM) {
    if (k_tail) {
      hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, float, true>), grid, block, 0, stream, p, tiles_m, tiles_n);
      LT_LAUNCH_CHECK();
      return LT_OK;
    }
  }
  if (bf16_io)
    hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, bf16, false>), grid, block, 0, stream, p, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, float, false>), grid, block, 0, stream, p, tiles_m, tiles_n);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

template <int BM, int BN, int WM, int WN, bool A_KM, bool B_KM, int KIND>
int launch_cfg(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  const bool gated = KIND == EPI_ACT_FWD && p.epi.gated;
  const int tiles_m = (int)((p.M + BM - 1) / BM);
  const int tiles_n = (int)(p.N / (gated ? BN / 2 : BN));
  dim3 grid((unsigned)(tiles_m * tiles_n)), block(WM * WN * 64);
  if (KIND == EPI_OUT && io_dtype == LT_BF16) {
    hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, WM, WN, A_KM, B_KM, KIND, bf16>), grid, block, 0, stream, p, tiles_m,
                       tiles_n);
  } else {
    hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, WM, WN, A_KM, B_KM, KIND, float>), grid, block, 0, stream, p, tiles_m,
                       tiles_n);
  }
  LT_LAUNCH_CHECK();
  return LT_OK;
}

// the copy-based kernel addresses its operands with 32-bit byte offsets from a per-tile base
bool dma_offsets_fit(const GemmProblem& p, int kind) {
  const bool gated = kind == EPI_ACT_FWD && p.epi.gated;
  for (int s = 0; s < p.nseg; s++) {
    const int64_t a_span = p.A[s].kmajor ? 256 * p.A[s].ld : 64 * p.A[s].ld;
    const int64_t b_span = p.B[s].kmajor ? ((gated ? p.N : 0) + 256) * p.B[s].ld : 64 * p.B[s].ld;
    if ((a_span + 512) * 2 >= (int64_t)1 << 32 || (b_span + 512) * 2 >= (int64_t)1 << 32) return false;
  }
  return true;
}

int g_mfma_variant = 0;  // 0: choose; 1: register-staged kernel; 2: copy-based kernel (tests and benchmarks)

template <bool A_KM, bool B_KM, int KIND> int launch_tile(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  bool k_tail = false;
  for (int s = 0; s < p.nseg; s++) k_tail = k_tail || (p.K[s] % DK != 0);
  const bool dma_ok = dma_offsets_fit(p, KIND) && !(k_tail && KIND == EPI_OUT && io_dtype == LT_BF16);
  if (g_mfma_variant != 1 && dma_ok) return launch_dma<A_KM, B_KM, KIND>(p, io_dtype, stream);
  return launch_cfg<256, 256, 2, 2, A_KM, B_KM, KIND>(p, io_dtype, stream);
}

template <int KIND> int launch_layout(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  if (a_km && b_km) return launch_tile<true, true, KIND>(p, io_dtype, stream);
  if (a_km && !b_km) return launch_tile<true, false, KIND>(p, io_dtype, stream);
  if (!a_km && !b_km) return launch_tile<false, false, KIND>(p, io_dtype, stream);
  LT_FAIL(LT_ERR_UNSUPPORTED, "tiled bf16 gemm: layout A mn-major x B k-major is not instantiated");
}

}  // namespace

bool lt_gemm_mfma_supported(const GemmProblem& p, int kind) {
  constexpr int BM = 256, BN = 256;
  const bool gated = kind == EPI_ACT_FWD && p.epi.gated;
  if (p.M <= 0 || p.N <= 0) return false;
  if (p.N % (gated ? BN / 2 : BN) != 0) return false;
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  if (!a_km && b_km) return false;
  if (!a_km && p.M % BM != 0) return false;  // mn-major A has no row clamp
  if ((int64_t)((p.M + BM - 1) / BM) * (p.N / (gated ? BN / 2 : BN)) > 0x7fffffff) return false;
  // the epilogue moves 8 columns at a time
  const EpiParams& e = p.epi;
  if (e.bias && !lt_aligned(e.bias, 16)) return false;
  if (kind == EPI_STORE && (e.ldo % 8 != 0 || !lt_aligned(e.out, 16))) return false;
  if ((kind == EPI_ACT_FWD || kind == EPI_ACT_BWD) &&
      (e.ld_pre % 8 != 0 || e.ld_hid % 8 != 0 || e.inter % 8 != 0 || !lt_aligned(e.pre, 16) ||
       (e.hid && !lt_aligned(e.hid, 16)) || (e.dpre && !lt_aligned(e.dpre, 16))))
    return false;
  if (kind == EPI_OUT && (e.ldy % 8 != 0 || !lt_aligned(e.y, 16) || (e.x && !lt_aligned(e.x, 16)))) return false;
  for (int s = 0; s < p.nseg; s++) {
    if ((bool)p.A[s].kmajor != a_km || (bool)p.B[s].kmajor != b_km) return false;
    if (p.K[s] <= 0) return false;
    // k-major operands are read in whole 64-element k-steps; mn-major ones are zero-filled past K
    if ((a_km || b_km) && p.K[s] % BK != 0) return false;
    if (p.A[s].ld % 8 != 0 || p.B[s].ld % 8 != 0) return false;
    if (!lt_aligned(p.A[s].ptr, 16) || !lt_aligned(p.B[s].ptr, 16)) return false;
  }
  return true;
}

static const char* mfma_tag(const GemmProblem& p, int kind) {
  static const char* names[3][4] = {
      {"gemm_bf16_nt_store", "gemm_bf16_nt_act_fwd", "gemm_bf16_nt_act_bwd", "gemm_bf16_nt_out"},
      {"gemm_bf16_nn_store", "gemm_bf16_nn_act_fwd", "gemm_bf16_nn_act_bwd", "gemm_bf16_nn_out"},
      {"gemm_bf16_tn_store", "gemm_bf16_tn_act_fwd", "gemm_bf16_tn_act_bwd", "gemm_bf16_tn_out"}};
  const int layout = p.A[0].kmajor ? (p.B[0].kmajor ? 0 : 1) : 2;
  return names[layout][kind];
}

double lt_gemm_flops(const GemmProblem& p, int kind) {
  const double n = (kind == EPI_ACT_FWD && p.epi.gated) ? 2.0 * p.N : (double)p.N;
  double k = (double)p.K[0] + (p.nseg > 1 ? (double)p.K[1] : 0.0);
  return 2.0 * (double)p.M * n * k;
}

int lt_launch_gemm_mfma(const GemmProblem& p, int kind, int io_dtype, hipStream_t stream) {
  LT_REQUIRE(lt_gemm_mfma_supported(p, kind), LT_ERR_UNSUPPORTED, "tiled bf16 gemm does not take this problem");
  LtProfileScope scope(mfma_tag(p, kind), lt_gemm_flops(p, kind), 0.0, stream);
  switch (kind) {
    case EPI_STORE: return launch_layout<EPI_STORE>(p, io_dtype, stream);
    case EPI_ACT_FWD: return launch_layout<EPI_ACT_FWD>(p, io_dtype, stream);
    case EPI_ACT_BWD: return launch_layout<EPI_ACT_BWD>(p, io_dtype, stream);
    case EPI_OUT: return launch_layout<EPI_OUT>(p, io_dtype, stream);
  }
  LT_FAIL(LT_ERR_BAD_ARG, "unknown epilogue kind %d", kind);
}

void lt_gemm_set_mfma_variant(int v) { g_mfma_variant = v; }

int lt_launch_gemm(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream) {
  if (dtype == LT_BF16 && lt_gemm_mfma_supported(p, kind)) return lt_launch_gemm_mfma(p, kind, io_dtype, stream);
  return lt_launch_gemm_generic(p, kind, dtype, io_dtype, stream);
}
