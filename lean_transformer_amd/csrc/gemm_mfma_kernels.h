// Kernels of the tiled bf16 GEMMs (internal header: included by gemm_mfma_bf16.hip for the host-side choices and by the
// per-epilogue translation units gemm_mfma_kind*.hip, which instantiate the kernels, so that they compile in parallel).
// Tiled bf16 GEMMs for gfx950 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulation) with the FFN epilogues fused.
// Two kernels share the LDS layouts and the epilogues:
//   gemm_bf16_dma_kernel  256 x 256 tile, operands copied global -> LDS without passing through registers; the kernel of
//                         the dense projections (second half of this file)
//   gemm_bf16_kernel      BM x BN tile, operands staged through registers; ragged reductions, the 128 x 128 tile of the
//                         skinny low-rank GEMMs, and the block-sparse walks over 64 x 64 blocks
//
// gemm_bf16_kernel.  Tile: BM x BN outputs per workgroup, 64 k per step, WM x WN wavefronts each owning a (BM/WM) x (BN/WN)
// sub-tile as 32 x 32 MFMA blocks.  Operand tiles go global -> registers -> LDS (16-byte accesses) and are double-buffered
// in LDS: while the matrix cores work on one stage the global loads of the next are in flight, with one barrier per k-step.
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
#pragma once
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "lt_gemm.h"

// Instrumented build (-DLT_TILE_TIMING, python tile_timing.py --build; never the product library):
// thread 0 of every workgroup of the copy-based kernel records the shader clock (s_memtime) when it starts, after the
// prologue, after 16 k-steps, after the main loop and after the epilogue, and the 100 MHz real-time counter at both ends,
// 8 words per workgroup, into the buffer whose address the environment variable LT_TILE_TIMING_BUFFER holds; copy-based
// launch number i of the process writes region i % 6 (4096 workgroups each), i.e. one region per GEMM of an FFN step.
// tile_timing.py (beside bench.py) reads them.
#ifdef LT_TILE_TIMING
int& lt_tile_timing_launch_counter();  // one counter for the whole library (defined in gemm_mfma_bf16.hip)
#define LT_TILE_STAMP(slot)                                                          \
  do {                                                                               \
    if (tile_stamps && threadIdx.x == 0) tile_stamps[slot] = __builtin_amdgcn_s_memtime(); \
  } while (0)
#define LT_TILE_STAMP_REALTIME(slot)                                                     \
  do {                                                                                   \
    if (tile_stamps && threadIdx.x == 0) tile_stamps[slot] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#else
#define LT_TILE_STAMP(slot) \
  do {                      \
  } while (0)
#define LT_TILE_STAMP_REALTIME(slot) \
  do {                               \
  } while (0)
#endif

namespace {

constexpr int BK = 64;
constexpr int GROUP_M = 8;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4;

__device__ __forceinline__ int swz_km(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_mn(int k) { return ((k & 3) << 2) | (((k >> 3) & 1) << 1); }
// mn-major tiles of COLS columns: the swizzle must stay inside a row's COLS / 8 chunks.  With 64 columns (128-byte rows,
// two rows per 256-byte bank line) k-rows 2 apart and 8 apart are the ones that would collide in a transposing read.
template <int COLS> __device__ __forceinline__ int swz_mn_cols(int k) {
  static_assert(COLS == 64 || COLS % 128 == 0, "mn-major tile width");
  if constexpr (COLS == 64) return (((k >> 1) & 1) << 1) | (((k >> 3) & 1) << 2);
  else return swz_mn(k);
}

// scheduling hint for one k-substep: spread READS LDS-read instructions evenly between MFMAS matrix instructions
template <int READS, int MFMAS, int G = 0> struct SchedInterleave {
  static __device__ __forceinline__ void run() {
    constexpr int n = READS * (G + 1) / MFMAS - READS * G / MFMAS;
    if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (G + 1 < MFMAS) SchedInterleave<READS, MFMAS, G + 1>::run();
  }
};

// SP != SPARSE_NONE: block-sparse walk with 64 x 64 blocks (see SparseWalk).  Each 64-wide k-step is one active block; its
// operand tiles are fetched through the index tables, so nothing is gathered or scattered in HBM.  tiles_n then counts
// groups: output blocks (FWD, tile 256 x 64), input blocks (DX, tile 256 x 64), or (input block, four of its active
// output blocks) (DW, tile 256 x 64: four gathered dY column blocks against one X column block, reduced over tokens;
// the four weight-gradient blocks are adjacent in the native [in_blocks, A, 64, 64] order).
// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{})
template <typename F, int... Is> __device__ __forceinline__ void lt_static_for_impl(F& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void lt_static_for(F&& f) {
  lt_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// PH = 2 (block-sparse forward with the gated activation epilogue only): a workgroup owns gate block tn and the matching
// linear block tn + N / 64, which have index lists of their own.  It walks the two lists one after the other (two phases
// over the same LDS stages) into two sets of accumulators and pairs them in the epilogue, so the gated activation needs no
// pass of its own over the pre-activations.
// PF: how many k-steps ahead of the matrix instructions the operand tiles are requested (in registers; the LDS holds two
// stages whatever PF is).  1 for the MFMA-bound uses; the rank-r products stream a large operand once against a small one and
// are bound by how many bytes a CU has in flight, so they ask further ahead.
template <int BM, int BN, int WM, int WN, bool A_KM, bool B_KM, int KIND, typename TX, int SP = SPARSE_NONE, int PH = 1, int PF = 1>
__global__ __launch_bounds__(WM * WN * 64)
__attribute__((amdgpu_waves_per_eu((SP != SPARSE_NONE || PF > 1) ? 2 : 1)))  // block-sparse walks, rank-r products: two workgroups per CU
void gemm_bf16_kernel(GemmProblem p, int tiles_m, int tiles_n) {
  constexpr int NT = WM * WN * 64;
  static_assert(PF == 1 || (SP == SPARSE_NONE && PH == 1), "deeper prefetch: dense single-phase only");
  static_assert(PH == 1 || (PH == 2 && SP == SPARSE_FWD && KIND == EPI_ACT_FWD && WN == 1), "two phases: gated block-sparse forward");
  static_assert(SP == SPARSE_NONE || (SP == SPARSE_FWD && A_KM && B_KM && BN == 64) ||
                    (SP == SPARSE_DX && A_KM && !B_KM && BN == 64) ||
                    (SP == SPARSE_DW && !A_KM && !B_KM && BM == 256 && BN == 64 && WM == 4 && WN == 1),
                "operand layouts and tile shape of the block-sparse walks");
  constexpr int WTM = BM / WM;
  constexpr int WTN_IN = BN / WN, FN_IN = WTN_IN / 32;  // columns / column blocks of a wavefront in one phase
  constexpr int WTN = WTN_IN * PH, FN = FN_IN * PH;     // ... and of its output sub-tile
  constexpr int FM = WTM / 32;
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

#ifdef LT_TILE_TIMING
  unsigned long long* const tile_stamps =
      ((SP == SPARSE_FWD || SP == SPARSE_DX) && p.tile_stamps) ? p.tile_stamps + (size_t)blockIdx.x * 8 : nullptr;
#endif
  LT_TILE_STAMP(0);
  LT_TILE_STAMP_REALTIME(4);
  // ---- tile assignment: XCD-contiguous, grouped along M
  int pid = blockIdx.x;
  const int num_pid = tiles_m * tiles_n;
  if ((num_pid & 7) == 0) pid = (pid & 7) * (num_pid >> 3) + (pid >> 3);
  // Block-sparse FWD / DX: the workgroups of one token tile gather column blocks of the same 256 activation rows (a few MiB
  // that stay in the XCD's L2) while every block column has a weight list of its own, so one XCD's concurrent workgroups
  // take one token tile and consecutive block columns.
  constexpr int GROUP_ROWS = (SP == SPARSE_FWD || SP == SPARSE_DX) ? 1 : GROUP_M;
  const int group = GROUP_ROWS * tiles_n;
  const int first_m = (pid / group) * GROUP_ROWS;
  const int gsz = min(tiles_m - first_m, GROUP_ROWS);
  const int tm = first_m + (pid % group) % gsz;
  const int tn = (pid % group) / gsz;
  const int64_t m0 = (int64_t)tm * BM;
  // gated: in gate columns; sparse FWD / DX: tn = block index (two phases: the gate block)
  const int64_t n0 = (int64_t)tn * ((gated && PH == 1) ? BN / 2 : BN);

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  u32x4 ra_set[PF][A_CHUNKS], rb_set[PF][B_CHUNKS];

  // k-steps: dense: segment 0 then segment 1; sparse FWD / DX: the active blocks of this group, then the low-rank segment
  const SparseWalk& sp = p.sp;
  const int sp_steps = SP == SPARSE_FWD ? sp.blocks_per_out : sp.blocks_per_in;
  const int kt_seg0 = SP == SPARSE_NONE ? (int)((p.K[0] + BK - 1) / BK)
                      : SP == SPARSE_DW ? (int)((sp.tokens + BK - 1) / BK)
                                        : sp_steps;
  const int kt_total = kt_seg0 + ((SP != SPARSE_DW && p.nseg > 1) ? (int)((p.K[1] + BK - 1) / BK) : 0);
  // sparse DW: group tn = (input block, quad of its active output blocks a0 .. a0 + 3); a short last quad repeats the last
  // block (computed, not stored)
  int dw_ib = 0, dw_a0 = 0, dw_valid = 0;
  int64_t dw_ob[4] = {0, 0, 0, 0};
  if constexpr (SP == SPARSE_DW) {
    const int quads = (sp.blocks_per_in + 3) / 4;
    dw_ib = tn / quads;
    dw_a0 = (tn % quads) * 4;
    dw_valid = min(4, sp.blocks_per_in - dw_a0);
#pragma unroll
    for (int j = 0; j < 4; j++)
      dw_ob[j] = sp.backward_indices[(int64_t)dw_ib * sp.blocks_per_in + min(dw_a0 + j, sp.blocks_per_in - 1)];
  }

  // position in the group's index list taken at step t of the walk (see SparseWalk::walk_run)
  auto walk_entry = [&](int t) {
    if (sp.walk_run <= 1) return t;
    const int runs = sp_steps / sp.walk_run;
    return (t % runs) * sp.walk_run + t / runs;
  };
  // global -> registers for k-step kt (ph: 0 = the tile's own block column, 1 = the matching linear block column)
  auto load_tiles = [&](int kt, int ph, u32x4 (&ra)[A_CHUNKS], u32x4 (&rb)[B_CHUNKS]) __attribute__((always_inline)) {
    const int seg = kt >= kt_seg0;
    int64_t k0 = (int64_t)(seg ? kt - kt_seg0 : kt) * BK;
    int64_t K = p.K[seg];
    const bf16* A = reinterpret_cast<const bf16*>(p.A[seg].ptr);
    const bf16* B = reinterpret_cast<const bf16*>(p.B[seg].ptr);
    int64_t lda = p.A[seg].ld, ldb = p.B[seg].ld;
    int64_t b_row0 = n0 + (PH == 2 ? ph * p.N : 0);  // first B row (k-major) / column (mn-major) of this tile
    if constexpr (SP == SPARSE_FWD) {
      if (!seg) {  // A: column block ib of X; B: weight block f, a [64 rows][64 k] matrix of its own
        const int f = sp.forward_indices[(int64_t)(tn + (PH == 2 ? ph * tiles_n : 0)) * sp.blocks_per_out + walk_entry(kt)];
        A = reinterpret_cast<const bf16*>(sp.act); lda = sp.ld_act; k0 = (int64_t)(f / sp.blocks_per_in) * 64;
        B = reinterpret_cast<const bf16*>(sp.weight) + (int64_t)f * 4096; ldb = 64; b_row0 = 0;
        K = k0 + 64;
      }
    } else if constexpr (SP == SPARSE_DX) {
      if (!seg) {  // A: column block ob of dY; B: weight block (ib, a) read as [64 k = output row][64 n = input column]
        const int a = walk_entry(kt);
        const int64_t ob = sp.backward_indices[(int64_t)tn * sp.blocks_per_in + a];
        A = reinterpret_cast<const bf16*>(sp.act); lda = sp.ld_act; k0 = ob * 64;
        B = reinterpret_cast<const bf16*>(sp.weight) + ((int64_t)tn * sp.blocks_per_in + a) * 4096 - k0 * 64; ldb = 64;
        b_row0 = 0;
        K = k0 + 64;
      }
    } else if constexpr (SP == SPARSE_DW) {  // A: four gathered dY column blocks; B: X column block ib; k = tokens
      A = reinterpret_cast<const bf16*>(sp.act); lda = sp.ld_act;
      B = reinterpret_cast<const bf16*>(sp.act2) + (int64_t)dw_ib * 64; ldb = sp.ld_act2; b_row0 = 0;
      K = sp.tokens;
    }
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (A_KM) {
        const int row = q >> 3, c = q & 7;
        const int64_t gm = min(m0 + row, p.M - 1);  // rows past M are clamped (their results are never stored)
        ra[i] = *reinterpret_cast<const u32x4*>(A + gm * lda + k0 + c * 8);
      } else {
        // rows past K: the last row again, zeroed on the way into LDS (store_tiles) -- a load under a branch would make
        // every later wait on the memory counter a wait for all of them, and no load could stay in flight across a step
        const int kr = q / (BM / 8), c = q % (BM / 8);
        const int64_t gk = min(k0 + kr, K - 1);
        int64_t col = m0 + c * 8;
        if constexpr (SP == SPARSE_DW) col = dw_ob[c >> 3] * 64 + (c & 7) * 8;
        ra[i] = *reinterpret_cast<const u32x4*>(A + gk * lda + col);
      }
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (B_KM) {
        const int row = q >> 3, c = q & 7;
        int64_t gn;
        if (gated && PH == 1) {
          const int rr = row % WTN;
          gn = (rr / (WTN / 2)) * p.N + n0 + (row / WTN) * (WTN / 2) + rr % (WTN / 2);
        } else {
          gn = b_row0 + row;
        }
        // a sparse FWD weight block holds its own 64 k: its columns start at 0, not at the gathered k0
        const int64_t bk0 = (SP == SPARSE_FWD && !seg) ? 0 : k0;
        rb[i] = *reinterpret_cast<const u32x4*>(B + gn * ldb + bk0 + c * 8);
      } else {
        const int kr = q / (BN / 8), c = q % (BN / 8);
        const int64_t gk = min(k0 + kr, K - 1);
        rb[i] = *reinterpret_cast<const u32x4*>(B + gk * ldb + b_row0 + c * 8);
      }
    }
  };
  // how many of the BK k-rows of step kt exist; mn-major operand tiles are zero-filled past them
  auto k_rows = [&](int kt) -> int {
    const int seg = kt >= kt_seg0;
    if ((SP == SPARSE_FWD || SP == SPARSE_DX) && !seg) return BK;
    const int64_t k0 = (int64_t)(seg ? kt - kt_seg0 : kt) * BK;
    const int64_t K = SP == SPARSE_DW ? (int64_t)sp.tokens : p.K[seg];
    return (int)min((int64_t)BK, K - k0);
  };
  // registers -> LDS stage s
  auto store_tiles = [&](int s, int rows, const u32x4 (&ra)[A_CHUNKS], const u32x4 (&rb)[B_CHUNKS]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (A_KM) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<u32x4*>(&lds_a[s][(row * 8 + (c ^ swz_km(row))) * 8]) = (PF == 1 || rows > 0) ? ra[i] : u32x4{0u, 0u, 0u, 0u};
      } else {
        const int kr = q / (BM / 8), c = q % (BM / 8);
        *reinterpret_cast<u32x4*>(&lds_a[s][kr * BM + ((c ^ swz_mn_cols<BM>(kr)) << 3)]) = kr < rows ? ra[i] : u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      const int q = tid + i * NT;
      if constexpr (B_KM) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<u32x4*>(&lds_b[s][(row * 8 + (c ^ swz_km(row))) * 8]) = (PF == 1 || rows > 0) ? rb[i] : u32x4{0u, 0u, 0u, 0u};
      } else {
        const int kr = q / (BN / 8), c = q % (BN / 8);
        *reinterpret_cast<u32x4*>(&lds_b[s][kr * BN + ((c ^ swz_mn_cols<BN>(kr)) << 3)]) = kr < rows ? rb[i] : u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  // one MFMA operand fragment (8 k values of row/column `lane & 31` of 32-wide block starting at `base`) for k-substep kk
  auto frag_km = [&](const bf16* tile, int base, int kk) -> bf16x8 {
    const int row = base + (lane & 31);
    const int c = kk * 2 + (lane >> 5);
    return *reinterpret_cast<const bf16x8*>(&tile[(row * 8 + (c ^ swz_km(row))) * 8]);
  };
  auto frag_mn = [&](const bf16* tile, auto cols_c, int base, int kk) -> bf16x8 {
    constexpr int cols = decltype(cols_c)::value;
    union { bf16x8 v; s16x4 h[2]; } u;
    const int i16 = lane & 15;
    const int col = base + ((lane >> 4) & 1) * 16 + 4 * (i16 & 3);
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int kr = kk * 16 + 8 * (lane >> 5) + 4 * s + (i16 >> 2);
      const bf16* src = &tile[kr * cols + ((((col >> 3) ^ swz_mn_cols<cols>(kr)) << 3) | (col & 7))];
      u.h[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(src));
    }
    return u.v;
  };

  auto load_frags = [&](int s, int kk, bf16x8 (&a)[FM], bf16x8 (&b)[FN_IN]) {
#pragma unroll
    for (int i = 0; i < FM; i++) {
      if constexpr (A_KM) a[i] = frag_km(lds_a[s], wm * WTM + i * 32, kk);
      else a[i] = frag_mn(lds_a[s], std::integral_constant<int, BM>{}, wm * WTM + i * 32, kk);
    }
#pragma unroll
    for (int j = 0; j < FN_IN; j++) {
      if constexpr (B_KM) b[j] = frag_km(lds_b[s], wn * WTN_IN + j * 32, kk);
      else b[j] = frag_mn(lds_b[s], std::integral_constant<int, BN>{}, wn * WTN_IN + j * 32, kk);
    }
  };
  constexpr int FRAG_READS = FM * (A_KM ? 1 : 2) + FN_IN * (B_KM ? 1 : 2);  // LDS read instructions per k-substep

  // split-k: this workgroup's slice of the k-steps
  int kt_begin = 0, kt_end = kt_total;
  if (p.ksplit > 1) {
    const int per = (kt_total + p.ksplit - 1) / p.ksplit;
    kt_begin = min(kt_total, (int)blockIdx.y * per);
    kt_end = min(kt_total, kt_begin + per);
  }
  // the matrix instructions of one k-step on LDS stage s.  Fragments are double-buffered in registers: the LDS reads of
  // k-substep kk + 1 are issued before, and interleaved with, the MFMAs of k-substep kk
  auto multiply_stage = [&](int s, auto PHASE) __attribute__((always_inline)) {
    constexpr int j0 = decltype(PHASE)::value * FN_IN;  // this phase's accumulator columns
    bf16x8 af[2][FM], bfr[2][FN_IN];
    load_frags(s, 0, af[0], bfr[0]);
#pragma unroll
    for (int kk = 0; kk < BK / 16; kk++) {
      if (kk + 1 < BK / 16) load_frags(s, kk + 1, af[(kk + 1) & 1], bfr[(kk + 1) & 1]);
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN_IN; j++)
          acc[i][j0 + j] = LT_MFMA_32X32X16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j0 + j]);
      if (kk + 1 < BK / 16) SchedInterleave<FRAG_READS, FM * FN_IN>::run();
    }
  };
  LT_TILE_STAMP(1);
  if constexpr (PF == 1) {
    lt_static_for<PH>([&](auto PHASE) __attribute__((always_inline)) {
      constexpr int ph = decltype(PHASE)::value;
      if (kt_begin < kt_end) {
        load_tiles(kt_begin, ph, ra_set[0], rb_set[0]);
        store_tiles(kt_begin & 1, k_rows(kt_begin), ra_set[0], rb_set[0]);
      }
      __syncthreads();
      for (int kt = kt_begin; kt < kt_end; kt++) {
        const int s = kt & 1;
        const bool has_next = kt + 1 < kt_end;
        if (has_next) load_tiles(kt + 1, ph, ra_set[0], rb_set[0]);
        multiply_stage(s, PHASE);
        if (has_next) store_tiles(s ^ 1, k_rows(kt + 1), ra_set[0], rb_set[0]);
        __syncthreads();
      }
    });
  } else {
    // Register set d holds step i with i % PF == d from its request until it is written to LDS stage i & 1 at the end of
    // step i - 1; the set is then free for step i + PF, requested at the start of step i.
    // A k-major operand with a power-of-two row pitch: the 128 rows of a tile, and the same k-step of every tile row, sit
    // on the same memory channels, so tile row tm starts its walk over the slice tm steps in and wraps around.
    // Nothing in the loop is conditional (a load or an LDS write under a branch makes every later wait on the memory counter
    // a wait for all loads): the walk is padded to a multiple of PF steps, requests past its end repeat the last tile and
    // such a tile is written to LDS as zeros.
    const int steps = kt_end - kt_begin;
    if (steps > 0) {
      const int padded = (steps + PF - 1) / PF * PF;
      const int rot = (A_KM && steps > 1) ? tm % steps : 0;
      auto kt_of = [&](int i) {
        const int j = min(i, steps - 1) + rot;
        return kt_begin + (j >= steps ? j - steps : j);
      };
      auto rows_of = [&](int i) { return i < steps ? k_rows(kt_of(i)) : 0; };
      lt_static_for<PF>([&](auto D) __attribute__((always_inline)) {
        constexpr int d = decltype(D)::value;
        load_tiles(kt_of(d), 0, ra_set[d], rb_set[d]);
      });
      store_tiles(0, rows_of(0), ra_set[0], rb_set[0]);
      __syncthreads();
      for (int i0 = 0; i0 < padded; i0 += PF) {
        lt_static_for<PF>([&](auto D) __attribute__((always_inline)) {
          constexpr int d = decltype(D)::value;
          const int i = i0 + d;
          const int s = i & 1;
          load_tiles(kt_of(i + PF), 0, ra_set[d], rb_set[d]);
          multiply_stage(s, std::integral_constant<int, 0>{});
          store_tiles(s ^ 1, rows_of(i + 1), ra_set[(d + 1) % PF], rb_set[(d + 1) % PF]);
          __syncthreads();
        });
      }
    }
  }
  LT_TILE_STAMP(2);

  // ---- epilogue.  The accumulators of a 32 x 32 block sit column-per-lane (register r = row 8 * (r / 4) + 4 * (lane / 32)
  //      + r % 4, column lane % 32); each wavefront transposes one 32-row strip of its sub-tile at a time through its own
  //      LDS region and reads it back row-major, 8 consecutive columns per lane, so that the fused epilogue reads and
  //      writes HBM in 16-byte pieces of contiguous rows.  (The main loop ended with a barrier: the stages are free.)
  float* stage = reinterpret_cast<float*>(smem) + wave * (32 * STAGE_LD);
  const bool pair = (KIND == EPI_ACT_FWD) && gated;
  // sparse DW: the tile is the [4 x 64][64] stack of weight-gradient blocks (ib, a0 .. a0 + 3), adjacent in memory
  EpiParams epi = p.epi;
  int64_t m_limit = p.M, n_base = n0 + wn * WTN, m_base = m0;
  if (p.ksplit > 1) epi.out = reinterpret_cast<float*>(epi.out) + (int64_t)blockIdx.y * p.split_stride;
  if constexpr (SP == SPARSE_DW) {
    epi.out = reinterpret_cast<char*>(epi.out) +
              ((int64_t)dw_ib * sp.blocks_per_in + dw_a0) * 4096 * (epi.out_dtype == LT_F32 ? 4 : 2);
    epi.ldo = 64;
    m_limit = dw_valid * 64;
    n_base = 0;
    m_base = 0;
  }
  // The bias is added while the accumulators are staged (a lane holds one column per 32-wide block), so no epilogue body has
  // to.  Gated forward: the first half of a wavefront's column blocks are gate columns, the second half the matching linear
  // columns.  (A split reduction passes no bias; the sparse weight-gradient walk has none.)
  float bias0[FN];
#pragma unroll
  for (int j = 0; j < FN; j++) {
    bias0[j] = 0.f;
    if (SP != SPARSE_DW && epi.bias) {
      const int64_t col = gated ? (j >= FN / 2 ? epi.inter : 0) + n0 + wn * (WTN / 2) + (j % (FN / 2 > 0 ? FN / 2 : 1)) * 32 + (lane & 31)
                                : n0 + wn * WTN + j * 32 + (lane & 31);
      bias0[j] = epi.bias[col];
    }
  }
  epi.bias = nullptr;
  auto stage_strip = [&](auto I) __attribute__((always_inline)) {
    constexpr int i = decltype(I)::value;
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * STAGE_LD + j * 32 + (lane & 31)] = acc[i][j][r] + bias0[j];
    __builtin_amdgcn_wave_barrier();
  };
  // general strip: every choice (row in range, output type, activation, dropout, ...) is made per row
  auto generic_strip = [&](auto I) __attribute__((always_inline)) {
    constexpr int i = decltype(I)::value;
    stage_strip(I);
    const int64_t mrow0 = m_base + wm * WTM + i * 32;
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
        if (m < p.M) epi_act_fwd_gated8(epi, m, n0 + wn * (WTN / 2) + c, vg, vl);
      }
    } else {
      constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        const int64_t n = n_base + c;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = stage[row * STAGE_LD + c + e];
        if (m < m_limit) {
          if constexpr (KIND == EPI_STORE) epi_store8(epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_FWD) epi_act_fwd8(epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_BWD) epi_act_bwd8(epi, m, n, v);
          else epi_out8<TX>(epi, m, n, v);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  };
  // Straight-line strips for whole tiles in the usual configurations: the choices are made once per tile and the global
  // reads of a strip (pre-activations, residual) go out before the strip is staged.
  constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
  const int lane_c = (lane % LANES_PER_ROW) * 8;
  const int64_t lane_n = n_base + lane_c;
  auto lane_row = [&](int i) -> int64_t { return m_base + wm * WTM + i * 32 + lane / LANES_PER_ROW; };
  auto read_staged = [&](int it, float (&v)[8]) {
    const float* sv = &stage[(it * ROWS_PER_IT + lane / LANES_PER_ROW) * STAGE_LD + lane_c];
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = sv[e];
  };
  auto store_strip = [&](auto I, auto out_type) __attribute__((always_inline)) {
    using TO = decltype(out_type);
    constexpr int i = decltype(I)::value;
    stage_strip(I);
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      float v[8];
      read_staged(it, v);
      epi_store8_plain<TO>(epi, lane_row(i) + it * ROWS_PER_IT, lane_n, v);
    }
    __builtin_amdgcn_wave_barrier();
  };
  float colsum[16];  // EPI_ACT_BWD: column sums of this lane's 8 (+ 8) dpre columns over the rows it writes
#pragma unroll
  for (int e = 0; e < 16; e++) colsum[e] = 0.f;
  auto act_bwd_strip = [&](auto I, auto G) __attribute__((always_inline)) {
    constexpr int i = decltype(I)::value;
    constexpr bool GATED = decltype(G)::value;
    EpiLoad rows[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) rows[it] = epi_load_pre8<GATED>(epi, lane_row(i) + it * ROWS_PER_IT, lane_n);
    stage_strip(I);
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      float v[8];
      read_staged(it, v);
      epi_act_bwd8_gelu<GATED>(epi, lane_row(i) + it * ROWS_PER_IT, lane_n, v, rows[it], colsum);
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto out_strip = [&](auto I) __attribute__((always_inline)) {
    constexpr int i = decltype(I)::value;
    EpiLoad rows[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) rows[it] = epi_load_x8<TX>(epi, lane_row(i) + it * ROWS_PER_IT, lane_n);
    stage_strip(I);
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      float v[8];
      read_staged(it, v);
      epi_out8_residual<TX>(epi, lane_row(i) + it * ROWS_PER_IT, lane_n, v, rows[it]);
    }
    __builtin_amdgcn_wave_barrier();
  };
  // forward activation, tanh GELU, h stored: the gate (or only) half and the linear half of a strip are read back from the
  // stage with all LDS loads issued before the first value is used
  auto act_fwd_strip = [&](auto I, auto G) __attribute__((always_inline)) {
    constexpr int i = decltype(I)::value;
    constexpr bool GATED = decltype(G)::value;
    constexpr int LPR = (GATED ? WTN / 2 : WTN) / 8, RPI = 64 / LPR, NITF = 32 / RPI;
    const int c = (lane % LPR) * 8;
    const int64_t n = n0 + wn * (GATED ? WTN / 2 : WTN) + c;
    const int64_t mlane = m_base + wm * WTM + i * 32 + lane / LPR;
    stage_strip(I);
    float vg[NITF][8], vl[GATED ? NITF : 1][8];
#pragma unroll
    for (int it = 0; it < NITF; it++) {
      const float* sv = &stage[(it * RPI + lane / LPR) * STAGE_LD + c];
#pragma unroll
      for (int e = 0; e < 8; e++) vg[it][e] = sv[e];
      if constexpr (GATED) {
#pragma unroll
        for (int e = 0; e < 8; e++) vl[it][e] = sv[WTN / 2 + e];
      }
    }
#pragma unroll
    for (int it = 0; it < NITF; it++) epi_act_fwd8_gelu<GATED>(epi, mlane + it * RPI, n, vg[it], vl[GATED ? it : 0]);
    __builtin_amdgcn_wave_barrier();
  };
  const bool whole_tile = m_base + BM <= m_limit;
  if constexpr (KIND == EPI_ACT_FWD && SP != SPARSE_NONE) {
    const bool straight = whole_tile && epi.act == LT_ACT_GELU_FUSED && epi.hid != nullptr && epi.pre != nullptr;
    if (straight && pair) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { act_fwd_strip(I, std::true_type{}); });
    else if (straight) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { act_fwd_strip(I, std::false_type{}); });
    else lt_static_for<FM>(generic_strip);
  } else if constexpr (NIT <= 4 && KIND == EPI_STORE) {
    if (whole_tile && epi.out_dtype == LT_F32) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { store_strip(I, float{}); });
    else if (whole_tile) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { store_strip(I, bf16{}); });
    else lt_static_for<FM>(generic_strip);
  } else if constexpr (NIT <= 4 && KIND == EPI_ACT_BWD) {
    const bool straight = whole_tile && epi.act == LT_ACT_GELU_FUSED && epi.hid != nullptr;
    if (straight && epi.gated) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { act_bwd_strip(I, std::true_type{}); });
    else if (straight) lt_static_for<FM>([&](auto I) __attribute__((always_inline)) { act_bwd_strip(I, std::false_type{}); });
    else lt_static_for<FM>(generic_strip);
    if (straight && epi.colsum) {
      // lanes with equal lane % LANES_PER_ROW hold the same columns for different rows of the wavefront's WTM-row sub-tile:
      // one partial row per wavefront sub-tile
      static_assert(WTM == 64 || KIND != EPI_ACT_BWD || NIT > 4, "the caller reduces one partial row per 64 output rows");
#pragma unroll
      for (int e = 0; e < 16; e++) {
#pragma unroll
        for (int d = LANES_PER_ROW; d < 64; d <<= 1) colsum[e] += __shfl_xor(colsum[e], d);
      }
      if (lane < LANES_PER_ROW) {
        float* dst = epi.colsum + ((m_base + wm * WTM) / 64) * epi.ld_pre + lane_n;
        float lo[8], hi[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          lo[e] = colsum[e];
          hi[e] = colsum[8 + e];
        }
        store8(dst, lo);
        if (epi.gated) store8(dst + epi.inter, hi);
      }
    }
  } else if constexpr (NIT <= 4 && KIND == EPI_OUT) {
    if (whole_tile && epi.x && epi.drop.p == 0.f) lt_static_for<FM>(out_strip);
    else lt_static_for<FM>(generic_strip);
  } else {
    lt_static_for<FM>(generic_strip);
  }
  LT_TILE_STAMP(3);
  LT_TILE_STAMP_REALTIME(5);
}

// =====================================================================================================================
// Variant with asynchronous global -> LDS copies (global_load_lds_dwordx4): operand tiles never pass through registers.
// A wavefront's copy instruction deposits the 64 lanes' 16-byte pieces at consecutive LDS addresses (lane i at base + 16 i),
// so the swizzled LDS layouts are produced by choosing which global chunk each lane fetches.
//
// Tile 256 x 256, 4 wavefronts (2 x 2, 128 x 128 each), k-steps of 32, k-loop unrolled by 4.  Per operand, 64 KiB of LDS:
//   mn-major  a ring of four [32 k][256] tiles, one k-step each; every row of a tile is 512 contiguous bytes in HBM.  The
//             copy of k-step kt + 3 is issued during k-step kt.
//   k-major   two [256][64 k] buffers, one block of two k-steps each, so that every row contributes a full 128-byte line
//             to a copy (with 32 k per copy the L2 would see twice as many half-line requests).  The two halves of the
//             copy of block kt / 2 + 1 go out in slots around the even k-step kt (BlockSlots below).
// Every LDS buffer is a separate array, so that copies into one provably do not alias reads of another.
// Pipeline of k-step kt:
//     matrix instructions on the first 16 k (fragments already in registers)
//         interleaved with: LDS reads of the second 16 k, the copies listed above
//     wait until this wavefront's copies of k-step kt + 1 have landed and its LDS reads are done; workgroup barrier
//     matrix instructions on the second 16 k
//         interleaved with: LDS reads of the first 16 k of k-step kt + 1
// so no LDS read latency is exposed after the barrier and copies have 1 to 2.5 k-steps to land.  The epilogue stages the
// accumulators through LDS one 32-row strip at a time; whole tiles in the usual configurations take straight-line strips.
// =====================================================================================================================
__device__ const u32x4 lt_zero_chunk = {0u, 0u, 0u, 0u};  // source of the lanes past the end of a ragged reduction

constexpr int DK = 32;  // k per step of the copy-based kernel

// scheduling hint for one half k-step: READS LDS reads over the first READ_SPAN of MFMAS matrix instructions and COPIES
// global->LDS copies evenly over all of them (packing the reads into the first quarter measured slower)
template <int READS, int COPIES, int MFMAS, int READ_SPAN, int G = 0> struct SchedInterleave3 {
  static __device__ __forceinline__ void run() {
    // the LDS reads go out over the first SPAN matrix instructions, the copies over all of them
    constexpr int SPAN = READ_SPAN < MFMAS ? READ_SPAN : MFMAS;
    constexpr int g0 = G < SPAN ? G : SPAN, g1 = G + 1 < SPAN ? G + 1 : SPAN;
    constexpr int nr = READS * g1 / SPAN - READS * g0 / SPAN;
    constexpr int nc = COPIES * (G + 1) / MFMAS - COPIES * G / MFMAS;
    if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
    if constexpr (nc > 0) __builtin_amdgcn_sched_group_barrier(0x020, nc, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (G + 1 < MFMAS) SchedInterleave3<READS, COPIES, MFMAS, READ_SPAN, G + 1>::run();
  }
};

// wait until at most N of this wavefront's copies are in flight and (WAIT_LDS) all its LDS reads have returned, then barrier.
// The wait is a real s_waitcnt instruction (not inline assembly) so that the compiler's own wait-count bookkeeping sees
// that older copies have landed; the empty asm statements only keep it from moving LDS accesses across the barrier.
template <int N, bool WAIT_LDS = true> __device__ __forceinline__ void wait_copies_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  // vmcnt(N) expcnt(7: none) lgkmcnt(0, or 15: none)
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | ((WAIT_LDS ? 0 : 15) << 8));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Per-lane copy state of one operand: byte offsets of this wavefront's copy instructions relative to a wavefront-uniform
// base that advances by `unit_bytes` per copy unit (k-major: a block of 64 k; mn-major: a k-step of 32 k).
template <bool KM> struct DmaOperand {
  static constexpr int LOADS = KM ? 8 : 4;  // copy instructions per wavefront per unit (32 or 16 KiB / 4 wavefronts / 1 KiB)
  uint32_t off[LOADS];
  int krow[LOADS];  // mn-major: k-row inside the k-step (for the ragged-reduction test)
  const char* base;
  int64_t unit_bytes;
  int seg;

  // row0: first row / column of the tile; the operand has row_limit of them.  A tile that sticks out past row_limit copies
  // the last row (k-major) or the last 8 columns (mn-major; row_limit is a multiple of 8) again in place of what is not
  // there: those only feed result rows / columns that the epilogue does not write.  k-major with pair_rows > 0: tile row r
  // maps to the gated up-projection's weight rows (gate half, then linear half at + pair_rows), 64 of each per 128-row
  // wavefront sub-tile.
  __device__ __forceinline__ void setup(const GemmOperand& op, int s, int64_t row0, int64_t row_limit, int64_t pair_rows,
                                        int wave, int lane) {
    seg = __builtin_amdgcn_readfirstlane(s);
    const int64_t ld = op.ld;
    const char* ptr = reinterpret_cast<const char*>(op.ptr);
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
      const int q = (wave * LOADS + j) * 64 + lane;  // 16-byte slot of the LDS buffer this lane fills
      if constexpr (KM) {
        const int row = q >> 3, c = (q & 7) ^ swz_km(row);
        const int local = pair_rows > 0 ? (row >> 7) * 64 + (row & 63) : row;
        int64_t g = min(row0 + local, row_limit - 1) - row0;
        if (pair_rows > 0) g += ((row & 127) >> 6) * pair_rows;
        off[j] = (uint32_t)((g * ld + c * 8) * 2);
        krow[j] = 0;
      } else {
        const int kr = q >> 5, c = (q & 31) ^ swz_mn(kr);
        const int64_t col = min(row0 + c * 8, row_limit - 8) - row0;
        off[j] = (uint32_t)((kr * ld + col) * 2);
        krow[j] = kr;
      }
    }
    base = KM ? ptr + row0 * ld * 2 : ptr + row0 * 2;
    unit_bytes = KM ? 64 * 2 : DK * ld * 2;
  }

  // mn-major operand whose 256 tile columns are four 64-wide column blocks gathered from anywhere in the matrix: block j of
  // the tile is the operand's column block blocks[j]
  __device__ __forceinline__ void setup_gather(const GemmOperand& op, const int (&blocks)[4], int wave, int lane) {
    static_assert(!KM, "column blocks are gathered for mn-major operands");
    seg = 0;
    const int64_t ld = op.ld;
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
      const int q = (wave * LOADS + j) * 64 + lane;
      const int kr = q >> 5, c = (q & 31) ^ swz_mn(kr);
      const int slot = c >> 3;
      const int blk = slot == 0 ? blocks[0] : slot == 1 ? blocks[1] : slot == 2 ? blocks[2] : blocks[3];
      off[j] = (uint32_t)((kr * ld + (int64_t)blk * 64 + (c & 7) * 8) * 2);
      krow[j] = kr;
    }
    base = reinterpret_cast<const char*>(op.ptr);
    unit_bytes = DK * ld * 2;
  }

  // all copies of unit u (counted inside the k-segment) into `dst`; k_limit: reduction length for the ragged test
  // J0, J1: range of this wavefront's copy instructions (a k-major block can go out in two halves)
  template <bool K_TAIL, int J0 = 0, int J1 = LOADS>
  __device__ __forceinline__ void issue(int u, bf16* dst, int wave, int64_t k_limit) const {
    if constexpr (!(K_TAIL && !KM)) {
      // Buffer form: wavefront-uniform descriptor of the unit + the lane's 32-bit offset.  No vector address arithmetic,
      // and unlike the global form the compiler does not count it as a FLAT access, after which it turns every wait for
      // LDS data into a wait for all of it.
      const __amdgpu_buffer_rsrc_t rsrc =
          __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base + u * unit_bytes), 0, -1, 0x00020000);
#pragma unroll
      for (int j = J0; j < J1; j++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + (wave * LOADS + j) * 512),
                                                 16, (int)off[j], 0, 0, 0);
      return;
    }
    // ragged reduction over mn-major operands: lanes past the end read a chunk of zeros instead
#pragma unroll
    for (int j = J0; j < J1; j++) {
      const char* g = base + u * unit_bytes + off[j];
      if constexpr (K_TAIL && !KM) {
        if ((int64_t)u * DK + krow[j] >= k_limit) g = reinterpret_cast<const char*>(&lt_zero_chunk);
      }
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                       (__attribute__((address_space(3))) void*)(dst + (wave * LOADS + j) * 512), 16, 0, 0);
    }
  }
};

// Where the two halves (4 copy instructions per wavefront each) of a k-major block go out.  The buffer of the block that
// holds k-steps 2b + 2, 2b + 3 is free after the barrier of k-step 2b - 1 and must be full at the barrier of 2b + 1:
//   slot 0: second half of k-step 2b - 1      slot 1: first half of 2b      slot 2: second half of 2b
struct BlockSlots {
  int half[2];
};

// Copies complete in issue order, so the wait before the barrier of k-step t names how many of the youngest copies may
// still be in flight: those issued after the last copy k-step t + 1 reads.  This replays the issue order of the steady
// loop and counts them.  First half of s: mn-major A and B for s + 3 (B only when not split), then on even s the slot-1
// halves of the k-major blocks of s + 2; second half of s, after its barrier: split mn-major B for s + 3, then on odd s
// the slot-0 halves of the blocks of s + 3, on even s the slot-2 halves of the blocks of s + 2.
constexpr int copies_in_flight(bool a_km, bool b_km, BlockSlots sa, BlockSlots sb, bool b_split, int parity) {
  const int t = 8 + parity;
  int counts[128] = {}, needed[128] = {}, n = 0;
  for (int s = t - 8; s <= t; s++) {
    if (!a_km) { counts[n] = 4; needed[n++] = s + 3; }
    if (!b_km && !b_split) { counts[n] = 4; needed[n++] = s + 3; }
    if (s % 2 == 0) {
      for (int h = 0; h < 2; h++) if (a_km && sa.half[h] == 1) { counts[n] = 4; needed[n++] = s + 2; }
      for (int h = 0; h < 2; h++) if (b_km && sb.half[h] == 1) { counts[n] = 4; needed[n++] = s + 2; }
    }
    if (s == t) break;
    if (!b_km && b_split) { counts[n] = 4; needed[n++] = s + 3; }
    const int want = s % 2 ? 0 : 2, first = s % 2 ? s + 3 : s + 2;
    for (int h = 0; h < 2; h++) if (a_km && sa.half[h] == want) { counts[n] = 4; needed[n++] = first; }
    for (int h = 0; h < 2; h++) if (b_km && sb.half[h] == want) { counts[n] = 4; needed[n++] = first; }
  }
  int last = -1;
  for (int i = 0; i < n; i++)
    if (needed[i] <= t + 1) last = i;
  int sum = 0;
  for (int i = last + 1; i < n; i++) sum += counts[i];
  return sum;
}
static_assert(copies_in_flight(false, false, {}, {}, false, 0) == 16 && copies_in_flight(true, true, {{1, 1}}, {{1, 1}}, false, 1) == 0 &&
              copies_in_flight(true, true, {{1, 1}}, {{1, 1}}, false, 0) == 16 && copies_in_flight(true, false, {{1, 1}}, {}, false, 1) == 4 &&
              copies_in_flight(true, false, {{1, 1}}, {}, false, 0) == 16 && copies_in_flight(true, true, {{0, 0}}, {{1, 1}}, false, 0) == 16 &&
              copies_in_flight(true, true, {{0, 0}}, {{1, 1}}, false, 1) == 0 && copies_in_flight(false, false, {}, {}, true, 0) == 12,
              "issue-order model");

// Measured choices (config-3 GEMM shapes): two k-major operands -- A block right after the odd barrier, B block after the
// even one; k-major A next to mn-major B -- A split over both barriers; two mn-major operands -- B in the second half-step.
constexpr BlockSlots SLOTS_NT_A = {{0, 0}}, SLOTS_NT_B = {{2, 2}}, SLOTS_NN_A = {{0, 2}};
constexpr bool SPLIT_MN_B = true;

// Block number of member j (0 .. 3) of the quad of run members that tile index t stands for.  Runs of `len` blocks that share
// one list are either consecutive (stride 0 or 1: tile t is blocks 4 t .. 4 t + 3) or `stride` blocks apart (a layout tiled
// from a square pattern `stride` blocks wide: run r is blocks r, r + stride, ...; tile t is quad t % (len / 4) of run
// t / (len / 4)).
__device__ __forceinline__ int lt_run_member(int t, int j, int len, int stride) {
  if (stride <= 1) return t * 4 + j;
  const int quads = len >> 2;
  return t / quads + stride * ((t % quads) * 4 + j);
}

// Epilogue of one wavefront's (FM * 32) x 128 sub-tile of a copy-based kernel: acc[i][j] is the 32 x 32 block at rows
// m0 + wm * WTM + 32 i, columns n0 + wn * 128 + 32 j of the result (gated forward: blocks 0, 1 gate columns, 2, 3 the
// matching linear columns).  `stage` is 16 KiB of LDS that belongs to this wavefront alone; tile_rows x tile_cols is the
// workgroup's tile (for the whole-tile test).  The bias is already in the accumulators.
// SCATTER (EPI_STORE only; the grouped block-sparse weight gradient): the tile is 4 output blocks (rows) x 4 entries of
// their shared list of input blocks (columns); each 64 x 64 piece goes to its own block of the native [in, A, block] weight
// gradient, at the flat position the forward table names.  List entries past the end (the last column tile) are not stored.
// SCATTER == 2: the tile is 4 entries of a list of output blocks (rows) x the run of 4 input blocks that shares the list
// (columns); piece (entry a, input block ib) is block ib * blocks_per_in + a.
template <int FM, int KIND, typename TX, int tile_rows, int tile_cols, int SCATTER = 0>
__device__ __forceinline__ void dma_tile_epilogue(f32x16 (&acc)[FM][4], const GemmProblem& p, float* stage, const int64_t m0,
                                                  const int64_t n0, const int wm, const int wn, const bool gated) {
  constexpr int FN = 4, WTN = 128, WTM = FM * 32;
  // the lane index is formed anew rather than kept in a register across the main loop, through an asm statement so that a
  // workgroup that loops over tiles does not keep what is derived from it alive from one tile's epilogue to the next's either
  int lane;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
  // ---- epilogue.  The accumulators of a 32 x 32 block sit column-per-lane (register r = row 8 * (r / 4) + 4 * (lane / 32)
  //      + r % 4, column lane % 32).  Each wavefront transposes one 32-row strip of its sub-tile at a time through an LDS
  //      buffer of its own (32 x 128 floats = 16 KiB, the size of the smallest buffer) and reads it back row-major, 8
  //      consecutive columns per lane, so that the fused epilogue reads and writes HBM in 16-byte pieces of contiguous rows.
  //      Staged column c of row r sits at c ^ 32 when bit 2 of r is set: the two half-waves of a transposing write (rows
  //      r and r + 4, same columns) then hit different banks without padding the rows.
  EpiParams epi = p.epi;
  epi.bias = nullptr;  // already in the accumulators
  if (KIND == EPI_STORE && p.ksplit > 1) epi.out = reinterpret_cast<float*>(epi.out) + (int64_t)blockIdx.y * p.split_stride;
  auto staged = [&](int row, int col) -> float* { return &stage[row * WTN + (col ^ (((row >> 2) & 1) << 5))]; };
  const bool pair = (KIND == EPI_ACT_FWD) && gated;
  float colsum[16];  // EPI_ACT_BWD: column sums of this lane's 8 (+ 8) dpre columns over the rows it writes
#pragma unroll
  for (int e = 0; e < 16; e++) colsum[e] = 0.f;
  // accumulators of strip I -> this wavefront's staging buffer
  auto stage_strip = [&](auto I) {
    constexpr int i = decltype(I)::value;
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) *staged(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), j * 32 + (lane & 31)) = acc[i][j][r];
    __builtin_amdgcn_wave_barrier();
  };
  auto for_each_strip = [&](auto&& strip) { lt_static_for<FM>(strip); };
  auto generic_strip = [&](auto I) {
    constexpr int i = decltype(I)::value;
    stage_strip(I);
    const int64_t mrow0 = m0 + wm * WTM + i * 32;
    if (pair) {
      // columns [0, WTN/2) of the sub-tile are gate columns, [WTN/2, WTN) the matching linear columns
      constexpr int LANES_PER_ROW = WTN / 2 / 8, ROWS_PER_IT = 64 / LANES_PER_ROW;
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
        const int64_t m = mrow0 + row;
        float vg[8], vl[8];
        const float* sg = staged(row, c);
        const float* sl = staged(row, WTN / 2 + c);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          vg[e] = sg[e];
          vl[e] = sl[e];
        }
        const int64_t n = n0 + wn * (WTN / 2) + c;
        if (m < p.M && n < p.N) epi_act_fwd_gated8(epi, m, n, vg, vl);
      }
    } else {
      constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
      const int c = (lane % LANES_PER_ROW) * 8;
      const int64_t n = n0 + wn * WTN + c;
      const bool in_n = n < p.N;  // N is a multiple of 8: the lane's 8 columns are all inside or all outside
      const int64_t mlane = mrow0 + lane / LANES_PER_ROW;  // this lane's row in iteration 0
      // global reads of the epilogue run two iterations ahead of their use
      EpiLoad l0 = epi_load8<KIND, TX>(epi, mlane, n, in_n && mlane < p.M);
      EpiLoad l1 = epi_load8<KIND, TX>(epi, mlane + ROWS_PER_IT, n, in_n && mlane + ROWS_PER_IT < p.M);
      for (int it = 0; it < NIT; it++) {
        const int row = it * ROWS_PER_IT + lane / LANES_PER_ROW;
        const int64_t m = mrow0 + row;
        const int64_t m2 = m + 2 * ROWS_PER_IT;
        const EpiLoad l2 = epi_load8<KIND, TX>(epi, m2, n, in_n && it + 2 < NIT && m2 < p.M);
        float v[8];
        const float* sv = staged(row, c);
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = sv[e];
        if (in_n && m < p.M) {
          if constexpr (KIND == EPI_STORE) epi_store8(epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_FWD) epi_act_fwd8(epi, m, n, v);
          else if constexpr (KIND == EPI_ACT_BWD) epi_act_bwd8_loaded(epi, m, n, v, l0, colsum);
          else epi_out8_loaded<TX>(epi, m, n, v, l0);
        }
        l0 = l1;
        l1 = l2;
      }
    }
    __builtin_amdgcn_wave_barrier();
  };
  // One lane's share of the staged strip: NIT rows x 8 columns starting at column c, fetched with 16-byte LDS reads that all
  // go out before the first value is used, so that a strip exposes the LDS latency once and not once per row (one wavefront
  // per SIMD: nobody else would hide it).  The registers come from the accumulators of the strip just staged.
  auto read_staged_rows = [&](auto nit_c, auto rows_per_it_c, int lanes_per_row, int c, float (&v)[decltype(nit_c)::value][8]) {
    constexpr int NIT_ = decltype(nit_c)::value, RPI = decltype(rows_per_it_c)::value;
    f32x4 raw[NIT_][2];
#pragma unroll
    for (int it = 0; it < NIT_; it++) {
      const float* sv = staged(it * RPI + lane / lanes_per_row, c);
      raw[it][0] = *reinterpret_cast<const f32x4*>(sv);
      raw[it][1] = *reinterpret_cast<const f32x4*>(sv + 4);
    }
#pragma unroll
    for (int it = 0; it < NIT_; it++)
#pragma unroll
      for (int e = 0; e < 8; e++) v[it][e] = raw[it][e >> 2][e & 3];
  };
  // EPI_ACT_BWD, the usual case (whole tile in range, tanh GELU, h wanted): straight-line strips.  The pre-activation reads
  // of ACT_WINDOW rows are in flight at any time -- the first window goes out before the strip is staged -- and, with no
  // branches in between, each row waits only for its own reads.
  constexpr int ACT_WINDOW = 3;
  auto act_bwd_strip = [&](auto I, auto G) {
    constexpr int i = decltype(I)::value;
    constexpr bool GATED = decltype(G)::value;
    constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
    const int c = (lane % LANES_PER_ROW) * 8;
    const int64_t n = n0 + wn * WTN + c;
    const int64_t mlane = m0 + wm * WTM + i * 32 + lane / LANES_PER_ROW;
    EpiLoad win[ACT_WINDOW];
#pragma unroll
    for (int it = 0; it < ACT_WINDOW; it++) win[it] = epi_load_pre8<GATED>(epi, mlane + it * ROWS_PER_IT, n);
    stage_strip(I);
    float v[NIT][8];
    read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, c, v);
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      epi_act_bwd8_gelu<GATED>(epi, mlane + it * ROWS_PER_IT, n, v[it], win[it % ACT_WINDOW], colsum);
      if (it + ACT_WINDOW < NIT) win[it % ACT_WINDOW] = epi_load_pre8<GATED>(epi, mlane + (it + ACT_WINDOW) * ROWS_PER_IT, n);
    }
    __builtin_amdgcn_wave_barrier();
  };
  // The other kinds, same idea: whole tile in range, tanh GELU, no dropout, residual present.
  const bool whole_tile = m0 + tile_rows <= p.M && n0 + (gated ? tile_cols / 2 : tile_cols) <= p.N;
  auto act_fwd_strip = [&](auto I, auto G) {
    constexpr int i = decltype(I)::value;
    constexpr bool GATED = decltype(G)::value;
    constexpr int LANES_PER_ROW = (GATED ? WTN / 2 : WTN) / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
    const int c = (lane % LANES_PER_ROW) * 8;
    const int64_t n = n0 + wn * (GATED ? WTN / 2 : WTN) + c;
    const int64_t mlane = m0 + wm * WTM + i * 32 + lane / LANES_PER_ROW;
    stage_strip(I);
    float v0[NIT][8], v1[GATED ? NIT : 1][8];
    read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, c, v0);
    if constexpr (GATED)
      read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, WTN / 2 + c, v1);
#pragma unroll
    for (int it = 0; it < NIT; it++) epi_act_fwd8_gelu<GATED>(epi, mlane + it * ROWS_PER_IT, n, v0[it], v1[GATED ? it : 0]);
    __builtin_amdgcn_wave_barrier();
  };
  auto store_strip = [&](auto I, auto out_type) {
    using TO = decltype(out_type);
    constexpr int i = decltype(I)::value;
    constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
    const int c = (lane % LANES_PER_ROW) * 8;
    const int64_t n = n0 + wn * WTN + c;
    const int64_t mlane = m0 + wm * WTM + i * 32 + lane / LANES_PER_ROW;
    stage_strip(I);
    float v[NIT][8];
    read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, c, v);
#pragma unroll
    for (int it = 0; it < NIT; it++) epi_store8_plain<TO>(epi, mlane + it * ROWS_PER_IT, n, v[it]);
    __builtin_amdgcn_wave_barrier();
  };
  auto out_strip = [&](auto I, auto D) {
    constexpr bool DROPOUT = decltype(D)::value;
    constexpr int i = decltype(I)::value;
    constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
    const int c = (lane % LANES_PER_ROW) * 8;
    const int64_t n = n0 + wn * WTN + c;
    const int64_t mlane = m0 + wm * WTM + i * 32 + lane / LANES_PER_ROW;
    EpiLoad win[ACT_WINDOW];
#pragma unroll
    for (int it = 0; it < ACT_WINDOW; it++) win[it] = epi_load_x8<TX>(epi, mlane + it * ROWS_PER_IT, n);
    stage_strip(I);
    float v[NIT][8];
    read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, c, v);
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      epi_out8_residual<TX, DROPOUT>(epi, mlane + it * ROWS_PER_IT, n, v[it], win[it % ACT_WINDOW]);
      if (it + ACT_WINDOW < NIT) win[it % ACT_WINDOW] = epi_load_x8<TX>(epi, mlane + (it + ACT_WINDOW) * ROWS_PER_IT, n);
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto scatter_strip = [&](auto I, auto out_type) {
    using TO = decltype(out_type);
    constexpr int i = decltype(I)::value;
    constexpr int LANES_PER_ROW = WTN / 8, ROWS_PER_IT = 64 / LANES_PER_ROW, NIT = 32 / ROWS_PER_IT;
    const int c = (lane % LANES_PER_ROW) * 8;
    int per_out, entry;  // length of the list, position in it
    int64_t flat;
    if constexpr (SCATTER == 1) {
      per_out = p.sp.blocks_per_out;
      const int64_t ob = lt_run_member((int)(m0 / 256), (wm * WTM + i * 32) / 64, p.sp.out_group, p.sp.out_stride);
      entry = (int)(n0 / 64) + wn * 2 + (c >> 6);
      flat = p.sp.forward_indices[ob * per_out + min(entry, per_out - 1)];
    } else {
      per_out = p.sp.blocks_per_in;
      entry = (int)(m0 / 64) + (wm * WTM + i * 32) / 64;
      const int64_t ib = lt_run_member((int)(n0 / 256), wn * 2 + (c >> 6), p.sp.in_group, p.sp.in_stride);
      flat = ib * per_out + min(entry, per_out - 1);
    }
    TO* dst = reinterpret_cast<TO*>(epi.out) + flat * 4096 + ((i & 1) * 32 + lane / LANES_PER_ROW) * 64 + (c & 63);
    stage_strip(I);
    float v[NIT][8];
    read_staged_rows(std::integral_constant<int, NIT>{}, std::integral_constant<int, ROWS_PER_IT>{}, LANES_PER_ROW, c, v);
    if (entry < per_out) {
#pragma unroll
      for (int it = 0; it < NIT; it++) store8(dst + it * ROWS_PER_IT * 64, v[it]);
    }
    __builtin_amdgcn_wave_barrier();
  };
  if constexpr (SCATTER != 0) {
    static_assert(KIND == EPI_STORE, "scattered blocks: plain store");
    if (epi.out_dtype == LT_F32) for_each_strip([&](auto I) { scatter_strip(I, float{}); });
    else for_each_strip([&](auto I) { scatter_strip(I, bf16{}); });
  } else if constexpr (KIND == EPI_ACT_BWD) {
    const bool straight = whole_tile && epi.act == LT_ACT_GELU_FUSED && epi.hid != nullptr;
    if (straight && epi.gated) for_each_strip([&](auto I) { act_bwd_strip(I, std::true_type{}); });
    else if (straight) for_each_strip([&](auto I) { act_bwd_strip(I, std::false_type{}); });
    else for_each_strip(generic_strip);
  } else if constexpr (KIND == EPI_ACT_FWD) {
    const bool straight = whole_tile && epi.act == LT_ACT_GELU_FUSED;
    if (straight && pair) for_each_strip([&](auto I) { act_fwd_strip(I, std::true_type{}); });
    else if (straight) for_each_strip([&](auto I) { act_fwd_strip(I, std::false_type{}); });
    else for_each_strip(generic_strip);
  } else if constexpr (KIND == EPI_STORE) {
    if (whole_tile && epi.out_dtype == LT_F32) for_each_strip([&](auto I) { store_strip(I, float{}); });
    else if (whole_tile) for_each_strip([&](auto I) { store_strip(I, bf16{}); });
    else for_each_strip(generic_strip);
  } else {
    if (whole_tile && epi.x && epi.drop.p == 0.f) {
      for_each_strip([&](auto I) { out_strip(I, std::false_type{}); });
    } else if (whole_tile && epi.x) {
      for_each_strip([&](auto I) { out_strip(I, std::true_type{}); });
    } else {
      for_each_strip(generic_strip);
    }
  }
  if constexpr (KIND == EPI_ACT_BWD) {
    if (epi.colsum) {
      // lanes l, l + 16, l + 32, l + 48 hold the same columns for different rows of the wavefront's WTM-row sub-tile
      // (the shuffles name their source lane from this function's own lane number: the library routine forms one of its
      // own, which the compiler would compute once and keep in a register through every main loop of a looping workgroup)
      auto from_lane = [&](float v, int mask) {
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __builtin_bit_cast(int, v)));
      };
#pragma unroll
      for (int e = 0; e < 16; e++) {
        colsum[e] += from_lane(colsum[e], 16);
        colsum[e] += from_lane(colsum[e], 32);
      }
      // a sub-tile wholly past the last row has no partial row: the caller sizes the buffer for ceil(M / 128) of them
      if (lane < 16 && n0 + wn * WTN + lane * 8 < p.N && m0 + wm * WTM < p.M) {
        float* dst = epi.colsum + ((m0 + wm * WTM) / WTM) * epi.ld_pre + n0 + wn * WTN + lane * 8;
        float lo[8], hi[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          lo[e] = colsum[e];
          hi[e] = colsum[8 + e];
        }
        store8(dst, lo);
        if (epi.gated) store8(dst + epi.inter, hi);
      }
    }
  }
}

// Block-sparse layouts in which every aligned run of 4 consecutive output blocks shares one list of input blocks are dense
// products over gathered operands:
// GATHER == 1 (both operands mn-major, plain store): the weight gradient.  A = dY [tokens, out], a tile row = a run of 4
//   output blocks; B = X [tokens, in], a tile column = 4 entries of the run's list, gathered as four 64-wide column blocks;
//   the result is scattered to the weight gradient's blocks (SCATTER above).
// GATHER == 3 (both operands mn-major, plain store): the weight gradient of a layout whose runs are on the input side (every
//   aligned run of 4 consecutive input blocks has the same list of output blocks).  A = dY, a tile row = 4 entries of the
//   run's list, gathered as four 64-wide column blocks; B = X, a tile column = the run of 4 input blocks; the 64 x 64 piece
//   (entry a, input block ib) is weight-gradient block ib * blocks_per_in + a.
// GATHER == 2 (both operands k-major): the forward product.  A tile column = a run of 4 output blocks; k-block e of the first
//   k-segment is entry e of the run's list: A = column block ib_e of X, B = the four weight blocks (ib_e, a_e .. a_e + 3),
//   which are adjacent in the native [in, A, block] layout (the run's blocks are consecutive among the active output blocks of
//   ib_e) and so form one [256 rows][64 k] k-major matrix.  The list sits in one register (lane e: ib_e << 16 | flat
//   position) and is read with v_readlane, so the k-loop issues no memory instruction for it.  A second k-segment (the
//   low-rank term) is an ordinary one.
template <bool A_KM, bool B_KM, int KIND, typename TX, bool K_TAIL, int GATHER = 0>
__global__ __launch_bounds__(256) void gemm_bf16_dma_kernel(GemmProblem problem, int tiles_m, int tiles_n) {
  // A workgroup may loop over tiles.  Whatever the compiler finds to be the same in every tile -- values loaded from the problem
  // description, the wavefront's LDS addresses, lane offsets -- it would compute once and keep in registers across the whole
  // loop, epilogues included, and neither register file has room for that.  So the three roots of those values are laundered
  // (an asm statement the compiler cannot see through) at the start of every tile and before every epilogue: the pointer to
  // the problem description (the kernel's first argument, read through the constant address space so that the loads still
  // move freely in between), the wavefront number and the lane number.  Each tile then has the register budget of a kernel
  // that runs a single tile.
  (void)problem;
  typedef const __attribute__((address_space(4))) GemmProblem* KernargProblem;
  KernargProblem pk = (KernargProblem)__builtin_amdgcn_kernarg_segment_ptr();
#define p (*pk)
  static_assert((GATHER != 1 && GATHER != 3) || (!A_KM && !B_KM && KIND == EPI_STORE && !K_TAIL), "gathered columns: weight-gradient layout");
  static_assert(GATHER != 2 || (A_KM && B_KM && !K_TAIL), "gathered k-blocks: forward layout");
  constexpr int BM = 256, BN = 256, WN = 2, WTM = 128, WTN = 128, FM = 4, FN = 4;
  constexpr int HALF = 4;  // copy instructions per wavefront for a mn-major k-step or half a k-major block
  constexpr int KM_ELEMS = 256 * 64, MN_ELEMS = DK * 256;
  // k-major operands use the two d buffers, mn-major ones the four s tiles; the unused set is never referenced and takes
  // no LDS
  __shared__ __attribute__((aligned(1024))) bf16 a_d0[KM_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 a_d1[KM_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 a_s0[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 a_s1[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 a_s2[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 a_s3[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_d0[KM_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_d1[KM_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_s0[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_s1[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_s2[MN_ELEMS];
  __shared__ __attribute__((aligned(1024))) bf16 b_s3[MN_ELEMS];

  auto fresh_lane = []() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
  };
  int lane = fresh_lane();
  int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  int wm = wave / WN, wn = wave % WN;
  auto refresh = [&]() {
    asm volatile("" : "+s"(pk), "+s"(wave));
    lane = fresh_lane();
    wm = wave / WN;
    wn = wave % WN;
  };
#ifdef LT_TILE_TIMING
  unsigned long long* tile_stamps = p.tile_stamps ? p.tile_stamps + (size_t)blockIdx.x * 8 : nullptr;  // 8 words per tile
#endif
  LT_TILE_STAMP(0);
  LT_TILE_STAMP_REALTIME(4);

  // k-steps of the problem (kt_all), of this workgroup's slice of them (kt_total, from kt_begin; split-k: one k-segment only,
  // slices of an even number of k-steps so that k-major blocks stay whole; below, k-step numbers are local to the slice) and
  // of the first k-segment (kt_seg0).  Recomputed from the laundered problem description at every tile, like everything else.
  int kt_all = 0, kt_begin = 0, kt_total = 0, kt_seg0 = 0;
  bool gated = false;
  auto k_steps = [&]() {
    gated = (KIND == EPI_ACT_FWD) && p.epi.gated;
    kt_all = (int)((p.K[0] + DK - 1) / DK) + (p.nseg > 1 ? (int)((p.K[1] + DK - 1) / DK) : 0);
    kt_begin = 0;
    kt_total = kt_all;
    if (p.ksplit > 1) {
      const int per = (((kt_all + p.ksplit - 1) / p.ksplit) + 1) & ~1;
      kt_begin = min(kt_all, (int)blockIdx.y * per);
      kt_total = min(per, kt_all - kt_begin);
    }
    kt_seg0 = p.nseg > 1 ? (int)((p.K[0] + DK - 1) / DK) : kt_total;
  };
  k_steps();

  // A workgroup takes tiles blockIdx.x, blockIdx.x + gridDim.x, ... of the launch order (the host launches one workgroup per
  // tile, or one per CU that loops: then the first copies of the next tile go out before the epilogue of the current one).
  // Tile v of the launch order goes to XCD v % 8 either way; each XCD walks a contiguous range of tiles, GROUP_M tile-rows at a
  // time.
  const int num_pid = tiles_m * tiles_n;
  int vb = blockIdx.x;
  int tm = 0, tn = 0;
  int64_t m0 = 0, n0 = 0;
  auto place = [&](int v) {
    int pid = v;
    if ((num_pid & 7) == 0) pid = (pid & 7) * (num_pid >> 3) + (pid >> 3);
    const int group = GROUP_M * tiles_n;
    const int first_m = (pid / group) * GROUP_M;
    const int gsz = min(tiles_m - first_m, GROUP_M);
    tm = first_m + (pid % group) % gsz;
    tn = (pid % group) / gsz;
    m0 = (int64_t)tm * BM;
    n0 = (int64_t)tn * (gated ? BN / 2 : BN);
  };
  place(vb);

  f32x16 acc[FM][FN];  // initialised in the prologue, after the first copies have gone out

  // ---- buffer of k-step position I (k-step index mod 4) and copy targets, selected at compile time
  auto a_buf = [&](auto I) -> bf16* {
    constexpr int i = decltype(I)::value & 3;
    if constexpr (A_KM) return (i & 2) ? a_d1 : a_d0;
    else return i == 0 ? a_s0 : i == 1 ? a_s1 : i == 2 ? a_s2 : a_s3;
  };
  auto b_buf = [&](auto I) -> bf16* {
    constexpr int i = decltype(I)::value & 3;
    if constexpr (B_KM) return (i & 2) ? b_d1 : b_d0;
    else return i == 0 ? b_s0 : i == 1 ? b_s1 : i == 2 ? b_s2 : b_s3;
  };

  // Workgroups start their walk over k at different offsets and wrap around: with a power-of-two leading dimension every
  // row of a k-major tile otherwise maps to the same memory channels at the same time, chip-wide.  The offset is the same
  // for the workgroups of one XCD that run next to each other (they share operand panels through that XCD's L2) and
  // differs between XCDs.  Measured on the up- and down-projection shapes: +16 % and +25 % for two k-major operands,
  // nothing to gain for mn-major ones.
  int rot = 0;
  auto set_rot = [&](int v) {
    if (!K_TAIL && GATHER == 0 && p.nseg == 1 && (kt_all & 1) == 0 && p.krot) {
      const unsigned bx = (unsigned)v;
      // (inside an XCD the eight tile rows start 2 k-steps apart at most: tiles that share a B panel then read it within 14
      // k-steps of each other, inside what the XCD's L2 still holds; 8 apart, as a long reduction would otherwise give,
      // measured 1.4 % slower on the down-projection shape and fetched the panels more than once)
      const unsigned r = (bx & 7) * (kt_all >> 3) +
                         (p.krot == 1 ? ((bx >> 3) & 3) * (kt_all >> 5) : ((bx >> 3) & 7) * min(kt_all >> 6, 2));
      rot = __builtin_amdgcn_readfirstlane((int)((r % (unsigned)kt_all) & ~1u));
    }
  };
  set_rot(vb);
  auto rotated = [&](int ks) {
    const int r = ks + rot;
    return r >= kt_all ? r - kt_all : r;
  };
  DmaOperand<A_KM> ca;
  DmaOperand<B_KM> cb;
  int list_entry = 0;  // GATHER == 2: lane e holds entry e of this tile's list
  auto load_list = [&]() {
    if constexpr (GATHER == 2) {
      const int e = min(lane, p.sp.blocks_per_out - 1);
      // (clamped so that the four blocks read from `flat` on lie inside the weight even if the caller's promise of shared
      // lists is false: wrong results then, but no access outside the weight)
      const int flat = min(p.sp.forward_indices[(n0 / 64) * p.sp.blocks_per_out + e],
                           (int)(p.sp.ld_act / 64) * p.sp.blocks_per_in - 4);
      list_entry = (flat / p.sp.blocks_per_in) << 16 | flat;
    }
  };
  load_list();
  auto setup_a = [&](int seg) {
    if (GATHER == 2 && seg == 0) {
      const GemmOperand x = {p.sp.act, p.sp.ld_act, 1};
      ca.setup(x, 0, m0, p.M, 0, wave, lane);  // unit u = column block u of X
    } else if constexpr (GATHER == 3) {
      // the output blocks of list entries tm * 4 .. tm * 4 + 3 of the first input block of tile column tn (past the end: the
      // last entry again)
      const int64_t ib0 = lt_run_member(tn, 0, p.sp.in_group, p.sp.in_stride);
      int blocks[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int entry = min(tm * 4 + j, p.sp.blocks_per_in - 1);
        blocks[j] = (int)p.sp.backward_indices[ib0 * p.sp.blocks_per_in + entry];
      }
      const GemmOperand a = {p.A[0].ptr, p.A[0].ld, p.A[0].kmajor};
      ca.setup_gather(a, blocks, wave, lane);
    } else if (GATHER == 1 && p.sp.out_stride > 1) {
      // the four members of the run that tile row tm stands for lie out_stride blocks apart
      int blocks[4];
#pragma unroll
      for (int j = 0; j < 4; j++) blocks[j] = lt_run_member(tm, j, p.sp.out_group, p.sp.out_stride);
      const GemmOperand a = {p.A[0].ptr, p.A[0].ld, p.A[0].kmajor};
      if constexpr (!A_KM) ca.setup_gather(a, blocks, wave, lane);
    } else {
      const GemmOperand a = {p.A[seg].ptr, p.A[seg].ld, p.A[seg].kmajor};
      ca.setup(a, seg, m0, p.M, 0, wave, lane);
    }
  };
  auto setup_b = [&](int seg) {
    if (GATHER == 2 && seg == 0) {
      const GemmOperand w = {p.sp.weight, 64, 1};
      cb.setup(w, 0, 0, 256, 0, wave, lane);
      cb.unit_bytes = 64 * 64 * 2;  // unit u = weight block at flat position u (and the three after it)
      return;
    }
    if constexpr (GATHER == 1) {
      // the input blocks of list entries tn * 4 .. tn * 4 + 3 of the first output block of tile row tm (past the end: the last
      // entry again)
      const int64_t ob0 = lt_run_member(tm, 0, p.sp.out_group, p.sp.out_stride);
      int blocks[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int entry = min(tn * 4 + j, p.sp.blocks_per_out - 1);
        blocks[j] = p.sp.forward_indices[ob0 * p.sp.blocks_per_out + entry] / p.sp.blocks_per_in;
      }
      const GemmOperand b = {p.B[0].ptr, p.B[0].ld, p.B[0].kmajor};
      cb.setup_gather(b, blocks, wave, lane);
    } else if (GATHER == 3 && p.sp.in_stride > 1) {
      int blocks[4];
#pragma unroll
      for (int j = 0; j < 4; j++) blocks[j] = lt_run_member(tn, j, p.sp.in_group, p.sp.in_stride);
      const GemmOperand b = {p.B[0].ptr, p.B[0].ld, p.B[0].kmajor};
      if constexpr (!B_KM) cb.setup_gather(b, blocks, wave, lane);
    } else {
      const GemmOperand b = {p.B[seg].ptr, p.B[seg].ld, p.B[seg].kmajor};
      cb.setup(b, seg, n0, p.N, (B_KM && gated) ? p.N : 0, wave, lane);
    }
  };
  setup_a(0);
  setup_b(0);
  // copies of the unit that holds k-step t (a block for k-major operands) into the buffer of position I
  auto copy_a = [&](auto steady, auto I, int t, auto J0, auto J1) {
    int seg = ca.seg;
    if constexpr (!decltype(steady)::value) {  // the steady loop never crosses a k-segment boundary
      seg = __builtin_amdgcn_readfirstlane((int)(t >= kt_seg0));  // wavefront-uniform: keep it in a scalar register
      if (seg != ca.seg) setup_a(seg);
    }
    const int ks = rotated(seg ? t - kt_seg0 : t + kt_begin);
    int unit = A_KM ? ks >> 1 : ks;
    if (GATHER == 2 && seg == 0) unit = __builtin_amdgcn_readlane(list_entry, ks >> 1) >> 16;
    ca.template issue<K_TAIL, decltype(J0)::value, decltype(J1)::value>(unit, a_buf(I), wave, p.K[seg]);
  };
  auto copy_b = [&](auto steady, auto I, int t, auto J0, auto J1) {
    int seg = cb.seg;
    if constexpr (!decltype(steady)::value) {
      seg = __builtin_amdgcn_readfirstlane((int)(t >= kt_seg0));  // wavefront-uniform: keep it in a scalar register
      if (seg != cb.seg) setup_b(seg);
    }
    const int ks = rotated(seg ? t - kt_seg0 : t + kt_begin);
    int unit = B_KM ? ks >> 1 : ks;
    if (GATHER == 2 && seg == 0) unit = __builtin_amdgcn_readlane(list_entry, ks >> 1) & 0xffff;
    cb.template issue<K_TAIL, decltype(J0)::value, decltype(J1)::value>(unit, b_buf(I), wave, p.K[seg]);
  };

  // ---- MFMA operand fragments: 8 k values of row / column lane % 32 of a 32-wide block
  auto frag_km = [&](const bf16* buf, int base, int kk, int half) -> bf16x8 {
    const int row = base + (lane & 31);
    const int c = half * 4 + kk * 2 + (lane >> 5);
    return *reinterpret_cast<const bf16x8*>(&buf[(row * 8 + (c ^ swz_km(row))) * 8]);
  };
  auto frag_mn = [&](const bf16* tile, int base, int kk) -> bf16x8 {
    union { bf16x8 v; s16x4 h[2]; } u;
    const int i16 = lane & 15;
    const int col = base + ((lane >> 4) & 1) * 16 + 4 * (i16 & 3);
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const int kr = kk * 16 + 8 * (lane >> 5) + 4 * s + (i16 >> 2);
      const bf16* src = &tile[kr * 256 + ((((col >> 3) ^ swz_mn(kr)) << 3) | (col & 7))];
      u.h[s] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(src));
    }
    return u.v;
  };
  auto load_frags = [&](auto I, int kk, bf16x8 (&a)[FM], bf16x8 (&b)[FN]) {
    constexpr int half = decltype(I)::value & 1;
    const bf16* ta = a_buf(I);
    const bf16* tb = b_buf(I);
    // pair (A block i, B block i) after pair i - 1: the order in which the matrix instructions below first need them
    static_assert(FM == FN, "reads alternate between the operands");
#pragma unroll
    for (int i = 0; i < FM; i++) {
      if constexpr (A_KM) a[i] = frag_km(ta, wm * WTM + i * 32, kk, half);
      else a[i] = frag_mn(ta, wm * WTM + i * 32, kk);
      if constexpr (B_KM) b[i] = frag_km(tb, wn * WTN + i * 32, kk, half);
      else b[i] = frag_mn(tb, wn * WTN + i * 32, kk);
    }
  };
  // the 16 matrix instructions of a half-step, in the order in which their fragments arrive (pair 0 first, pair 3 last):
  // the wait before the first one then covers two LDS reads, not all eight
  auto mfma_half = [&](bf16x8 (&a)[FM], bf16x8 (&b)[FN]) {
    constexpr int ORDER[16][2] = {{0, 0}, {1, 0}, {0, 1}, {1, 1}, {2, 0}, {2, 1}, {0, 2}, {1, 2},
                                  {2, 2}, {3, 0}, {3, 1}, {3, 2}, {0, 3}, {1, 3}, {2, 3}, {3, 3}};
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const int x = ORDER[q][0], y = ORDER[q][1];
      acc[x][y] = LT_MFMA_32X32X16(a[x], b[y], acc[x][y]);
    }
  };
  constexpr int FRAG_READS = FM * (A_KM ? 1 : 2) + FN * (B_KM ? 1 : 2);
  // LDS reads of a half-step spread over this many of its 16 matrix instructions: evenly over all of them, except for the
  // mixed layout, which measured 2 % faster with the reads done by the twelfth
  constexpr int READ_SPAN = (A_KM && !B_KM) ? FM * FN * 3 / 4 : FM * FN;
  constexpr int N_MN = (A_KM ? 0 : HALF) + (B_KM ? 0 : HALF);  // copy instructions per k-step for the mn-major operands
  constexpr int N_KM = (A_KM ? 2 * HALF : 0) + (B_KM ? 2 * HALF : 0);  // copy instructions per block for the k-major operands

  bf16x8 af[2][FM], bfr[2][FN];  // [0]: first 16 k of the current k-step, [1]: second 16 k

  // A k-step is issued as two halves so that the loop body can start at the barrier:
  //   first_half(t)   LDS reads of the second 16 k of k-step t, the copies due at t, matrix instructions on the first 16 k
  //   second_half(t)  wait for the copies k-step t + 1 needs + barrier, LDS reads of the first 16 k of k-step t + 1,
  //                   matrix instructions on the second 16 k
  // I = t mod 4 at compile time.  steady == true: straight-line code, valid while every copy it issues exists and stays
  // inside the current k-segment.
  // Copies are spread over the half-steps so that the address unit, which the four wavefronts share, is not handed whole
  // blocks at once: the halves of a k-major block go out in the slots of SA / SB, mn-major B (next to mn-major A) in the
  // second half of every k-step (B_SPLIT); the rest in the first half.
  constexpr BlockSlots SA = B_KM ? SLOTS_NT_A : SLOTS_NN_A, SB = SLOTS_NT_B;
  constexpr bool B_SPLIT = !B_KM && !A_KM && SPLIT_MN_B;
  using J0 = std::integral_constant<int, 0>;
  using J4 = std::integral_constant<int, HALF>;      // named for the four-wavefront case: half a k-major block,
  using J8 = std::integral_constant<int, 2 * HALF>;  // a whole one
  // the halves of the k-major blocks assigned to `slot`, for the block that starts at k-step t, into position I
  auto copy_block_halves = [&](auto steady, auto slot, auto I, int t) {
    constexpr int SLOT = decltype(slot)::value;
    if constexpr (A_KM && SA.half[0] == SLOT) copy_a(steady, I, t, J0{}, J4{});
    if constexpr (A_KM && SA.half[1] == SLOT) copy_a(steady, I, t, J4{}, J8{});
    if constexpr (B_KM && SB.half[0] == SLOT) copy_b(steady, I, t, J0{}, J4{});
    if constexpr (B_KM && SB.half[1] == SLOT) copy_b(steady, I, t, J4{}, J8{});
  };
  auto slot_copies = [&](int slot) constexpr {
    return (A_KM ? HALF * ((SA.half[0] == slot) + (SA.half[1] == slot)) : 0) +
           (B_KM ? HALF * ((SB.half[0] == slot) + (SB.half[1] == slot)) : 0);
  };
  // LDS reads in flight at the barrier of k-step t are the second 16 k of that k-step (position i).  Copies issued before
  // the next barrier that overwrite that buffer: mn-major copies of the next first half (the ring tile of k-step t), and
  // after an odd k-step the slot-0 and slot-1 halves of a k-major block.  Without those the reads may stay in flight
  // across the barrier.
  constexpr bool MN_FIRST_HALF = !A_KM || (!B_KM && !B_SPLIT);
  constexpr bool KM_EARLY_SLOTS = (A_KM && (SA.half[0] < 2 || SA.half[1] < 2)) || (B_KM && (SB.half[0] < 2 || SB.half[1] < 2));
  auto first_half = [&](auto steady, auto I, int t) {
    constexpr bool STEADY = decltype(steady)::value;
    constexpr int i = decltype(I)::value & 3;
    load_frags(I, 1, af[1], bfr[1]);
    if (STEADY || t + 3 < kt_total) {  // mn-major: k-step t + 3 into the tile freed by the last barrier
      if constexpr (!A_KM) copy_a(steady, std::integral_constant<int, (i + 3) & 3>{}, t + 3, J0{}, J4{});
      if constexpr (!B_KM && !B_SPLIT) copy_b(steady, std::integral_constant<int, (i + 3) & 3>{}, t + 3, J0{}, J4{});
    }
    if constexpr ((i & 1) == 0 && N_KM > 0) {  // k-major: the block of k-steps t + 2, t + 3 into the other buffer
      if (STEADY || t + 2 < kt_total)
        copy_block_halves(steady, std::integral_constant<int, 1>{}, std::integral_constant<int, (i + 2) & 3>{}, t + 2);
    }
    mfma_half(af[0], bfr[0]);
    constexpr int COPIES = (A_KM ? 0 : HALF) + ((B_KM || B_SPLIT) ? 0 : HALF) + ((i & 1) == 0 ? slot_copies(1) : 0);
    SchedInterleave3<FRAG_READS, COPIES, FM * FN, READ_SPAN>::run();
  };
  auto second_half = [&](auto steady, auto I, int t) {
    constexpr bool STEADY = decltype(steady)::value;
    constexpr int i = decltype(I)::value & 3;
    constexpr int IN_FLIGHT = copies_in_flight(A_KM, B_KM, SA, SB, B_SPLIT, i & 1);
    constexpr bool READS_MUST_LAND = MN_FIRST_HALF || ((i & 1) == 1 && KM_EARLY_SLOTS);
    if constexpr (STEADY) wait_copies_and_barrier<IN_FLIGHT, READS_MUST_LAND>();
    else wait_copies_and_barrier<0>();
    if (STEADY || t + 1 < kt_total) load_frags(std::integral_constant<int, (i + 1) & 3>{}, 0, af[0], bfr[0]);
    // the barrier above freed the buffers of k-step t - 1 and, on odd t, the k-major buffer of k-steps t - 1, t
    if constexpr (B_SPLIT) {
      if (STEADY || t + 3 < kt_total) copy_b(steady, std::integral_constant<int, (i + 3) & 3>{}, t + 3, J0{}, J4{});
    }
    if constexpr (N_KM > 0 && (i & 1) == 1) {
      if (STEADY || t + 3 < kt_total)
        copy_block_halves(steady, std::integral_constant<int, 0>{}, std::integral_constant<int, (i + 3) & 3>{}, t + 3);
    }
    if constexpr (N_KM > 0 && (i & 1) == 0) {
      if (STEADY || t + 2 < kt_total)
        copy_block_halves(steady, std::integral_constant<int, 2>{}, std::integral_constant<int, (i + 2) & 3>{}, t + 2);
    }
    mfma_half(af[1], bfr[1]);
    constexpr int COPIES = (B_SPLIT ? HALF : 0) + (N_KM > 0 ? slot_copies((i & 1) ? 0 : 2) : 0);
    SchedInterleave3<FRAG_READS, COPIES, FM * FN, READ_SPAN>::run();
  };
  using Steady = std::integral_constant<bool, true>;
  using Ragged = std::integral_constant<bool, false>;
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;

  // ---- prologue of a tile, in two parts.  Early: k-steps 0 and 1 (k-major: block 0), into buffers the epilogue's staging
  //      leaves alone, so that a looping workgroup issues them for its next tile before the epilogue of the current one.
  //      Late: k-step 2 and the slot-0 halves of block 1, into the staging buffers, once the epilogue is done.  Same issue
  //      order as the steady loop's.
  auto prologue_early = [&]() {
    if constexpr (A_KM) copy_a(Ragged{}, P0{}, 0, J0{}, J8{});
    if constexpr (B_KM) copy_b(Ragged{}, P0{}, 0, J0{}, J8{});
    if constexpr (!A_KM) copy_a(Ragged{}, P0{}, 0, J0{}, J4{});
    if constexpr (!B_KM) copy_b(Ragged{}, P0{}, 0, J0{}, J4{});
    if (kt_total > 1) {
      if constexpr (!A_KM) copy_a(Ragged{}, P1{}, 1, J0{}, J4{});
      if constexpr (!B_KM) copy_b(Ragged{}, P1{}, 1, J0{}, J4{});
    }
  };
  auto prologue_late = [&]() {
    if (kt_total > 2) {
      if constexpr (!A_KM) copy_a(Ragged{}, P2{}, 2, J0{}, J4{});
      if constexpr (!B_KM) copy_b(Ragged{}, P2{}, 2, J0{}, J4{});
      if constexpr (N_KM > 0) copy_block_halves(Ragged{}, std::integral_constant<int, 0>{}, P2{}, 2);
    }
  };
  constexpr int LATE_COPIES = (A_KM ? 0 : HALF) + (B_KM ? 0 : HALF) + slot_copies(0);
  LT_TILE_STAMP(6);
  prologue_early();
  for (;;) {
    refresh();
    k_steps();
    setup_a(0);
    setup_b(0);
    prologue_late();
    // The accumulators start at the bias of their column (a lane holds one column per 32-wide block), so no epilogue has to
    // add it.  The bias loads wait behind the first copies rather than in front of them.  Gated forward: blocks 0, 1 of a
    // wavefront are gate columns, 2, 3 the matching linear columns.
    {
      float bias0[FN];
#pragma unroll
      for (int j = 0; j < FN; j++) {
        bias0[j] = 0.f;
        if (p.epi.bias) {
          // columns past N (a tile that sticks out) take the last column's bias and are never written
          const int64_t col = gated ? (j >= FN / 2 ? p.epi.inter : 0) +
                                          min(n0 + wn * (WTN / 2) + (j % (FN / 2)) * 32 + (lane & 31), p.N - 1)
                                    : min(n0 + wn * WTN + j * 32 + (lane & 31), p.N - 1);
          bias0[j] = p.epi.bias[col];
        }
      }
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = bias0[j];
    }
    // everything older than the late copies has landed (the early copies; a looping workgroup's previous stores)
    if (kt_total > 2) wait_copies_and_barrier<LATE_COPIES>();
    else wait_copies_and_barrier<0>();
    LT_TILE_STAMP(1);
    load_frags(P0{}, 0, af[0], bfr[0]);
    first_half(Ragged{}, P0{}, 0);

    // loop body i of a group of four: second half of k-step kt + i, first half of k-step kt + i + 1
    int kt = 0;
    for (;;) {
      // copies issued by the steady loop reach k-step kt + 7: they must exist and lie in the k-segment both operands' copy
      // offsets are set up for
      const int bound = (ca.seg == 0 && p.nseg > 1) ? kt_seg0 : kt_total;
      if (ca.seg == cb.seg) {
        for (; kt + 7 < bound; kt += 4) {
#ifdef LT_TILE_TIMING
          if (kt == 16) LT_TILE_STAMP(7);
#endif
          second_half(Steady{}, P0{}, kt);
          first_half(Steady{}, P1{}, kt + 1);
          second_half(Steady{}, P1{}, kt + 1);
          first_half(Steady{}, P2{}, kt + 2);
          second_half(Steady{}, P2{}, kt + 2);
          first_half(Steady{}, P3{}, kt + 3);
          second_half(Steady{}, P3{}, kt + 3);
          first_half(Steady{}, P0{}, kt + 4);
        }
      }
      if (kt >= kt_total) break;
      second_half(Ragged{}, P0{}, kt);
      if (kt + 1 < kt_total) { first_half(Ragged{}, P1{}, kt + 1); second_half(Ragged{}, P1{}, kt + 1); }
      if (kt + 2 < kt_total) { first_half(Ragged{}, P2{}, kt + 2); second_half(Ragged{}, P2{}, kt + 2); }
      if (kt + 3 < kt_total) { first_half(Ragged{}, P3{}, kt + 3); second_half(Ragged{}, P3{}, kt + 3); }
      if (kt + 4 < kt_total) first_half(Ragged{}, P0{}, kt + 4);
      kt += 4;
      if (kt >= kt_total) break;
    }
    __syncthreads();  // every wavefront is done with the buffers: the early ones may take the next tile, the late ones stage
    LT_TILE_STAMP(2);

    refresh();
    k_steps();
    const int64_t epi_m0 = m0, epi_n0 = n0;
    const int next = vb + (int)gridDim.x;
    const bool more = next < num_pid;
    if (more) {
      place(next);
      set_rot(next);
      load_list();
      setup_a(0);
      setup_b(0);
      prologue_early();
    }
    // 16 KiB of staging space per wavefront, in the buffers the early copies do not touch
    bf16* const stage_buf = wave == 0   ? (A_KM ? a_d1 : a_s2)
                            : wave == 1 ? (A_KM ? a_d1 + KM_ELEMS / 2 : a_s3)
                            : wave == 2 ? (B_KM ? b_d1 : b_s2)
                                        : (B_KM ? b_d1 + KM_ELEMS / 2 : b_s3);
    dma_tile_epilogue<FM, KIND, TX, BM, BN, GATHER == 1 ? 1 : GATHER == 3 ? 2 : 0>(acc, *(const GemmProblem*)pk, reinterpret_cast<float*>(stage_buf), epi_m0,
                                                          epi_n0, wm, wn, gated);
    LT_TILE_STAMP(3);
    LT_TILE_STAMP_REALTIME(5);
    if (!more) break;
    vb = next;
    __syncthreads();  // the staging buffers are free: the late copies may go out
#ifdef LT_TILE_TIMING
    if (tile_stamps) tile_stamps = p.tile_stamps + (size_t)vb * 8;
#endif
    LT_TILE_STAMP(0);
    LT_TILE_STAMP_REALTIME(4);
    LT_TILE_STAMP(6);
  }
  static_assert(32 * WTN * 4 <= MN_ELEMS * 2, "a 32-row strip must fit the smallest buffer");
#undef p
}

// Workgroups of a copy-based launch with `tiles` tiles: one per tile, or, when there are more tiles than compute units and
// the problem allows it, one per compute unit that loops over tiles v, v + grid, ... (the kernel's LDS use keeps it alone on
// its CU either way).  The looping workgroup issues the first copies of its next tile before the epilogue of the current
// one, which takes the start of a tile (workgroup launch, first operand blocks arriving) off the critical path.
inline unsigned dma_grid(const GemmProblem& p, int tiles) {
  static int cus[64] = {};  // per device; filled on first use (every thread writes the same value)
  int dev = 0;
  if (p.tile_loop == 1 || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return (unsigned)tiles;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = -1;
    cus[dev] = n;
  }
  const int n = cus[dev] & ~7;  // a multiple of the 8 XCDs, so that a workgroup's tiles stay on its XCD's range
  return (n > 0 && tiles > n) ? (unsigned)n : (unsigned)tiles;
}

template <bool A_KM, bool B_KM, int KIND>
int launch_dma(const GemmProblem& problem, int io_dtype, hipStream_t stream) {
  GemmProblem p = problem;
#ifdef LT_TILE_TIMING
  if (const char* e = getenv("LT_TILE_TIMING_BUFFER"))
    p.tile_stamps = (unsigned long long*)(strtoull(e, nullptr, 0) + (size_t)(lt_tile_timing_launch_counter()++ % 6) * 4096 * 64);
#endif
  // k-walk stagger: on unless the caller chose (15: off)
  if (p.krot == 0) p.krot = (A_KM && B_KM) ? 2 : 0;
  else if (p.krot == 15) p.krot = 0;
  const bool gated = KIND == EPI_ACT_FWD && p.epi.gated;
  const int tiles_m = (int)((p.M + 255) / 256);
  const int tiles_n = (int)((p.N + (gated ? 127 : 255)) / (gated ? 128 : 256));
  bool k_tail = false;
  for (int s = 0; s < p.nseg; s++) k_tail = k_tail || (p.K[s] % DK != 0);
  dim3 grid(dma_grid(p, tiles_m * tiles_n), (unsigned)(p.ksplit > 1 ? p.ksplit : 1)), block(256);
  const bool bf16_io = KIND == EPI_OUT && io_dtype == LT_BF16;
  if constexpr (!A_KM && !B_KM) {
    if (k_tail) {
      hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, float, true>), grid, block, 0, stream, p, tiles_m, tiles_n);
      LT_LAUNCH_CHECK();
      return LT_OK;
    }
  }
  // the type of x / y only enters the EPI_OUT epilogue: the other kinds have one instantiation
  if constexpr (KIND == EPI_OUT) {
    if (bf16_io) {
      hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, bf16, false>), grid, block, 0, stream, p, tiles_m, tiles_n);
      LT_LAUNCH_CHECK();
      return LT_OK;
    }
  }
  hipLaunchKernelGGL((gemm_bf16_dma_kernel<A_KM, B_KM, KIND, float, false>), grid, block, 0, stream, p, tiles_m, tiles_n);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

template <int BM, int BN, int WM, int WN, bool A_KM, bool B_KM, int KIND>
int launch_cfg(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  const bool gated = KIND == EPI_ACT_FWD && p.epi.gated;
  const int tiles_m = (int)((p.M + BM - 1) / BM);
  const int tiles_n = (int)(p.N / (gated ? BN / 2 : BN));
  dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)(p.ksplit > 1 ? p.ksplit : 1)), block(WM * WN * 64);
  if constexpr (KIND == EPI_OUT) {
    if (io_dtype == LT_BF16) {
      hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, WM, WN, A_KM, B_KM, KIND, bf16>), grid, block, 0, stream, p, tiles_m,
                         tiles_n);
      LT_LAUNCH_CHECK();
      return LT_OK;
    }
  }
  hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, WM, WN, A_KM, B_KM, KIND, float>), grid, block, 0, stream, p, tiles_m, tiles_n);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

template <int KIND> int launch_sparse(const GemmProblem& problem, int io_dtype, hipStream_t stream) {
  GemmProblem p = problem;
#ifdef LT_TILE_TIMING
  // block-sparse FWD / DX launch number i of the process writes region i % 4 (8192 workgroups each) of its own buffer
  if (const char* e = getenv("LT_TILE_TIMING_BUFFER_SPARSE")) {
    if (p.sp.mode == SPARSE_FWD || p.sp.mode == SPARSE_DX)
      p.tile_stamps = (unsigned long long*)(strtoull(e, nullptr, 0) + (size_t)(lt_tile_timing_launch_counter()++ % 4) * 8192 * 64);
  }
#endif
  const SparseWalk& sp = p.sp;
  const bool bf16_io = KIND == EPI_OUT && io_dtype == LT_BF16;
  dim3 block(256);
  if (sp.mode == SPARSE_FWD || sp.mode == SPARSE_DX) {
    const int tiles_m = (int)((p.M + 255) / 256), groups = (int)(p.N / 64);
    dim3 grid((unsigned)(tiles_m * groups));
    using TXB = std::conditional_t<KIND == EPI_OUT, bf16, float>;  // only EPI_OUT touches x / y
    if constexpr (KIND == EPI_STORE || KIND == EPI_ACT_FWD) {
      if (lt_sparse_forward_grouped(p, KIND)) {
        // runs of 4 output blocks share one list: a dense product over gathered k-blocks on 256 x 256 tiles
        GemmProblem q = p;
        q.K[0] = (int64_t)sp.blocks_per_out * 64;
        q.ksplit = 0; q.krot = 0;
        const int tiles_n = (int)(p.N / 256);
        hipLaunchKernelGGL((gemm_bf16_dma_kernel<true, true, KIND, float, false, 2>), dim3(dma_grid(q, tiles_m * tiles_n)), block, 0,
                           stream, q, tiles_m, tiles_n);
        LT_LAUNCH_CHECK();
        return LT_OK;
      }
    }
    if (sp.mode == SPARSE_FWD && KIND == EPI_ACT_FWD && p.epi.gated) {
      // p.N counts the gate columns: one workgroup per (token tile, gate block), paired with linear block tn + groups
      if constexpr (KIND == EPI_ACT_FWD)
        hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, true, true, EPI_ACT_FWD, float, SPARSE_FWD, 2>), grid, block, 0, stream, p, tiles_m, groups);
    } else if (sp.mode == SPARSE_FWD) {
      if (bf16_io) hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, true, true, KIND, TXB, SPARSE_FWD>), grid, block, 0, stream, p, tiles_m, groups);
      else hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, true, true, KIND, float, SPARSE_FWD>), grid, block, 0, stream, p, tiles_m, groups);
    } else {
      if (bf16_io) hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, true, false, KIND, TXB, SPARSE_DX>), grid, block, 0, stream, p, tiles_m, groups);
      else hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, true, false, KIND, float, SPARSE_DX>), grid, block, 0, stream, p, tiles_m, groups);
    }
  } else {
    if constexpr (KIND == EPI_STORE) {
      const int64_t out_features = sp.ld_act;
      if (lt_sparse_dw_out_grouped(p)) {
        // grouped: a dense both-operands-mn-major product dY^T X per run of 4 output blocks, over their shared list
        GemmProblem q = p;
        q.M = out_features;
        const int tiles_m = (int)(out_features / 256), tiles_n = (sp.blocks_per_out + 3) / 4;
        q.N = (int64_t)tiles_n * 256;
        q.nseg = 1; q.K[0] = sp.tokens; q.K[1] = 0;
        q.A[0].ptr = sp.act; q.A[0].ld = sp.ld_act; q.A[0].kmajor = 0;
        q.B[0].ptr = sp.act2; q.B[0].ld = sp.ld_act2; q.B[0].kmajor = 0;
        q.ksplit = 0; q.krot = 0;
        hipLaunchKernelGGL((gemm_bf16_dma_kernel<false, false, EPI_STORE, float, false, 1>), dim3(dma_grid(q, tiles_m * tiles_n)),
                           block, 0, stream, q, tiles_m, tiles_n);
        LT_LAUNCH_CHECK();
        return LT_OK;
      }
      if (lt_sparse_dw_in_grouped_slices(p) > 0) {
        // grouped on the input side: dY^T X per run of 4 input blocks, over their shared list of output blocks.  The
        // reduction is split only when the caller asked (p.ksplit slices, epi.out pointing at fp32 partial sums)
        const int slices = p.ksplit > 1 ? p.ksplit : 1;
        GemmProblem q = p;
        const int tiles_m = (sp.blocks_per_in + 3) / 4, tiles_n = (int)(p.N / 256);
        q.M = (int64_t)tiles_m * 256;
        q.nseg = 1; q.K[0] = sp.tokens; q.K[1] = 0;
        q.A[0].ptr = sp.act; q.A[0].ld = sp.ld_act; q.A[0].kmajor = 0;
        q.B[0].ptr = sp.act2; q.B[0].ld = sp.ld_act2; q.B[0].kmajor = 0;
        q.ksplit = slices > 1 ? slices : 0; q.krot = 0;
        hipLaunchKernelGGL((gemm_bf16_dma_kernel<false, false, EPI_STORE, float, false, 3>),
                           dim3(dma_grid(q, tiles_m * tiles_n), (unsigned)slices), block, 0, stream, q, tiles_m, tiles_n);
        LT_LAUNCH_CHECK();
        return LT_OK;
      }
      const int groups = (int)((p.N / 64) * ((sp.blocks_per_in + 3) / 4));  // p.N = in_features
      hipLaunchKernelGGL((gemm_bf16_kernel<256, 64, 4, 1, false, false, EPI_STORE, float, SPARSE_DW>), dim3((unsigned)groups),
                         block, 0, stream, p, 1, groups);
    } else {
      LT_FAIL(LT_ERR_UNSUPPORTED, "block-sparse weight gradient takes the plain store epilogue only");
    }
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

// whether a problem the tiled kernels take goes to the copy-based one
bool dma_selected(const GemmProblem& p, int kind, int io_dtype) {
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  bool k_tail = false, k_blocks = true;
  for (int s = 0; s < p.nseg; s++) {
    k_tail = k_tail || (p.K[s] % DK != 0);
    k_blocks = k_blocks && (p.K[s] % 64 == 0);  // k-major operands are copied in whole blocks of 64 k
  }
  const bool dma_ok = dma_offsets_fit(p, kind) && !(k_tail && kind == EPI_OUT && io_dtype == LT_BF16) &&
                      ((!a_km && !b_km) || k_blocks);
  return p.variant != 1 && dma_ok;
}

template <bool A_KM, bool B_KM, int KIND> int launch_tile(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  if (dma_selected(p, KIND, io_dtype)) return launch_dma<A_KM, B_KM, KIND>(p, io_dtype, stream);
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
