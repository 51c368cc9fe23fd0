// Host side of the tiled bf16 GEMMs: which problems the kernels of gemm_mfma_kernels.h take, which kernel a problem goes
// to, split reductions and their summing passes.  The kernels are instantiated per epilogue kind in gemm_mfma_kind*.hip.
#include "gemm_mfma_kernels.h"
#ifdef LT_TILE_TIMING
int& lt_tile_timing_launch_counter() { static int n = 0; return n; }
#endif

// defined in gemm_mfma_kind{0,1,2,3}.hip (KIND = EPI_STORE, EPI_ACT_FWD, EPI_ACT_BWD, EPI_OUT)
int lt_mfma_launch_dense_kind0(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_dense_kind1(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_dense_kind2(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_dense_kind3(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_sparse_kind0(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_sparse_kind1(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_sparse_kind2(const GemmProblem& p, int io_dtype, hipStream_t stream);
int lt_mfma_launch_sparse_kind3(const GemmProblem& p, int io_dtype, hipStream_t stream);
// 128 x 128 tile, plain store, `slices` slices of the reduction (gemm_mfma_kind0.hip)
int lt_mfma_launch_skinny(const GemmProblem& p, int slices, hipStream_t stream);


bool lt_gemm_mfma_supported(const GemmProblem& p, int kind) {
  constexpr int BM = 256, BN = 256;
  const bool gated = kind == EPI_ACT_FWD && p.epi.gated;
  if (p.M <= 0 || p.N <= 0) return false;
  const int64_t tile_n = gated ? BN / 2 : BN;
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  if (!a_km && b_km) return false;
  // Tiles that stick out past N (and past M for an mn-major A) are the copy-based kernel's: it copies the last row or the
  // last 8 columns again and its epilogue skips what is outside, 8 columns at a time.
  if (p.N % tile_n != 0 || (!a_km && p.M % BM != 0)) {
    if (p.N % 8 != 0 || (!a_km && p.M % 8 != 0) || !dma_selected(p, kind, LT_BF16)) return false;
  }
  if ((int64_t)((p.M + BM - 1) / BM) * ((p.N + tile_n - 1) / tile_n) > 0x7fffffff) return false;
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

bool lt_sparse_mfma_supported(const GemmProblem& p, int kind);

int lt_gemm_colsum_rows(const GemmProblem& p, int dtype, int io_dtype) {
  if (dtype != LT_BF16 || p.epi.ld_pre % 8 != 0) return 0;
  if (p.sp.mode == SPARSE_NONE)
    return lt_gemm_mfma_supported(p, EPI_ACT_BWD) && dma_selected(p, EPI_ACT_BWD, io_dtype) ? 128 : 0;
  // the walk's straight-line strips keep the sums: every tile must take them
  return p.sp.mode == SPARSE_DX && lt_sparse_mfma_supported(p, EPI_ACT_BWD) && p.M % 256 == 0 &&
                 p.epi.act == LT_ACT_GELU_FUSED && p.epi.hid
             ? 64 : 0;
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
    case EPI_STORE: return lt_mfma_launch_dense_kind0(p, io_dtype, stream);
    case EPI_ACT_FWD: return lt_mfma_launch_dense_kind1(p, io_dtype, stream);
    case EPI_ACT_BWD: return lt_mfma_launch_dense_kind2(p, io_dtype, stream);
    case EPI_OUT: return lt_mfma_launch_dense_kind3(p, io_dtype, stream);
  }
  LT_FAIL(LT_ERR_BAD_ARG, "unknown epilogue kind %d", kind);
}

namespace {
constexpr int SKINNY_MAX_SLICES = 16;
}  // namespace

// partial sums of up to SKINNY_MAX_SLICES slices of a [tokens, lowrank] (or equally large) fp32 result
size_t lt_gemm_skinny_workspace(int64_t tokens, int64_t lowrank) {
  return lt_align_up((size_t)SKINNY_MAX_SLICES * (size_t)tokens * (size_t)lowrank * sizeof(float), 256);
}

namespace {
// slices of the reduction for an [M, N] result on 256 x 256 tiles: enough workgroups for the 256 CUs, each slice at least
// 16 k-steps long
int splitk_slices(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (tiles >= 128) return 1;
  const int64_t by_k = K / (16 * DK);
  return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / tiles, by_k), 8));
}
}  // namespace

size_t lt_gemm_splitk_workspace(int64_t M, int64_t N, int64_t K) {
  const int slices = splitk_slices(M, N, K);
  return slices > 1 ? lt_align_up((size_t)slices * (size_t)M * (size_t)N * sizeof(float), 256) : 0;
}

namespace {
// the any-shape kernel runs four 128 x 128 workgroups per CU: slices of at least eight k-steps until about 1024 workgroups
int generic_splitk_slices(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  if (tiles >= 768) return 1;
  return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(1024 / tiles, K / 128), 16));
}
}  // namespace

size_t lt_gemm_generic_splitk_workspace(int64_t M, int64_t N, int64_t K) {
  const int slices = generic_splitk_slices(M, N, K);
  return slices > 1 ? lt_align_up((size_t)slices * (size_t)M * (size_t)N * sizeof(float), 256) : 0;
}

int lt_launch_gemm_skinny(const GemmProblem& p, int dtype, int io_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t stream) {
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  const EpiParams& e = p.epi;
  bool ok = dtype == LT_BF16 && p.nseg == 1 && p.sp.mode == SPARSE_NONE && p.M > 0 && p.N > 0 && p.N % 128 == 0 &&
            !(!a_km && b_km) && (a_km || p.M % 128 == 0) && ((!a_km && !b_km) || p.K[0] % BK == 0) && p.K[0] > 0 &&
            p.A[0].ld % 8 == 0 && p.B[0].ld % 8 == 0 && lt_aligned(p.A[0].ptr, 16) && lt_aligned(p.B[0].ptr, 16) &&
            e.ldo == p.N && lt_aligned(e.out, 16) && (!e.bias || lt_aligned(e.bias, 16));
  const int64_t tiles = ((p.M + 127) / 128) * (p.N / 128);
  // a result only 128 wide (or, for an mn-major A, 128 tall) would leave half of every 256 x 256 tile empty: the 128 x 128
  // tile below takes it when it can
  const bool half_tiles = ok && (p.N == 128 || (!a_km && p.M == 128));
  if (!half_tiles && dtype == LT_BF16 && p.sp.mode == SPARSE_NONE && lt_gemm_mfma_supported(p, EPI_STORE)) {
    // 256 x 256 tiles fit: the copy-based kernel, its reduction split when the tiles alone leave CUs idle
    const int slices = p.nseg == 1 ? splitk_slices(p.M, p.N, p.K[0]) : 1;
    const size_t need = (size_t)slices * (size_t)p.M * (size_t)p.N * sizeof(float);
    if (slices > 1 && workspace && workspace_bytes >= need && p.variant != 1 && p.K[0] % 64 == 0 && e.ldo == p.N &&
        dma_offsets_fit(p, EPI_STORE)) {
      GemmProblem q = p;
      q.ksplit = slices;
      q.split_stride = p.M * p.N;
      q.epi.out = workspace;
      q.epi.ldo = p.N;
      q.epi.out_dtype = LT_F32;
      q.epi.bias = nullptr;
      LT_TRY(lt_launch_gemm(q, EPI_STORE, dtype, io_dtype, stream));
      return lt_splitk_reduce((const float*)workspace, slices, p.M * p.N, p.M * p.N, (int)p.N, e.bias, e.out_dtype, e.out, stream);
    }
    if (((p.M + 255) / 256) * ((p.N + 255) / 256) >= 64 || slices == 1) ok = false;
  }
  if (!ok) {
    // any-shape kernel: split the reduction when the tiles alone leave most workgroup slots empty
    const bool tiled = dtype == LT_BF16 && lt_gemm_mfma_supported(p, EPI_STORE);
    const int slices = (!tiled && p.nseg == 1 && p.sp.mode == SPARSE_NONE && e.ldo == p.N && (p.N & 3) == 0 &&
                        lt_aligned(e.out, 16) && (!e.bias || lt_aligned(e.bias, 16)))
                           ? generic_splitk_slices(p.M, p.N, p.K[0]) : 1;
    if (slices > 1 && workspace && workspace_bytes >= (size_t)slices * (size_t)p.M * (size_t)p.N * sizeof(float)) {
      GemmProblem q = p;
      q.ksplit = slices;
      q.split_stride = p.M * p.N;
      q.epi.out = workspace;
      q.epi.out_dtype = LT_F32;
      q.epi.bias = nullptr;
      LT_TRY(lt_launch_gemm_generic(q, EPI_STORE, dtype, io_dtype, stream));
      return lt_splitk_reduce((const float*)workspace, slices, p.M * p.N, p.M * p.N, (int)p.N, e.bias, e.out_dtype, e.out, stream);
    }
    return lt_launch_gemm(p, EPI_STORE, dtype, io_dtype, stream);
  }
  const int kt_total = (int)((p.K[0] + BK - 1) / BK);
  int slices = 1;
  if (workspace && tiles < 192) {
    // two workgroups per CU (64 KiB of LDS each): the slices are short and bound by load latency
    // (one workgroup per CU where a slice's fp32 partial result is as large as the operand tile it read: with twice the
    // slices the partial sums cost more than the second workgroup hides -- measured on [4096, 128] results)
    const int64_t workgroups = tiles <= 64 ? 256 : 512;
    slices = (int)std::min<int64_t>(std::min<int64_t>(workgroups / tiles, kt_total / 4), SKINNY_MAX_SLICES);
    const int64_t fit = (int64_t)(workspace_bytes / ((size_t)p.M * (size_t)p.N * sizeof(float)));
    slices = (int)std::max<int64_t>(1, std::min<int64_t>(slices, fit));
  }
  GemmProblem q = p;
  if (slices > 1) {
    q.ksplit = slices;
    q.split_stride = p.M * p.N;
    q.epi.out = workspace;
    q.epi.out_dtype = LT_F32;
    q.epi.bias = nullptr;
  }
  {
    LtProfileScope scope("gemm_bf16_skinny", lt_gemm_flops(p, EPI_STORE), 0.0, stream);
    const int status = lt_mfma_launch_skinny(q, slices, stream);
    if (status != LT_OK || slices == 1) return status;
  }
  return lt_splitk_reduce((const float*)workspace, slices, p.M * p.N, p.M * p.N, (int)p.N, e.bias, e.out_dtype, e.out, stream);
}

namespace {
// sum of the split-k slices of an [M, N] result, 8 columns per thread, through the EPI_OUT epilogue (bias, dropout, residual)
template <typename TX>
__global__ __launch_bounds__(256) void splitk_reduce_out_kernel(const float* __restrict__ partial, int slices, int64_t stride,
                                                                 int64_t M, int64_t N, EpiParams e) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= M * N) return;
  float v[8];
  load8(partial + i, v);
  for (int s = 1; s < slices; s++) {
    float w[8];
    load8(partial + (int64_t)s * stride + i, w);
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] += w[k];
  }
  epi_out8<TX>(e, i / N, i % N, v);
}
}  // namespace

size_t lt_gemm_out_splitk_workspace(int64_t M, int64_t N, int64_t K, size_t cap_bytes) {
  const size_t full = std::max(lt_gemm_splitk_workspace(M, N, K), lt_gemm_generic_splitk_workspace(M, N, K));
  const size_t slice = (size_t)M * (size_t)N * sizeof(float);
  if (full == 0 || cap_bytes < 2 * slice) return 0;
  return std::min(full, lt_align_up(cap_bytes / slice * slice, 256));
}

int lt_launch_gemm_out(const GemmProblem& p, int dtype, int io_dtype, void* workspace, size_t workspace_bytes,
                       hipStream_t stream) {
  const EpiParams& e = p.epi;
  if (p.nseg == 1 && p.sp.mode == SPARSE_NONE && workspace && lt_aligned(workspace, 16) && p.M > 0 && p.N > 0 &&
      p.N % 8 == 0 && e.ldy % 8 == 0 && lt_aligned(e.y, 16) && (!e.x || lt_aligned(e.x, 16)) &&
      (!e.bias || lt_aligned(e.bias, 16))) {
    GemmProblem q = p;
    q.epi = EpiParams{};
    q.epi.out = workspace;
    q.epi.ldo = p.N;
    q.epi.out_dtype = LT_F32;
    const size_t slice = (size_t)p.M * (size_t)p.N * sizeof(float);
    // the tiled kernel where it takes the problem (a k-major reduction splits in blocks of 64), else the any-shape kernel
    const bool tiled = dtype == LT_BF16 && p.variant != 1 && p.K[0] % 64 == 0 && lt_gemm_mfma_supported(q, EPI_STORE) &&
                       dma_offsets_fit(q, EPI_STORE);
    const bool tiled_unsplit = dtype == LT_BF16 && lt_gemm_mfma_supported(p, EPI_OUT);
    const int wanted = tiled ? splitk_slices(p.M, p.N, p.K[0]) : tiled_unsplit ? 1 : generic_splitk_slices(p.M, p.N, p.K[0]);
    const int slices = (int)std::min<size_t>((size_t)wanted, workspace_bytes / slice);
    if (slices > 1) {
      q.ksplit = slices;
      q.split_stride = p.M * p.N;
      if (tiled) LT_TRY(lt_launch_gemm(q, EPI_STORE, dtype, io_dtype, stream));
      else LT_TRY(lt_launch_gemm_generic(q, EPI_STORE, dtype, io_dtype, stream));
      LtProfileScope scope("splitk_reduce_out", 0.0,
                           (double)p.M * p.N * (4.0 * slices + (e.x ? 2 : 1) * lt_dtype_size(io_dtype)), stream);
      const dim3 grid((unsigned)((p.M * p.N / 8 + 255) / 256)), block(256);
      if (io_dtype == LT_BF16)
        hipLaunchKernelGGL((splitk_reduce_out_kernel<bf16>), grid, block, 0, stream, (const float*)workspace, slices, p.M * p.N, p.M, p.N, e);
      else
        hipLaunchKernelGGL((splitk_reduce_out_kernel<float>), grid, block, 0, stream, (const float*)workspace, slices, p.M * p.N, p.M, p.N, e);
      LT_LAUNCH_CHECK();
      return LT_OK;
    }
  }
  return lt_launch_gemm(p, EPI_OUT, dtype, io_dtype, stream);
}

// block-sparse walk on the matrix cores: 64 x 64 blocks, bf16, 16-byte aligned operands
bool lt_sparse_mfma_supported(const GemmProblem& p, int kind) {
  const SparseWalk& sp = p.sp;
  const EpiParams& e = p.epi;
  if (sp.mode == SPARSE_NONE || sp.block != 64 || p.M <= 0) return false;
  // gated forward epilogue: p.N counts the gate columns; the walk pairs gate block j with linear block j + N / 64
  if (kind == EPI_ACT_FWD && e.gated && (sp.mode != SPARSE_FWD || p.N % 64 != 0 || e.inter != p.N)) return false;
  if (sp.ld_act % 8 != 0 || !lt_aligned(sp.act, 16)) return false;
  if (sp.mode == SPARSE_DW) {
    if (kind != EPI_STORE || sp.ld_act2 % 8 != 0 || !lt_aligned(sp.act2, 16) || !lt_aligned(e.out, 16)) return false;
    return true;
  }
  if (!lt_aligned(sp.weight, 16)) return false;
  if (p.nseg > 1) {
    if (p.K[1] <= 0 || p.K[1] % BK != 0 || p.A[1].ld % 8 != 0 || p.B[1].ld % 8 != 0 || !lt_aligned(p.A[1].ptr, 16) ||
        !lt_aligned(p.B[1].ptr, 16))
      return false;
  }
  if (e.bias && !lt_aligned(e.bias, 16)) return false;
  if (kind == EPI_STORE && (e.ldo % 8 != 0 || !lt_aligned(e.out, 16))) return false;
  if ((kind == EPI_ACT_FWD || kind == EPI_ACT_BWD) &&
      (e.ld_pre % 8 != 0 || e.ld_hid % 8 != 0 || e.inter % 8 != 0 || !lt_aligned(e.pre, 16) ||
       (e.hid && !lt_aligned(e.hid, 16)) || (e.dpre && !lt_aligned(e.dpre, 16))))
    return false;
  if (kind == EPI_OUT && (e.ldy % 8 != 0 || !lt_aligned(e.y, 16) || (e.x && !lt_aligned(e.x, 16)))) return false;
  return true;
}

bool lt_sparse_forward_grouped(const GemmProblem& p, int kind) {
  const SparseWalk& sp = p.sp;
  if (sp.mode != SPARSE_FWD || (kind != EPI_STORE && kind != EPI_ACT_FWD) || (kind == EPI_ACT_FWD && p.epi.gated)) return false;
  if (!lt_sparse_mfma_supported(p, kind)) return false;
  if (sp.out_group < 4 || sp.out_group % 4 != 0 || sp.out_stride > 1 || p.N % 256 != 0) return false;
  // the list travels in one register: at most 64 entries, input block and flat position in 16 bits each
  if (sp.blocks_per_out > 64 || sp.ld_act / 64 * sp.blocks_per_in > 65535) return false;
  if (p.nseg > 1 && p.K[1] % 64 != 0) return false;
  // 32-bit byte offsets inside a tile
  if (256 * sp.ld_act * 2 >= (int64_t)1 << 32) return false;
  if (p.nseg > 1 && (256 * p.A[1].ld * 2 >= (int64_t)1 << 32 || 256 * p.B[1].ld * 2 >= (int64_t)1 << 32)) return false;
  return true;
}

bool lt_sparse_dw_out_grouped(const GemmProblem& p) {
  const SparseWalk& sp = p.sp;
  const int64_t out_features = sp.ld_act;
  if (sp.out_stride > 1 && (int64_t)sp.out_group * sp.out_stride * 64 != out_features) return false;  // runs must tile the blocks
  return sp.mode == SPARSE_DW && sp.out_group >= 4 && sp.out_group % 4 == 0 && sp.forward_indices && out_features % 256 == 0 &&
         sp.tokens % DK == 0 && sp.tokens > 0 && 32 * sp.ld_act * 2 + out_features * 2 < (int64_t)1 << 32 &&
         32 * sp.ld_act2 * 2 + p.N * 2 < (int64_t)1 << 32;
}

int lt_sparse_dw_in_grouped_slices(const GemmProblem& p) {
  const SparseWalk& sp = p.sp;
  const int64_t out_features = sp.ld_act, in_features = p.N;
  if (sp.mode != SPARSE_DW || !lt_sparse_mfma_supported(p, EPI_STORE) || lt_sparse_dw_out_grouped(p)) return 0;
  if (sp.in_group < 4 || sp.in_group % 4 != 0 || !sp.backward_indices || in_features % 256 != 0) return 0;
  if (sp.in_stride > 1 && (int64_t)sp.in_group * sp.in_stride * 64 != in_features) return 0;  // runs must tile the blocks
  if (sp.tokens <= 0 || sp.tokens % DK != 0) return 0;
  if (32 * sp.ld_act * 2 + out_features * 2 >= (int64_t)1 << 32 || 32 * sp.ld_act2 * 2 + in_features * 2 >= (int64_t)1 << 32) return 0;
  // enough workgroups for the 256 CUs, each slice at least 32 k-steps long
  const int64_t tiles = (int64_t)((sp.blocks_per_in + 3) / 4) * (in_features / 256);
  if (tiles >= 192) return 1;
  return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / tiles, sp.tokens / (32 * DK)), 8));
}

size_t lt_sparse_dw_split_workspace(int64_t in_features, int blocks_per_in, int in_group, int64_t tokens) {
  if (in_group < 4 || in_features % 256 != 0) return 0;
  // (an upper bound that needs no more than the layer's shape: 8 slices at most)
  const int64_t tiles = (int64_t)((blocks_per_in + 3) / 4) * (in_features / 256);
  if (tiles >= 192) return 0;
  const int64_t slices = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / tiles, tokens / (32 * DK)), 8));
  return slices > 1 ? lt_align_up((size_t)slices * (size_t)(in_features / 64) * blocks_per_in * 4096 * sizeof(float), 256) : 0;
}

int lt_launch_gemm_sparse(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream) {
  if (dtype != LT_BF16 || !lt_sparse_mfma_supported(p, kind)) return lt_launch_gemm_generic(p, kind, dtype, io_dtype, stream);
  const SparseWalk& sp = p.sp;
  const double steps = sp.mode == SPARSE_FWD ? sp.blocks_per_out : sp.blocks_per_in;
  double flops = 2.0 * (double)p.M * (double)p.N * (steps * 64.0 + (p.nseg > 1 ? (double)p.K[1] : 0.0));
  if (kind == EPI_ACT_FWD && p.epi.gated) flops *= 2.0;
  if (sp.mode == SPARSE_DW) flops = 2.0 * (double)sp.tokens * (double)(p.N / 64) * sp.blocks_per_in * 4096.0;
  static const char* tags[4] = {"", "blocksparse_fwd_bf16", "blocksparse_dx_bf16", "blocksparse_dw_bf16"};
  LtProfileScope scope(tags[sp.mode], flops, 0.0, stream);
  switch (kind) {
    case EPI_STORE: return lt_mfma_launch_sparse_kind0(p, io_dtype, stream);
    case EPI_ACT_FWD: return lt_mfma_launch_sparse_kind1(p, io_dtype, stream);
    case EPI_ACT_BWD: return lt_mfma_launch_sparse_kind2(p, io_dtype, stream);
    case EPI_OUT: return lt_mfma_launch_sparse_kind3(p, io_dtype, stream);
  }
  LT_FAIL(LT_ERR_BAD_ARG, "unknown epilogue kind %d", kind);
}

int lt_launch_gemm(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream) {
  if (dtype == LT_BF16 && lt_gemm_mfma_supported(p, kind)) return lt_launch_gemm_mfma(p, kind, io_dtype, stream);
  return lt_launch_gemm_generic(p, kind, dtype, io_dtype, stream);
}
