// Any-shape GEMM with fused epilogues: fp32 or bf16 operands with arbitrary leading dimensions and either operand
// transposed, fp32 matrix-core arithmetic (v_mfma_f32_32x32x2_f32).  This is the kernel of the fp32 path, of every shape
// the tiled bf16 kernel does not take (ragged hidden sizes, skinny low-rank factors), and -- with a SparseWalk -- of the
// block-sparse matmul for any block size: a group of workgroups (blockIdx.z) then walks the index table of one output
// block / input block / weight block and treats each active block as one k-segment.
//
// Work decomposition: 256 threads = 4 wavefronts in a 2 x 2 grid over a 128 x 128 output tile; each wavefront owns a
// 64 x 64 quadrant as 2 x 2 MFMA blocks of 32 x 32.  Operand tiles of 16 k-steps are converted to fp32 on load and staged
// in LDS k-major ([k][row], padded by 4 floats so the 32 rows x 2 k-lanes of one MFMA operand read conflict-free); the loads
// of the next step are in flight (in registers) while the matrix cores work on the current one.
#include "lt_gemm.h"

namespace {

constexpr int GBM = 128, GBN = 128, GBK = 16, GPAD = 4;

template <typename TI> struct Segment {
  const TI* A;
  const TI* B;
  int64_t lda, ldb, K;
  bool a_km, b_km;
};

template <typename TI, int KIND, typename TC, typename TX>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmProblem p) {
  __shared__ __attribute__((aligned(16))) float As[2][GBK][GBM + GPAD];
  __shared__ __attribute__((aligned(16))) float Bs[2][GBK][GBN + GPAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const bool gated = (KIND == EPI_ACT_FWD) && p.epi.gated;
  const int64_t m0 = (int64_t)blockIdx.y * GBM;
  // gated forward: a tile holds 64 gate columns and the 64 matching linear columns, split per wavefront so that one lane
  // owns both members of a pair: tile column c -> wavefront c / 64, MFMA block (c % 64) / 32 = half, offset c % 32
  const int64_t n0 = (int64_t)blockIdx.x * (gated ? GBN / 2 : GBN);

  // ---- problem seen by this workgroup: dense, or one group of a block-sparse walk
  const SparseWalk& sp = p.sp;
  const int group = blockIdx.z;
  const int b = sp.block;
  int64_t M = p.M, N = p.N;  // bounds of the local tile coordinates
  int64_t n_off = 0;         // global column of local column 0 (epilogue indices)
  int nseg = p.nseg;
  EpiParams epi = p.epi;
  if (sp.mode == SPARSE_FWD) {
    N = b; n_off = (int64_t)group * b; nseg = sp.blocks_per_out + (p.nseg > 1);
  } else if (sp.mode == SPARSE_DX) {
    N = b; n_off = (int64_t)group * b; nseg = sp.blocks_per_in + (p.nseg > 1);
  } else if (sp.mode == SPARSE_DW) {
    M = b; N = b; nseg = 1;
    epi.out = reinterpret_cast<char*>(epi.out) + (int64_t)group * b * b * (epi.out_dtype == LT_F32 ? 4 : 2);
    epi.ldo = b;
  }
  if (m0 >= M || n0 >= N) return;  // whole workgroup
  const int64_t b_rows = gated ? 2 * N : N;

  auto segment = [&](int s) -> Segment<TI> {
    Segment<TI> g;
    if (sp.mode == SPARSE_NONE) {
      g.A = reinterpret_cast<const TI*>(p.A[s].ptr); g.lda = p.A[s].ld; g.a_km = p.A[s].kmajor;
      g.B = reinterpret_cast<const TI*>(p.B[s].ptr); g.ldb = p.B[s].ld; g.b_km = p.B[s].kmajor;
      g.K = p.K[s];
    } else if (sp.mode == SPARSE_FWD) {
      if (s < sp.blocks_per_out) {
        const int f = sp.forward_indices[(int64_t)group * sp.blocks_per_out + s];
        const int ib = f / sp.blocks_per_in;
        g.A = reinterpret_cast<const TI*>(sp.act) + (int64_t)ib * b; g.lda = sp.ld_act; g.a_km = true;
        g.B = reinterpret_cast<const TI*>(sp.weight) + (int64_t)f * b * b; g.ldb = b; g.b_km = true;
        g.K = b;
      } else {  // low-rank: hid [M, r] x second[out, r]^T restricted to this output block
        g.A = reinterpret_cast<const TI*>(p.A[1].ptr); g.lda = p.A[1].ld; g.a_km = true;
        g.B = reinterpret_cast<const TI*>(p.B[1].ptr) + n_off * p.B[1].ld; g.ldb = p.B[1].ld; g.b_km = true;
        g.K = p.K[1];
      }
    } else if (sp.mode == SPARSE_DX) {
      if (s < sp.blocks_per_in) {
        const int64_t ob = sp.backward_indices[(int64_t)group * sp.blocks_per_in + s];
        g.A = reinterpret_cast<const TI*>(sp.act) + ob * b; g.lda = sp.ld_act; g.a_km = true;
        // B(n = input column c, k = output row rho) = W4[ib, a, rho, c]: k strided by b
        g.B = reinterpret_cast<const TI*>(sp.weight) + ((int64_t)group * sp.blocks_per_in + s) * b * b; g.ldb = b;
        g.b_km = false;
        g.K = b;
      } else {  // low-rank: g_hid [M, r] x first[r, in] restricted to this input block
        g.A = reinterpret_cast<const TI*>(p.A[1].ptr); g.lda = p.A[1].ld; g.a_km = true;
        g.B = reinterpret_cast<const TI*>(p.B[1].ptr) + n_off; g.ldb = p.B[1].ld; g.b_km = false;
        g.K = p.K[1];
      }
    } else {  // SPARSE_DW: rows = output row rho of block ob, columns = input column c of block ib, reduce over tokens
      const int ib = group / sp.blocks_per_in;
      const int64_t ob = sp.backward_indices[group];
      g.A = reinterpret_cast<const TI*>(sp.act) + ob * b; g.lda = sp.ld_act; g.a_km = false;
      g.B = reinterpret_cast<const TI*>(sp.act2) + (int64_t)ib * b; g.ldb = sp.ld_act2; g.b_km = false;
      g.K = sp.tokens;
    }
    return g;
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // ---- main loop, software-pipelined: the 128 x 16 operand tiles of step i + 1 are fetched into registers (two 4-element
  //      vectors per operand and thread, along the contiguous axis; element by element where alignment or bounds do not
  //      allow vectors) while the matrix cores work on step i out of LDS; two LDS buffers, one barrier per step.
  struct Fetch {
    float a[2][4], b[2][4];
  };
  int seg = 0;
  Segment<TI> g = segment(0);
  int64_t k0 = 0;
  if (sp.mode == SPARSE_NONE && p.ksplit > 1) {
    // split reduction (one k-segment, EPI_STORE): slice blockIdx.z walks a whole number of k-steps and stores fp32 partial
    // sums at epi.out + slice * split_stride
    const int64_t steps = (g.K + GBK - 1) / GBK, per = (steps + p.ksplit - 1) / p.ksplit * GBK;
    k0 = min(g.K, (int64_t)blockIdx.z * per);
    g.K = min(g.K, k0 + per);
    epi.out = reinterpret_cast<float*>(epi.out) + (int64_t)blockIdx.z * p.split_stride;
  }
  auto fetch = [&](Fetch& f) {
    // A: k-major -> 4 consecutive k of one row; mn-major -> 4 consecutive rows of one k
    const bool va = (reinterpret_cast<uintptr_t>(g.A) % (4 * sizeof(TI)) == 0) && (g.lda & 3) == 0 &&
                    (g.a_km ? (g.K & 3) == 0 : (M & 3) == 0);
#pragma unroll
    for (int i = 0; i < 2; i++) {
      int kk, mm;
      if (g.a_km) { kk = (tid & 3) * 4; mm = (tid >> 2) + i * 64; } else { mm = (tid & 31) * 4; kk = (tid >> 5) + i * 8; }
      const int64_t gm = m0 + mm, gk = k0 + kk;
#pragma unroll
      for (int e = 0; e < 4; e++) f.a[i][e] = 0.f;
      if (gm < M && gk < g.K) {
        if (va) {
          load4(g.a_km ? g.A + gm * g.lda + gk : g.A + gk * g.lda + gm, f.a[i]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (g.a_km) { if (gk + e < g.K) f.a[i][e] = ldf(g.A, gm * g.lda + gk + e); }
            else if (gm + e < M) f.a[i][e] = ldf(g.A, gk * g.lda + gm + e);
          }
        }
      }
    }
    const bool vb = (reinterpret_cast<uintptr_t>(g.B) % (4 * sizeof(TI)) == 0) && (g.ldb & 3) == 0 &&
                    (g.b_km ? (g.K & 3) == 0 : (N & 3) == 0);
#pragma unroll
    for (int i = 0; i < 2; i++) {
      int kk, cc;
      if (g.b_km) { kk = (tid & 3) * 4; cc = (tid >> 2) + i * 64; } else { cc = (tid & 31) * 4; kk = (tid >> 5) + i * 8; }
      // global row of B for tile column cc (+ e along n when mn-major); b_rows = out of range
      int64_t gn;
      if (gated) {
        const int64_t ng = n0 + (cc >> 6) * 32 + (cc & 31);
        gn = ng < N ? ((cc >> 5) & 1) * N + ng : b_rows;
      } else {
        gn = n0 + cc < N ? n0 + cc : b_rows;
      }
      const int64_t gk = k0 + kk;
#pragma unroll
      for (int e = 0; e < 4; e++) f.b[i][e] = 0.f;
      if (gn < b_rows && gk < g.K) {
        if (vb) {
          load4(g.b_km ? g.B + gn * g.ldb + gk : g.B + gk * g.ldb + gn, f.b[i]);
        } else {
          const int64_t n_left = (gated ? N - (n0 + (cc >> 6) * 32 + (cc & 31)) : N - (n0 + cc));
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (g.b_km) { if (gk + e < g.K) f.b[i][e] = ldf(g.B, gn * g.ldb + gk + e); }
            else if (e < n_left) f.b[i][e] = ldf(g.B, gk * g.ldb + gn + e);
          }
        }
      }
    }
  };
  // f holds the step (seg, k0) points at: g is its segment
  auto stash = [&](const Fetch& f, int buf) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      if (g.a_km) {
        const int kk = (tid & 3) * 4, mm = (tid >> 2) + i * 64;
#pragma unroll
        for (int e = 0; e < 4; e++) As[buf][kk + e][mm] = f.a[i][e];
      } else {
        const int mm = (tid & 31) * 4, kk = (tid >> 5) + i * 8;
        *reinterpret_cast<float4*>(&As[buf][kk][mm]) = make_float4(f.a[i][0], f.a[i][1], f.a[i][2], f.a[i][3]);
      }
      if (g.b_km) {
        const int kk = (tid & 3) * 4, cc = (tid >> 2) + i * 64;
#pragma unroll
        for (int e = 0; e < 4; e++) Bs[buf][kk + e][cc] = f.b[i][e];
      } else {
        const int cc = (tid & 31) * 4, kk = (tid >> 5) + i * 8;
        *reinterpret_cast<float4*>(&Bs[buf][kk][cc]) = make_float4(f.b[i][0], f.b[i][1], f.b[i][2], f.b[i][3]);
      }
    }
  };
  // advance (seg, k0) to the next step; false at the end
  auto advance = [&]() -> bool {
    k0 += GBK;
    if (k0 < g.K) return true;
    if (++seg >= nseg) return false;
    g = segment(seg);
    k0 = 0;
    return true;
  };

  Fetch f;
  fetch(f);  // an empty slice (k0 == K) fetches zeros
  stash(f, 0);
  __syncthreads();
  int buf = 0;
  for (;;) {
    const bool more = advance();
    if (more) fetch(f);  // in flight while the matrix cores run
#pragma unroll
    for (int kk = 0; kk < GBK; kk += 2) {
      float a[2], bfrag[2];
#pragma unroll
      for (int i = 0; i < 2; i++) a[i] = As[buf][kk + (lane >> 5)][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < 2; j++) bfrag[j] = Bs[buf][kk + (lane >> 5)][wn * 64 + j * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], bfrag[j], acc[i][j], 0, 0, 0);
    }
    if (!more) break;
    stash(f, buf ^ 1);  // the other buffer: its last readers passed the previous barrier
    __syncthreads();
    buf ^= 1;
  }

  // ---- epilogue: accumulator register r of a 32 x 32 block is row 8 * (r / 4) + 4 * (lane / 32) + r % 4, column lane % 32
#pragma unroll
  for (int i = 0; i < 2; i++) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (m >= M) continue;
      if (gated) {
        const int64_t n = n0 + wn * 32 + (lane & 31);
        if (n < N) epi_act_fwd_gated<TC>(epi, m, n, acc[i][0][r], acc[i][1][r]);
      } else {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const int64_t nl = n0 + wn * 64 + j * 32 + (lane & 31);
          if (nl >= N) continue;
          const int64_t n = n_off + nl;
          const float v = acc[i][j][r];
          if constexpr (KIND == EPI_STORE) {
            if (epi.out_dtype == LT_F32) epi_store<float>(epi, m, n, v); else epi_store<bf16>(epi, m, n, v);
          } else if constexpr (KIND == EPI_ACT_FWD) {
            epi_act_fwd<TC>(epi, m, n, v);
          } else if constexpr (KIND == EPI_ACT_BWD) {
            epi_act_bwd<TC>(epi, m, n, v);
          } else {
            epi_out<TX>(epi, m, n, v);
          }
        }
      }
    }
  }
}

template <typename TI, int KIND, typename TC>
int launch_io(const GemmProblem& p, int io_dtype, dim3 grid, hipStream_t stream) {
  if (KIND == EPI_OUT && io_dtype == LT_BF16) {
    hipLaunchKernelGGL((gemm_generic_kernel<TI, KIND, TC, bf16>), grid, dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL((gemm_generic_kernel<TI, KIND, TC, float>), grid, dim3(256), 0, stream, p);
  }
  LT_LAUNCH_CHECK();
  return LT_OK;
}

template <typename T> int launch_kind(const GemmProblem& p, int kind, int io_dtype, dim3 grid, hipStream_t stream) {
  switch (kind) {
    case EPI_STORE: return launch_io<T, EPI_STORE, T>(p, io_dtype, grid, stream);
    case EPI_ACT_FWD: return launch_io<T, EPI_ACT_FWD, T>(p, io_dtype, grid, stream);
    case EPI_ACT_BWD: return launch_io<T, EPI_ACT_BWD, T>(p, io_dtype, grid, stream);
    case EPI_OUT: return launch_io<T, EPI_OUT, T>(p, io_dtype, grid, stream);
  }
  LT_FAIL(LT_ERR_BAD_ARG, "unknown epilogue kind %d", kind);
}

}  // namespace

int lt_launch_gemm_generic(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream) {
  LT_REQUIRE(p.M > 0 && p.N > 0 && p.nseg >= 1 && p.nseg <= 2, LT_ERR_BAD_ARG, "gemm: bad sizes M=%lld N=%lld nseg=%d",
             (long long)p.M, (long long)p.N, p.nseg);
  const bool gated = kind == EPI_ACT_FWD && p.epi.gated;
  int64_t rows = p.M, cols = p.N, groups = 1;
  const SparseWalk& sp = p.sp;
  if (sp.mode != SPARSE_NONE) {
    LT_REQUIRE(!gated, LT_ERR_UNSUPPORTED, "block-sparse gemm has no gated-activation epilogue");
    LT_REQUIRE(sp.block > 0 && sp.blocks_per_in > 0 && sp.blocks_per_out > 0, LT_ERR_BAD_ARG, "block-sparse gemm: bad layout");
    cols = sp.block;
    if (sp.mode == SPARSE_DW) {
      rows = sp.block;
      groups = p.N / sp.block * sp.blocks_per_in;  // N = in_features
    } else {
      groups = p.N / sp.block;  // N = out_features (FWD) or in_features (DX)
    }
    LT_REQUIRE(groups >= 1 && groups <= 65535, LT_ERR_UNSUPPORTED, "block-sparse gemm: %lld groups exceed the grid limit",
               (long long)groups);
  }
  const int64_t tiles_n = (cols + (gated ? GBN / 2 : GBN) - 1) / (gated ? GBN / 2 : GBN);
  const int64_t tiles_m = (rows + GBM - 1) / GBM;
  LT_REQUIRE(tiles_m <= 65535, LT_ERR_UNSUPPORTED, "gemm: M=%lld exceeds the grid limit", (long long)p.M);
  double flops = lt_gemm_flops(p, kind);
  if (sp.mode == SPARSE_FWD || sp.mode == SPARSE_DX) {
    flops = 2.0 * (double)p.M * (double)p.N * ((sp.mode == SPARSE_FWD ? sp.blocks_per_out : sp.blocks_per_in) * (double)sp.block +
                                                (p.nseg > 1 ? (double)p.K[1] : 0.0));
  } else if (sp.mode == SPARSE_DW) {
    flops = 2.0 * (double)sp.tokens * (double)groups * sp.block * sp.block;
  }
  static const char* tags[4] = {"gemm_generic", "blocksparse_fwd_generic", "blocksparse_dx_generic", "blocksparse_dw_generic"};
  LtProfileScope scope(tags[sp.mode], flops, 0.0, stream);
  if (sp.mode == SPARSE_NONE && p.ksplit > 1) {
    LT_REQUIRE(kind == EPI_STORE && p.nseg == 1 && p.epi.out_dtype == LT_F32 && !p.epi.bias, LT_ERR_BAD_ARG,
               "gemm: a split reduction stores fp32 partial sums of one k-segment");
    groups = p.ksplit;
  }
  dim3 grid((unsigned)tiles_n, (unsigned)tiles_m, (unsigned)groups);
  return dtype == LT_F32 ? launch_kind<float>(p, kind, io_dtype, grid, stream)
                         : launch_kind<bf16>(p, kind, io_dtype, grid, stream);
}
