// GEMM problem description and fused epilogues shared by the any-shape kernel and the tiled bf16 MFMA kernel.
#pragma once
#include "lt_common.h"

// C[m, n] = sum over up to two K segments of  sum_k A_s(m, k) * B_s(n, k)   (fp32 accumulation), then one epilogue.
// The second segment carries the low-rank term of a generalized linear layer without a second pass over C.
struct GemmOperand {
  const void* ptr;
  int64_t ld;   // leading dimension in elements
  int kmajor;   // 1: element (i, k) at ptr[i * ld + k]; 0: at ptr[k * ld + i]
};

enum EpiKind {
  EPI_STORE = 0,    // out[m, n] = acc + bias[n]
  EPI_ACT_FWD = 1,  // up-projection: store pre-activation, apply (gated) activation, store hidden
  EPI_ACT_BWD = 2,  // d(hidden) -> d(pre-activation) (both halves when gated) and the re-materialised hidden
  EPI_OUT = 3       // down-projection: + bias, dropout, + residual, store y
};

struct EpiParams {
  const float* bias;  // indexed by the global output column; may be null
  // EPI_STORE
  void* out;
  int64_t ldo;
  int out_dtype;
  // EPI_ACT_FWD / EPI_ACT_BWD
  void* pre;          // ACT_FWD: written, ACT_BWD: read.  [M, gated ? 2I : I]
  int64_t ld_pre;
  void* hid;          // [M, I], written (may be null in ACT_BWD)
  int64_t ld_hid;
  void* dpre;         // ACT_BWD: [M, gated ? 2I : I], written
  int gated;
  int act;
  int64_t inter;      // I
  // ACT_BWD where lt_gemm_colsum_rows says so: column sums of the dpre values as stored, one partial row per R rows of the
  // output (R = that function's result): colsum[(m / R) * ld_pre + column].  Null = off.
  float* colsum;
  // EPI_OUT
  const void* x;      // residual input [M, ldy] (null = no residual)
  void* y;            // [M, ldy]
  int64_t ldy;        // row width of x / y; element (m, n) draws dropout word m * ldy + n
  DropoutParams drop;
};

// Block-sparse operand walk (any-shape kernel only).  Workgroups with the same blockIdx.z form one group:
//   SPARSE_FWD  group = output block ob:  Y[:, ob] = sum_k X[:, ib_k] W4[ib_k, a_k]^T,  forward_indices[ob, k] = ib_k * A + a_k
//   SPARSE_DX   group = input block ib:   dX[:, ib] = sum_a dY[:, ob_a] W4[ib, a],       ob_a = backward_indices[ib, a]
//   SPARSE_DW   group = weight block (ib, a): dW4[ib, a] = dY[:, ob_a]^T X[:, ib]
// W4 = the native weight [in_features, A, block] read as [in_blocks, A, block (output row), block (input column)].
// In FWD / DX an optional dense low-rank segment (A[1], B[1], K[1] of the enclosing problem) is appended.
enum SparseMode { SPARSE_NONE = 0, SPARSE_FWD = 1, SPARSE_DX = 2, SPARSE_DW = 3 };

struct SparseWalk {
  int mode;
  int block;           // b
  int blocks_per_out;  // K
  int blocks_per_in;   // A
  const int32_t* forward_indices;
  const int64_t* backward_indices;
  const void* act;     // FWD: X [M, in]; DX / DW: dY [M(tokens), out]
  int64_t ld_act;
  const void* weight;  // FWD / DX: W4
  const void* act2;    // DW: X [tokens, in]
  int64_t ld_act2;
  int64_t tokens;      // DW: reduction length
  // FWD / DW: every aligned run of this many consecutive output blocks shares one list of input blocks (0 / 1: not known to).
  // With runs of 4 or more the weight gradient is computed on 256 x 256 tiles (4 output blocks x 4 input blocks of the
  // shared list), which read every dY column block once per 4 input blocks instead of once per input block.
  int out_group;
  // DW: every aligned run of this many consecutive input blocks shares one list of output blocks (0 / 1: not known to).  With
  // runs of 4 or more, and none on the output side, the weight gradient runs on 256 x 256 tiles of 4 list entries x 4 input
  // blocks.
  int in_group;
  // blocks between the members of such a run: 0 or 1 = consecutive blocks; s > 1 = blocks r, r + s, r + 2 s, ... (a layout tiled
  // from a square pattern s blocks wide; the group length times s is then the number of blocks).  Strided runs serve the
  // weight gradient only.
  int out_stride, in_stride;
  // FWD / DX walks (matrix-core kernel): order in which a group's index list is walked.  0 / 1: as listed.  g > 1 (must divide
  // the list's length n): entry (t % (n / g)) * g + t / (n / g) at step t, i.e. the first members of the list's runs of g,
  // then the second members, ...  In a stretched butterfly a list is made of runs of g consecutive blocks and the groups that
  // share an activation block hold it at neighbouring positions of neighbouring runs: taken run-member by run-member they
  // read it within a step or two of each other instead of g steps apart, while it is still in the XCD's L2.  Any g that
  // divides n gives the same sums in another order; a g that fits no structure only costs what it would have gained.
  int walk_run;
};

struct GemmProblem {
  int64_t M;
  int64_t N;  // output columns; for a gated EPI_ACT_FWD this counts gate columns (I) and B has 2I rows
  int nseg;
  int64_t K[2];
  GemmOperand A[2], B[2];
  EpiParams epi;
  SparseWalk sp;  // sp.mode == SPARSE_NONE for a dense problem
  // split-k (tiled kernel, EPI_STORE only): blockIdx.y = slice of the k-steps; slice s stores fp32 partial sums at
  // epi.out + s * split_stride elements, summed afterwards in slice order (deterministic)
  int ksplit;
  int64_t split_stride;
  int krot;  // copy-based kernel: how workgroups stagger their walk over k (0: all start at k = 0)
  int variant;  // tiled bf16 kernels: 0 the launcher's choice, 1 the register-staged kernel where the copy-based one applies
  int tile_loop;  // copy-based kernel: 0 the launcher's choice (one workgroup per CU that loops over its tiles when there are
                  // more tiles than CUs), 1 one workgroup per tile
  unsigned long long* tile_stamps;  // instrumented build only (-DLT_TILE_TIMING): 8 words of clock stamps per tile; else null
};

// ---------------------------------------------------------------------------------------------------------------------
// per-element epilogues.  TC: compute dtype (pre-activation, hidden, gradients of them), TX: dtype of x / y.
// ---------------------------------------------------------------------------------------------------------------------
template <typename TO> __device__ __forceinline__ void epi_store(const EpiParams& e, int64_t m, int64_t n, float v) {
  if (e.bias) v += e.bias[n];
  stf(reinterpret_cast<TO*>(e.out), m * e.ldo + n, v);
}

template <typename TC> __device__ __forceinline__ void epi_act_fwd(const EpiParams& e, int64_t m, int64_t n, float v) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  if (e.bias) v += e.bias[n];
  TC pv = from_f32<TC>(v);
  reinterpret_cast<TC*>(e.pre)[m * e.ld_pre + n] = pv;
  stf(reinterpret_cast<TC*>(e.hid), m * e.ld_hid + n, act_value<PRECISE>(e.act, to_f32(pv)));
}

// gated: column n of the gate half pairs with column I + n of the linear half
template <typename TC>
__device__ __forceinline__ void epi_act_fwd_gated(const EpiParams& e, int64_t m, int64_t n, float vg, float vl) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  if (e.bias) {
    vg += e.bias[n];
    vl += e.bias[e.inter + n];
  }
  TC pg = from_f32<TC>(vg), pl = from_f32<TC>(vl);
  TC* pre = reinterpret_cast<TC*>(e.pre);
  pre[m * e.ld_pre + n] = pg;
  pre[m * e.ld_pre + e.inter + n] = pl;
  stf(reinterpret_cast<TC*>(e.hid), m * e.ld_hid + n, act_value<PRECISE>(e.act, to_f32(pg)) * to_f32(pl));
}

template <typename TC> __device__ __forceinline__ void epi_act_bwd(const EpiParams& e, int64_t m, int64_t n, float dh) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  const TC* pre = reinterpret_cast<const TC*>(e.pre);
  TC* dpre = reinterpret_cast<TC*>(e.dpre);
  TC* hid = reinterpret_cast<TC*>(e.hid);
  float a, da;
  if (e.gated) {
    float pg = to_f32(pre[m * e.ld_pre + n]), pl = to_f32(pre[m * e.ld_pre + e.inter + n]);
    act_eval<PRECISE>(e.act, pg, a, da);
    stf(dpre, m * e.ld_pre + n, dh * pl * da);
    stf(dpre, m * e.ld_pre + e.inter + n, dh * a);
    if (hid) stf(hid, m * e.ld_hid + n, a * pl);
  } else {
    float p = to_f32(pre[m * e.ld_pre + n]);
    act_eval<PRECISE>(e.act, p, a, da);
    stf(dpre, m * e.ld_pre + n, dh * da);
    if (hid) stf(hid, m * e.ld_hid + n, a);
  }
}

template <typename TX> __device__ __forceinline__ void epi_out(const EpiParams& e, int64_t m, int64_t n, float v) {
  if (e.bias) v += e.bias[n];
  int64_t idx = m * e.ldy + n;
  if (e.drop.p > 0.f) v = dropout_keep(e.drop, idx) ? v * e.drop.scale : 0.f;
  if (e.x) v += ldf(reinterpret_cast<const TX*>(e.x), idx);
  stf(reinterpret_cast<TX*>(e.y), idx, v);
}

// ---------------------------------------------------------------------------------------------------------------------
// the same epilogues on 8 consecutive columns n .. n + 7 of row m (n a multiple of 8, all leading dimensions multiples
// of 8): 16-byte global accesses, one Philox block per 4 elements.  Used by the tiled bf16 kernel (TC = bf16).
// ---------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ void add_bias8(const float* bias, int64_t n, float (&v)[8]) {
  if (bias) {
    float b[8];
    load8(bias + n, b);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] += b[i];
  }
}

__device__ __forceinline__ void epi_store8(const EpiParams& e, int64_t m, int64_t n, float (&v)[8]) {
  add_bias8(e.bias, n, v);
  if (e.out_dtype == LT_F32) store8(reinterpret_cast<float*>(e.out) + m * e.ldo + n, v);
  else store8(reinterpret_cast<bf16*>(e.out) + m * e.ldo + n, v);
}

__device__ __forceinline__ void epi_act_fwd8(const EpiParams& e, int64_t m, int64_t n, float (&v)[8]) {
  add_bias8(e.bias, n, v);
  float h[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    v[i] = to_f32((bf16)v[i]);  // the activation sees the stored (rounded) pre-activation, as backward will
    h[i] = act_value<false>(e.act, v[i]);
  }
  store8(reinterpret_cast<bf16*>(e.pre) + m * e.ld_pre + n, v);
  store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, h);
}

__device__ __forceinline__ void epi_act_fwd_gated8(const EpiParams& e, int64_t m, int64_t n, float (&vg)[8], float (&vl)[8]) {
  add_bias8(e.bias, n, vg);
  add_bias8(e.bias, e.inter + n, vl);
  float h[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    vg[i] = to_f32((bf16)vg[i]);
    vl[i] = to_f32((bf16)vl[i]);
    h[i] = act_value<false>(e.act, vg[i]) * vl[i];
  }
  bf16* pre = reinterpret_cast<bf16*>(e.pre) + m * e.ld_pre + n;
  store8(pre, vg);
  store8(pre + e.inter, vl);
  store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, h);
}

__device__ __forceinline__ void epi_act_bwd8(const EpiParams& e, int64_t m, int64_t n, const float (&dh)[8]) {
  const bf16* pre = reinterpret_cast<const bf16*>(e.pre) + m * e.ld_pre + n;
  bf16* dpre = reinterpret_cast<bf16*>(e.dpre) + m * e.ld_pre + n;
  float pg[8], a[8], da[8], o[8];
  load8(pre, pg);
#pragma unroll
  for (int i = 0; i < 8; i++) act_eval<false>(e.act, pg[i], a[i], da[i]);
  if (e.gated) {
    float pl[8];
    load8(pre + e.inter, pl);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * pl[i] * da[i];
    store8(dpre, o);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * a[i];
    store8(dpre + e.inter, o);
#pragma unroll
    for (int i = 0; i < 8; i++) a[i] *= pl[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * da[i];
    store8(dpre, o);
  }
  if (e.hid) store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, a);
}

template <typename TX> __device__ __forceinline__ void epi_out8(const EpiParams& e, int64_t m, int64_t n, float (&v)[8]) {
  add_bias8(e.bias, n, v);
  const int64_t idx = m * e.ldy + n;
  if (e.drop.p > 0.f) {
    bool k0[4], k1[4];
    dropout_keep4(e.drop, idx, k0);
    dropout_keep4(e.drop, idx + 4, k1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[i] = k0[i] ? v[i] * e.drop.scale : 0.f;
      v[i + 4] = k1[i] ? v[i + 4] * e.drop.scale : 0.f;
    }
  }
  if (e.x) {
    float r[8];
    load8(reinterpret_cast<const TX*>(e.x) + idx, r);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] += r[i];
  }
  store8(reinterpret_cast<TX*>(e.y) + idx, v);
}

// ---------------------------------------------------------------------------------------------------------------------
// Epilogues that READ global memory (the pre-activation in EPI_ACT_BWD, the residual in EPI_OUT) are split into a load
// step and a compute/store step, so that the tiled kernel can keep the loads of later rows in flight while it works on
// the current ones (a workgroup owns a whole compute unit there: nobody else hides its memory latency).
// ---------------------------------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int lt_u32x4;
struct EpiLoad {
  lt_u32x4 a, b;  // EPI_ACT_BWD: 8 gate and 8 linear pre-activations (bf16); EPI_OUT: 8 residual values (fp32: a|b, bf16: a)
};

template <int KIND, typename TX>
__device__ __forceinline__ EpiLoad epi_load8(const EpiParams& e, int64_t m, int64_t n, bool valid) {
  EpiLoad l;
  l.a = lt_u32x4{0u, 0u, 0u, 0u};
  l.b = l.a;
  if (!valid) return l;
  if constexpr (KIND == EPI_ACT_BWD) {
    const bf16* pre = reinterpret_cast<const bf16*>(e.pre) + m * e.ld_pre + n;
    l.a = *reinterpret_cast<const lt_u32x4*>(pre);
    if (e.gated) l.b = *reinterpret_cast<const lt_u32x4*>(pre + e.inter);
  } else if constexpr (KIND == EPI_OUT) {
    if (e.x) {
      const TX* x = reinterpret_cast<const TX*>(e.x) + m * e.ldy + n;
      l.a = *reinterpret_cast<const lt_u32x4*>(x);
      if constexpr (sizeof(TX) == 4) l.b = *reinterpret_cast<const lt_u32x4*>(x + 4);
    }
  }
  return l;
}

__device__ __forceinline__ void unpack_bf16x8(const lt_u32x4& raw, float (&v)[8]) {
  union { lt_u32x4 u; bf16 h[8]; } t;
  t.u = raw;
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = (float)t.h[i];
}

// cs: running column sums of the 8 gate-side (and, gated, 8 linear-side at cs + 8) dpre values this lane has written
__device__ __forceinline__ void epi_act_bwd8_loaded(const EpiParams& e, int64_t m, int64_t n, const float (&dh)[8],
                                                    const EpiLoad& l, float (&cs)[16]) {
  bf16* dpre = reinterpret_cast<bf16*>(e.dpre) + m * e.ld_pre + n;
  float pg[8], a[8], da[8], o[8];
  unpack_bf16x8(l.a, pg);
#pragma unroll
  for (int i = 0; i < 8; i++) act_eval<false>(e.act, pg[i], a[i], da[i]);
  if (e.gated) {
    float pl[8];
    unpack_bf16x8(l.b, pl);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * pl[i] * da[i];
    store8(dpre, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[i] += (float)(bf16)o[i];
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * a[i];
    store8(dpre + e.inter, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[8 + i] += (float)(bf16)o[i];
#pragma unroll
    for (int i = 0; i < 8; i++) a[i] *= pl[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * da[i];
    store8(dpre, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[i] += (float)(bf16)o[i];
  }
  if (e.hid) store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, a);
}

// Straight-line epilogue bodies for the usual cases (whole tile in range, bias present, no dropout): the run-time choices of
// the general functions above are made once per tile by the caller, not once per row; bias values of a lane's 8 columns
// are loaded once per tile and passed in.
// forward activation with the tanh GELU fixed (bias already in the accumulators)
template <bool GATED>
__device__ __forceinline__ void epi_act_fwd8_gelu(const EpiParams& e, int64_t m, int64_t n, float (&vg)[8], float (&vl)[8]) {
  float h[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    vg[i] = to_f32((bf16)vg[i]);  // the activation sees the stored (rounded) pre-activation, as backward will
    h[i] = act_value<false>(LT_ACT_GELU_FUSED, vg[i]);
    if constexpr (GATED) {
      vl[i] = to_f32((bf16)vl[i]);
      h[i] *= vl[i];
    }
  }
  bf16* pre = reinterpret_cast<bf16*>(e.pre) + m * e.ld_pre + n;
  store8(pre, vg);
  if constexpr (GATED) store8(pre + e.inter, vl);
  store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, h);
}

template <typename TO> __device__ __forceinline__ void epi_store8_plain(const EpiParams& e, int64_t m, int64_t n, const float (&v)[8]) {
  store8(reinterpret_cast<TO*>(e.out) + m * e.ldo + n, v);
}

// y = acc + x, residual read ahead (no dropout; the bias is in the accumulators already)
template <typename TX> __device__ __forceinline__ EpiLoad epi_load_x8(const EpiParams& e, int64_t m, int64_t n) {
  EpiLoad l;
  const TX* x = reinterpret_cast<const TX*>(e.x) + m * e.ldy + n;
  l.a = *reinterpret_cast<const lt_u32x4*>(x);
  if constexpr (sizeof(TX) == 4) l.b = *reinterpret_cast<const lt_u32x4*>(x + 4);
  else l.b = l.a;
  return l;
}

// DROPOUT: Philox keep-mask of the 8 elements applied before the residual is added
template <typename TX, bool DROPOUT = false>
__device__ __forceinline__ void epi_out8_residual(const EpiParams& e, int64_t m, int64_t n, float (&v)[8], const EpiLoad& l) {
  if constexpr (DROPOUT) {
    const int64_t idx = m * e.ldy + n;
    bool k0[4], k1[4];
    dropout_keep4(e.drop, idx, k0);
    dropout_keep4(e.drop, idx + 4, k1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[i] = k0[i] ? v[i] * e.drop.scale : 0.f;
      v[i + 4] = k1[i] ? v[i + 4] * e.drop.scale : 0.f;
    }
  }
  float r[8];
  if constexpr (sizeof(TX) == 4) {
    union { lt_u32x4 u[2]; float f[8]; } t;
    t.u[0] = l.a;
    t.u[1] = l.b;
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = t.f[i];
  } else {
    unpack_bf16x8(l.a, r);
  }
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] += r[i];
  store8(reinterpret_cast<TX*>(e.y) + m * e.ldy + n, v);
}

// EPI_ACT_BWD without run-time choices -- tanh-approximated GELU, gating fixed at compile time, h always written, rows known to
// be in range: straight-line code, so the compiler can count exactly which of the reads in flight a row waits for
template <bool GATED> __device__ __forceinline__ EpiLoad epi_load_pre8(const EpiParams& e, int64_t m, int64_t n) {
  EpiLoad l;
  const bf16* pre = reinterpret_cast<const bf16*>(e.pre) + m * e.ld_pre + n;
  l.a = *reinterpret_cast<const lt_u32x4*>(pre);
  if constexpr (GATED) l.b = *reinterpret_cast<const lt_u32x4*>(pre + e.inter);
  else l.b = l.a;
  return l;
}

template <bool GATED>
__device__ __forceinline__ void epi_act_bwd8_gelu(const EpiParams& e, int64_t m, int64_t n, const float (&dh)[8],
                                                  const EpiLoad& l, float (&cs)[16]) {
  bf16* dpre = reinterpret_cast<bf16*>(e.dpre) + m * e.ld_pre + n;
  float pg[8], a[8], da[8], o[8];
  unpack_bf16x8(l.a, pg);
#pragma unroll
  for (int i = 0; i < 8; i++) act_eval<false>(LT_ACT_GELU_FUSED, pg[i], a[i], da[i]);
  if constexpr (GATED) {
    float pl[8];
    unpack_bf16x8(l.b, pl);
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * pl[i] * da[i];
    store8(dpre, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[i] += (float)(bf16)o[i];
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * a[i];
    store8(dpre + e.inter, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[8 + i] += (float)(bf16)o[i];
#pragma unroll
    for (int i = 0; i < 8; i++) a[i] *= pl[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++) o[i] = dh[i] * da[i];
    store8(dpre, o);
#pragma unroll
    for (int i = 0; i < 8; i++) cs[i] += (float)(bf16)o[i];
  }
  store8(reinterpret_cast<bf16*>(e.hid) + m * e.ld_hid + n, a);
}

template <typename TX>
__device__ __forceinline__ void epi_out8_loaded(const EpiParams& e, int64_t m, int64_t n, float (&v)[8], const EpiLoad& l) {
  add_bias8(e.bias, n, v);
  const int64_t idx = m * e.ldy + n;
  if (e.drop.p > 0.f) {
    bool k0[4], k1[4];
    dropout_keep4(e.drop, idx, k0);
    dropout_keep4(e.drop, idx + 4, k1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[i] = k0[i] ? v[i] * e.drop.scale : 0.f;
      v[i + 4] = k1[i] ? v[i + 4] * e.drop.scale : 0.f;
    }
  }
  if (e.x) {
    float r[8];
    if constexpr (sizeof(TX) == 4) {
      union { lt_u32x4 u[2]; float f[8]; } t;
      t.u[0] = l.a;
      t.u[1] = l.b;
#pragma unroll
      for (int i = 0; i < 8; i++) r[i] = t.f[i];
    } else {
      unpack_bf16x8(l.a, r);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] += r[i];
  }
  store8(reinterpret_cast<TX*>(e.y) + idx, v);
}

// ---------------------------------------------------------------------------------------------------------------------
// launchers (defined in gemm_generic.hip / gemm_mfma_bf16.hip)
// ---------------------------------------------------------------------------------------------------------------------
// any shape, fp32 or bf16 operands (dtype), fp32 MFMA arithmetic.  io_dtype: dtype of x / y for EPI_OUT.
int lt_launch_gemm_generic(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream);
// true when the tiled bf16 kernel handles this problem (operand layouts, alignment, tile divisibility)
bool lt_gemm_mfma_supported(const GemmProblem& p, int kind);
int lt_launch_gemm_mfma(const GemmProblem& p, int kind, int io_dtype, hipStream_t stream);
// algorithmic flops of a dense problem: 2 * M * N * (K0 + K1)
double lt_gemm_flops(const GemmProblem& p, int kind);
// block-sparse walk: matrix-core kernel for 64 x 64 bf16 blocks, else the any-shape kernel
// whether a block-sparse forward problem (plain store or non-gated activation epilogue) runs as a dense product over
// gathered k-blocks: its output blocks come in aligned runs of 4 or more that share one list of input blocks (sp.out_group)
bool lt_sparse_forward_grouped(const GemmProblem& p, int kind);
// whether a block-sparse weight-gradient problem (SPARSE_DW) runs as dense products per run of 4 output blocks (sp.out_group)
bool lt_sparse_dw_out_grouped(const GemmProblem& p);
// ... or per run of 4 input blocks (sp.in_group): 0 when not, else the number of slices its reduction over the tokens is
// best split into (1: no split).  With more than one slice the caller sets p.ksplit = slices, p.split_stride = elements of the
// weight gradient, and points epi.out at fp32 partial sums (lt_sparse_dw_split_workspace bytes) that it sums afterwards.
int lt_sparse_dw_in_grouped_slices(const GemmProblem& p);
size_t lt_sparse_dw_split_workspace(int64_t in_features, int blocks_per_in, int in_group, int64_t tokens);
// whether the bf16 matrix-core walk for 64 x 64 blocks takes this block-sparse problem with epilogue `kind`
bool lt_sparse_mfma_supported(const GemmProblem& p, int kind);
int lt_launch_gemm_sparse(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream);
// EPI_STORE problems with few output tiles and a long reduction (the low-rank factors of a generalized linear layer):
// 128 x 128 tiles, the reduction split over workgroups through `workspace` when that fills the chip better.  Falls back to
// lt_launch_gemm when the shape does not fit.
size_t lt_gemm_skinny_workspace(int64_t tokens, int64_t lowrank);
// partial sums of a split [M, N] result on 256 x 256 tiles (0 when the tiles alone fill the chip)
size_t lt_gemm_splitk_workspace(int64_t M, int64_t N, int64_t K);
// same for the any-shape kernel (fp32 path, shapes the tiled kernels do not take)
size_t lt_gemm_generic_splitk_workspace(int64_t M, int64_t N, int64_t K);
// rows per partial row of EpiParams::colsum when lt_launch_gemm / lt_launch_gemm_sparse sends this EPI_ACT_BWD problem to a
// kernel that fills it (128: copy-based dense kernel; 64: block-sparse walk on whole tiles with the tanh GELU); 0: it will not
int lt_gemm_colsum_rows(const GemmProblem& p, int dtype, int io_dtype);
// Column sums of partial rows that may wait: a caller that runs several passes with such a tail (the FFN backward: two bias
// gradients and the LayerNorm parameter gradients) hands the same queue to each of them and flushes it once, one launch
// for all sums instead of one each.  The partial rows must stay untouched until the flush.
struct ColReduceJob {
  const float* partial;
  float* out;
  int rows, cols;
  int64_t stride;
};
struct ColReduceQueue {
  ColReduceJob job[4];
  int n;
};
int lt_colreduce_flush(ColReduceQueue& queue, hipStream_t stream);
// out[c] = sum over `rows` partial rows of partial[r * stride + c] (now, or at the flush of `defer`)
int lt_colreduce(int rows, int64_t stride, int cols, const float* partial, float* out, hipStream_t stream,
                 ColReduceQueue* defer = nullptr);
int lt_launch_gemm_skinny(const GemmProblem& p, int dtype, int io_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t stream);
// EPI_OUT problems with few output tiles and a long reduction (the down-projection of a short batch): the reduction split
// over workgroups into fp32 partial sums in `workspace`, then one pass that sums them through the same epilogue.  Takes as
// many slices as the workspace holds; falls back to lt_launch_gemm when the shape does not fit or one slice is enough.
// lt_gemm_out_splitk_workspace: bytes worth having for an [M, N] result, at most cap_bytes (0: no split would be taken).
size_t lt_gemm_out_splitk_workspace(int64_t M, int64_t N, int64_t K, size_t cap_bytes);
int lt_launch_gemm_out(const GemmProblem& p, int dtype, int io_dtype, void* workspace, size_t workspace_bytes,
                       hipStream_t stream);
// out[i] = sum_s partial[s * stride + i] (+ bias[i % cols]) for i < count, cast to out_dtype
int lt_splitk_reduce(const float* partial, int slices, int64_t stride, int64_t count, int cols, const float* bias,
                     int out_dtype, void* out, hipStream_t stream);
// picks the tiled kernel when it applies and dtype is bf16, else the any-shape kernel
int lt_launch_gemm(const GemmProblem& p, int kind, int dtype, int io_dtype, hipStream_t stream);
