// C ABI of libleanffn and the host-side sequencing of the FFN forward / backward.
//
// Forward   LN(x) -> u | up-projection GEMM with the activation epilogue (stores the pre-activation P, the only large
//           tensor kept for backward, and the transient hidden h) | down-projection GEMM with bias + dropout + residual
//           in its epilogue.
// Backward  dropout replay on dy -> g | dh = g W2 with an epilogue that reads P and emits dP (both halves when gated) and
//           the re-materialised h | dW2 = g^T h | db1, LN(x) again -> u | dW1 = dP^T u | du = dP W1 | LayerNorm backward
//           with the residual gradient folded in.
// Low-rank terms ride along as a second k-segment of the same GEMM launches.  reference: lean_transformer/ffn.py:146-306,
// lean_transformer/blocksparse/linear.py:197-328.
#include <stdarg.h>

#include "lt_internal.h"

// ---------------------------------------------------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------------------------------------------------
static thread_local char g_error[1024] = "";

void lt_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* lt_last_error(void) { return g_error; }
extern "C" const char* lt_version(void) { return "libleanffn 0.1.0 (gfx950, 16-bit type " LT_HALF_NAME ")"; }

namespace {

// bump allocator over the caller's workspace; with a null base it only measures
struct Bump {
  char* base;
  size_t used = 0;
  explicit Bump(void* b) : base((char*)b) {}
  void* take(size_t bytes) {
    used = lt_align_up(used, 256);
    void* p = base ? base + used : nullptr;
    used += bytes;
    return p;
  }
};

int check_dtype(int d, const char* what) {
  LT_REQUIRE(d == LT_F32 || d == LT_BF16, LT_ERR_BAD_ARG, "%s: dtype code %d is not one of this library's (fp32 = %d, " LT_HALF_NAME " = %d)", what,
             d, (int)LT_F32, (int)LT_BF16);
  return LT_OK;
}

// which index tables a call reads: the forward walk takes forward_indices, both gradient walks take backward_indices
enum { NEED_FWD_TABLE = 1, NEED_BWD_TABLE = 2 };
// lt_linear::out_group / in_group: run length in the low 16 bits, blocks between the members of a run in the high 16 bits
inline int group_length(int32_t g) { return g & 0xffff; }
inline int group_stride(int32_t g) { return (g >> 16) & 0x7fff; }

int check_linear(const lt_linear& lin, const char* name, int tables = NEED_FWD_TABLE | NEED_BWD_TABLE) {
  LT_REQUIRE(lin.weight && lin.in_features > 0 && lin.out_features > 0, LT_ERR_BAD_ARG, "%s: weight / sizes missing", name);
  LT_REQUIRE(lin.lowrank >= 0 && ((lin.lowrank > 0) == (lin.lowrank_first != nullptr)) &&
                 ((lin.lowrank > 0) == (lin.lowrank_second != nullptr)),
             LT_ERR_BAD_ARG, "%s: lowrank=%d does not match the low-rank pointers", name, lin.lowrank);
  if (lin.block > 0) {
    LT_REQUIRE(!(tables & NEED_FWD_TABLE) || lin.forward_indices, LT_ERR_BAD_ARG, "%s: sparse weight without forward_indices", name);
    LT_REQUIRE(!(tables & NEED_BWD_TABLE) || lin.backward_indices, LT_ERR_BAD_ARG, "%s: sparse weight without backward_indices", name);
    LT_REQUIRE(lin.in_features % lin.block == 0 && lin.out_features % lin.block == 0, LT_ERR_BAD_ARG,
               "%s: features not divisible by block %d", name, lin.block);
    LT_REQUIRE(lin.blocks_per_in > 0 && lin.blocks_per_out > 0 &&
                   (int64_t)lin.blocks_per_in * (lin.in_features / lin.block) ==
                       (int64_t)lin.blocks_per_out * (lin.out_features / lin.block),
               LT_ERR_BAD_ARG, "%s: unbalanced layout (K=%d, A=%d)", name, lin.blocks_per_out, lin.blocks_per_in);
    const int out_blocks = lin.out_features / lin.block, in_blocks = lin.in_features / lin.block;
    const int og = group_length(lin.out_group), os = group_stride(lin.out_group);
    const int ig = group_length(lin.in_group), is = group_stride(lin.in_group);
    LT_REQUIRE(lin.out_group >= 0 && (og <= 1 || out_blocks % og == 0) && (os <= 1 || og * os == out_blocks), LT_ERR_BAD_ARG,
               "%s: out_group (runs of %d, %d apart) does not fit the %d output blocks", name, og, os > 1 ? os : 1, out_blocks);
    LT_REQUIRE(lin.in_group >= 0 && (ig <= 1 || in_blocks % ig == 0) && (is <= 1 || ig * is == in_blocks), LT_ERR_BAD_ARG,
               "%s: in_group (runs of %d, %d apart) does not fit the %d input blocks", name, ig, is > 1 ? is : 1, in_blocks);
  }
  return LT_OK;
}

namespace {
// flag[0] = 0 when output block ob's list differs from that of the first block of its aligned run of `group`, or its weight
// blocks do not follow that block's by ob % group (what lt_linear::out_group promises); untouched otherwise
// (runs `stride` blocks apart promise the same lists of input blocks only: first block of the run = ob % stride)
__global__ void check_out_group_kernel(const int32_t* __restrict__ forward_indices, int out_blocks, int per_out, int per_in,
                                       int group, int stride, int32_t* flag) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= out_blocks * per_out) return;
  const int ob = i / per_out, e = i % per_out, ob0 = stride > 1 ? ob % stride : ob - ob % group;
  const int mine = forward_indices[i], first = forward_indices[ob0 * per_out + e];
  if (mine / per_in != first / per_in || (stride <= 1 && mine != first + (ob - ob0))) flag[0] = 0;
}
// the same for lt_linear::in_group: input block ib's list of output blocks against that of the first block of its run
__global__ void check_in_group_kernel(const int64_t* __restrict__ backward_indices, int in_blocks, int per_in, int group,
                                      int stride, int32_t* flag) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= in_blocks * per_in) return;
  const int ib = i / per_in, e = i % per_in, ib0 = stride > 1 ? ib % stride : ib - ib % group;
  if (backward_indices[i] != backward_indices[ib0 * per_in + e]) flag[0] = 0;
}
__global__ void set_flag_kernel(int32_t* flag, int32_t value) { flag[0] = value; }
}  // namespace

extern "C" int lt_linear_check_out_group(const lt_linear* lin, int32_t* flag, void* stream_) {
  LT_REQUIRE(lin && flag, LT_ERR_BAD_ARG, "check out_group: null argument");
  LT_TRY(check_linear(*lin, "check out_group", NEED_FWD_TABLE));
  hipStream_t stream = (hipStream_t)stream_;
  hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, stream, flag, 1);
  LT_LAUNCH_CHECK();
  if (lin->block > 0 && group_length(lin->out_group) > 1) {
    const int out_blocks = lin->out_features / lin->block, entries = out_blocks * lin->blocks_per_out;
    hipLaunchKernelGGL(check_out_group_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0, stream,
                       lin->forward_indices, out_blocks, lin->blocks_per_out, lin->blocks_per_in, group_length(lin->out_group),
                       group_stride(lin->out_group), flag);
    LT_LAUNCH_CHECK();
  }
  return LT_OK;
}

extern "C" int lt_linear_check_in_group(const lt_linear* lin, int32_t* flag, void* stream_) {
  LT_REQUIRE(lin && flag, LT_ERR_BAD_ARG, "check in_group: null argument");
  LT_TRY(check_linear(*lin, "check in_group", NEED_BWD_TABLE));
  hipStream_t stream = (hipStream_t)stream_;
  hipLaunchKernelGGL(set_flag_kernel, dim3(1), dim3(1), 0, stream, flag, 1);
  LT_LAUNCH_CHECK();
  if (lin->block > 0 && group_length(lin->in_group) > 1) {
    const int in_blocks = lin->in_features / lin->block, entries = in_blocks * lin->blocks_per_in;
    hipLaunchKernelGGL(check_in_group_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0, stream,
                       lin->backward_indices, in_blocks, lin->blocks_per_in, group_length(lin->in_group),
                       group_stride(lin->in_group), flag);
    LT_LAUNCH_CHECK();
  }
  return LT_OK;
}

// Walk order of a block-sparse index list of `length` entries on the side with `many` blocks, seen from the side with `few`:
// a stretched butterfly repeats every block of the square pattern many / few times in a row, so the lists are made of runs of
// that many consecutive blocks (SparseWalk::walk_run; 0 when the shape suggests none).  Only an order: any layout computes right.
int walk_run_for(int many, int few, int length) {
  if (few <= 0 || many <= few || many % few != 0) return 0;
  const int g = many / few;
  return (g > 1 && length % g == 0) ? g : 0;
}

GemmOperand operand(const void* p, int64_t ld, bool kmajor) {
  GemmOperand o;
  o.ptr = p; o.ld = ld; o.kmajor = kmajor ? 1 : 0;
  return o;
}

EpiParams epi_store_params(void* out, int64_t ldo, int out_dtype, const float* bias) {
  EpiParams e;
  memset(&e, 0, sizeof(e));
  e.out = out; e.ldo = ldo; e.out_dtype = out_dtype; e.bias = bias;
  return e;
}

GemmProblem blank_problem() {
  GemmProblem p;
  memset(&p, 0, sizeof(p));
  p.nseg = 1;
  return p;
}

// y-side of one generalized linear layer: [lowrank_hid = x L1^T], then x W^T (+ lowrank_hid L2^T) through epilogue `kind`.
// For a gated EPI_ACT_FWD the epilogue pairs output column n with n + out_features / 2.
int linear_forward_impl(const lt_linear& lin, int64_t T, int dtype, const void* x, int kind, const EpiParams& epi,
                        void* lowrank_hid, int io_dtype, hipStream_t stream, void* skinny_ws = nullptr,
                        size_t skinny_bytes = 0) {
  const int64_t in = lin.in_features, out = lin.out_features, r = lin.lowrank;
  if (r > 0) {
    LT_REQUIRE(lowrank_hid, LT_ERR_BAD_ARG, "linear forward: lowrank_hid buffer missing");
    GemmProblem q = blank_problem();
    q.M = T; q.N = r; q.K[0] = in;
    q.A[0] = operand(x, in, true);
    q.B[0] = operand(lin.lowrank_first, in, true);
    q.epi = epi_store_params(lowrank_hid, r, dtype, nullptr);
    LT_TRY(lt_launch_gemm_skinny(q, dtype, io_dtype, skinny_ws, skinny_bytes, stream));
  }
  GemmProblem p = blank_problem();
  const bool gated = kind == EPI_ACT_FWD && epi.gated;
  p.M = T; p.N = gated ? out / 2 : out;
  p.epi = epi;
  if (r > 0) {
    p.nseg = 2; p.K[1] = r;
    p.A[1] = operand(lowrank_hid, r, true);
    p.B[1] = operand(lin.lowrank_second, r, true);
  }
  if (lin.block == 0) {
    p.K[0] = in;
    p.A[0] = operand(x, in, true);
    p.B[0] = operand(lin.weight, in, true);
    if (kind == EPI_OUT && r == 0) return lt_launch_gemm_out(p, dtype, io_dtype, skinny_ws, skinny_bytes, stream);
    return lt_launch_gemm(p, kind, dtype, io_dtype, stream);
  }
  p.K[0] = lin.block;
  p.sp.mode = SPARSE_FWD; p.sp.block = lin.block; p.sp.blocks_per_out = lin.blocks_per_out;
  p.sp.blocks_per_in = lin.blocks_per_in; p.sp.forward_indices = lin.forward_indices;
  p.sp.backward_indices = lin.backward_indices; p.sp.act = x; p.sp.ld_act = in; p.sp.weight = lin.weight;
  p.sp.out_group = group_length(lin.out_group); p.sp.out_stride = group_stride(lin.out_group);
  // (a tiled layout, known by its strided runs, lists the blocks of one tile of the square pattern together: as listed is
  // the order in which the groups that share an activation block read it close together)
  p.sp.walk_run = group_stride(lin.in_group) > 1
                      ? 0 : walk_run_for(lin.in_features / lin.block, lin.out_features / lin.block, lin.blocks_per_out);
  bool two_passes = gated && !(dtype == LT_BF16 && lt_sparse_mfma_supported(p, kind));
  if (gated && !two_passes) {
    // Gate and linear output blocks have index lists of their own; the bf16 walk for 64 x 64 blocks pairs them inside one
    // workgroup.  Where the layout lets the product run on 256 x 256 tiles instead (runs of output blocks with a shared
    // list), that and a separate activation pass are faster than the paired walk.
    GemmProblem s = p;
    s.N = out;
    s.epi = epi_store_params(epi.pre, epi.ld_pre, dtype, epi.bias);
    two_passes = lt_sparse_forward_grouped(s, EPI_STORE);
  }
  if (two_passes) {  // store the pre-activation, then the activation as a pass of its own
    p.N = out;
    p.epi = epi_store_params(epi.pre, epi.ld_pre, dtype, epi.bias);
    LT_TRY(lt_launch_gemm_sparse(p, EPI_STORE, dtype, io_dtype, stream));
    return lt_act_forward(T, epi.inter, 1, epi.act, dtype, epi.pre, epi.hid, stream);
  }
  return lt_launch_gemm_sparse(p, kind, dtype, io_dtype, stream);
}

struct LinearBwdScratch {
  void* g_hid;     // [T, r] dtype
  void* colsum;    // lt_colsum_workspace(T, out)
  size_t colsum_bytes;
  void* skinny;    // split-k partial sums of the low-rank GEMMs
  size_t skinny_bytes;
};

void plan_linear_backward(const lt_linear& lin, int64_t T, int dtype, Bump& ws, LinearBwdScratch& s) {
  s.g_hid = lin.lowrank > 0 ? ws.take((size_t)T * lin.lowrank * lt_dtype_size(dtype)) : nullptr;
  s.colsum_bytes = lt_colsum_workspace(T, lin.out_features);
  s.colsum = ws.take(s.colsum_bytes);
  s.skinny_bytes = lin.lowrank > 0 ? lt_gemm_skinny_workspace(T, lin.lowrank) : 0;
  if (lin.block == 0) {  // dW (and dx) of a small dense layer: the reduction is split across workgroups
    s.skinny_bytes = std::max(s.skinny_bytes, lt_gemm_splitk_workspace(lin.out_features, lin.in_features, T));
    s.skinny_bytes = std::max(s.skinny_bytes, lt_gemm_generic_splitk_workspace(lin.out_features, lin.in_features, T));
    if (lin.lowrank == 0)
      s.skinny_bytes = std::max(s.skinny_bytes, lt_gemm_generic_splitk_workspace(T, lin.in_features, lin.out_features));
  }
  if (lin.block == 64 && dtype == LT_BF16)
    s.skinny_bytes = std::max(s.skinny_bytes,
                              lt_sparse_dw_split_workspace(lin.in_features, lin.blocks_per_in, group_length(lin.in_group), T));
  s.skinny = s.skinny_bytes ? ws.take(s.skinny_bytes) : nullptr;
}

// gradient side of one generalized linear layer.  The input-gradient GEMM runs FIRST, through epilogue `kind_dx`
// (EPI_ACT_BWD for the down-projection, whose epilogue also re-materialises this layer's own input `x_act`), then the
// parameter gradients, which may therefore read x_act.  Pass kind_dx < 0 to skip the input gradient.
// act_colsum / act_colsum_rows: with an EPI_ACT_BWD input-gradient epilogue, room for the partial column sums of the dpre it
// writes (one row of epi_dx.ld_pre floats per 64 tokens); *act_colsum_rows = tokens per partial row the kernel that ran
// filled (0: it did not)
int linear_backward_impl(const lt_linear& lin, int64_t T, int dtype, const void* x_act, const void* dy,
                         const void* lowrank_hid, int kind_dx, const EpiParams& epi_dx, const lt_linear_grads& grads,
                         const LinearBwdScratch& s, int io_dtype, hipStream_t stream, float* act_colsum = nullptr,
                         int* act_colsum_rows = nullptr) {
  const int64_t in = lin.in_features, out = lin.out_features, r = lin.lowrank;
  const bool need_dx = kind_dx >= 0;
  if (r > 0 && (need_dx || grads.lowrank_first)) {  // g_hid = dy L2  [T, r]
    GemmProblem q = blank_problem();
    q.M = T; q.N = r; q.K[0] = out;
    q.A[0] = operand(dy, out, true);
    q.B[0] = operand(lin.lowrank_second, r, false);
    q.epi = epi_store_params(s.g_hid, r, dtype, nullptr);
    LT_TRY(lt_launch_gemm_skinny(q, dtype, io_dtype, s.skinny, s.skinny_bytes, stream));
  }
  if (need_dx) {  // dx = dy W (+ g_hid L1)
    GemmProblem p = blank_problem();
    p.M = T; p.N = in;
    p.epi = epi_dx;
    if (r > 0) {
      p.nseg = 2; p.K[1] = r;
      p.A[1] = operand(s.g_hid, r, true);
      p.B[1] = operand(lin.lowrank_first, in, false);
    }
    if (lin.block == 0) {
      p.K[0] = out;
      p.A[0] = operand(dy, out, true);
      p.B[0] = operand(lin.weight, in, false);
      if (kind_dx == EPI_ACT_BWD && act_colsum && (*act_colsum_rows = lt_gemm_colsum_rows(p, dtype, io_dtype)) > 0)
        p.epi.colsum = act_colsum;
      if (kind_dx == EPI_STORE && r == 0) LT_TRY(lt_launch_gemm_skinny(p, dtype, io_dtype, s.skinny, s.skinny_bytes, stream));
      else LT_TRY(lt_launch_gemm(p, kind_dx, dtype, io_dtype, stream));
    } else {
      p.K[0] = lin.block;
      p.sp.mode = SPARSE_DX; p.sp.block = lin.block; p.sp.blocks_per_out = lin.blocks_per_out;
      p.sp.blocks_per_in = lin.blocks_per_in; p.sp.forward_indices = lin.forward_indices;
      p.sp.backward_indices = lin.backward_indices; p.sp.act = dy; p.sp.ld_act = out; p.sp.weight = lin.weight;
      p.sp.walk_run = group_stride(lin.out_group) > 1
                          ? 0 : walk_run_for(lin.out_features / lin.block, lin.in_features / lin.block, lin.blocks_per_in);
      if (kind_dx == EPI_ACT_BWD && act_colsum && (*act_colsum_rows = lt_gemm_colsum_rows(p, dtype, io_dtype)) > 0)
        p.epi.colsum = act_colsum;
      LT_TRY(lt_launch_gemm_sparse(p, kind_dx, dtype, io_dtype, stream));
    }
  }
  if (grads.bias) LT_TRY(lt_colsum(T, (int)out, out, dtype, dy, grads.bias, s.colsum, s.colsum_bytes, stream));
  if (grads.weight) {
    GemmProblem p = blank_problem();
    if (lin.block == 0) {  // dW[out, in] = dy^T x
      p.M = out; p.N = in; p.K[0] = T;
      p.A[0] = operand(dy, out, false);
      p.B[0] = operand(x_act, in, false);
      p.epi = epi_store_params(grads.weight, in, dtype, nullptr);
      LT_TRY(lt_launch_gemm_skinny(p, dtype, io_dtype, s.skinny, s.skinny_bytes, stream));
    } else {
      p.M = lin.block; p.N = in; p.K[0] = T;
      p.sp.mode = SPARSE_DW; p.sp.block = lin.block; p.sp.blocks_per_out = lin.blocks_per_out;
      p.sp.blocks_per_in = lin.blocks_per_in; p.sp.forward_indices = lin.forward_indices;
      p.sp.backward_indices = lin.backward_indices; p.sp.act = dy; p.sp.ld_act = out; p.sp.act2 = x_act;
      p.sp.ld_act2 = in; p.sp.tokens = T;
      // (the grouped kernel reads the list from the forward table)
      p.sp.out_group = lin.forward_indices ? group_length(lin.out_group) : 0; p.sp.out_stride = group_stride(lin.out_group);
      p.sp.in_group = group_length(lin.in_group); p.sp.in_stride = group_stride(lin.in_group);
      p.epi = epi_store_params(grads.weight, lin.block, dtype, nullptr);
      const int slices = dtype == LT_BF16 ? lt_sparse_dw_in_grouped_slices(p) : 0;
      const size_t elements = (size_t)(in / lin.block) * lin.blocks_per_in * lin.block * lin.block;
      if (slices > 1 && s.skinny && s.skinny_bytes >= (size_t)slices * elements * sizeof(float)) {
        // the reduction over the tokens split over workgroups: fp32 partial gradients, summed into the parameter's dtype
        p.ksplit = slices;
        p.split_stride = (int64_t)elements;
        p.epi.out = s.skinny;
        p.epi.out_dtype = LT_F32;
        LT_TRY(lt_launch_gemm_sparse(p, EPI_STORE, dtype, io_dtype, stream));
        LT_TRY(lt_splitk_reduce((const float*)s.skinny, slices, (int64_t)elements, (int64_t)elements, lin.block, nullptr, dtype,
                                grads.weight, stream));
      } else {
        if (slices > 1) p.sp.in_group = 0;  // no room for the partial sums: the walk
        LT_TRY(lt_launch_gemm_sparse(p, EPI_STORE, dtype, io_dtype, stream));
      }
    }
  }
  if (r > 0 && grads.lowrank_second) {  // dL2[out, r] = dy^T hid
    LT_REQUIRE(lowrank_hid, LT_ERR_BAD_ARG, "linear backward: lowrank_hid missing");
    GemmProblem q = blank_problem();
    q.M = out; q.N = r; q.K[0] = T;
    q.A[0] = operand(dy, out, false);
    q.B[0] = operand(lowrank_hid, r, false);
    q.epi = epi_store_params(grads.lowrank_second, r, dtype, nullptr);
    LT_TRY(lt_launch_gemm_skinny(q, dtype, io_dtype, s.skinny, s.skinny_bytes, stream));
  }
  if (r > 0 && grads.lowrank_first) {  // dL1[r, in] = g_hid^T x
    GemmProblem q = blank_problem();
    q.M = r; q.N = in; q.K[0] = T;
    q.A[0] = operand(s.g_hid, r, false);
    q.B[0] = operand(x_act, in, false);
    q.epi = epi_store_params(grads.lowrank_first, in, dtype, nullptr);
    LT_TRY(lt_launch_gemm_skinny(q, dtype, io_dtype, s.skinny, s.skinny_bytes, stream));
  }
  return LT_OK;
}

int check_ffn_desc(const lt_ffn_desc* d) {
  LT_REQUIRE(d, LT_ERR_BAD_ARG, "ffn: null descriptor");
  LT_REQUIRE(d->tokens > 0 && d->hidden > 0 && d->intermediate > 0, LT_ERR_BAD_ARG, "ffn: bad sizes T=%lld H=%d I=%d",
             (long long)d->tokens, d->hidden, d->intermediate);
  LT_TRY(check_dtype(d->io_dtype, "ffn io_dtype"));
  LT_TRY(check_dtype(d->compute_dtype, "ffn compute_dtype"));
  LT_REQUIRE(d->act >= 0 && d->act < LT_ACT_COUNT, LT_ERR_UNSUPPORTED, "ffn: unknown activation %d", d->act);
  LT_REQUIRE(d->ln_weight && d->ln_bias, LT_ERR_BAD_ARG, "ffn: LayerNorm parameters missing");
  LT_REQUIRE((d->post_ln_weight == nullptr) == (d->post_ln_bias == nullptr), LT_ERR_BAD_ARG, "ffn: post-LN needs weight and bias");
  LT_REQUIRE(d->dropout_p >= 0.f && d->dropout_p < 1.f, LT_ERR_BAD_ARG, "ffn: dropout %f outside [0, 1)", d->dropout_p);
  LT_TRY(check_linear(d->i2h, "ffn i2h"));
  LT_TRY(check_linear(d->h2o, "ffn h2o"));
  const int n1 = d->gated ? 2 * d->intermediate : d->intermediate;
  LT_REQUIRE(d->i2h.in_features == d->hidden && d->i2h.out_features == n1, LT_ERR_BAD_ARG,
             "ffn: i2h is %d -> %d, expected %d -> %d", d->i2h.in_features, d->i2h.out_features, d->hidden, n1);
  LT_REQUIRE(d->h2o.in_features == d->intermediate && d->h2o.out_features == d->hidden, LT_ERR_BAD_ARG,
             "ffn: h2o is %d -> %d, expected %d -> %d", d->h2o.in_features, d->h2o.out_features, d->intermediate, d->hidden);
  return LT_OK;
}

struct FwdScratch {
  void* u;       // [T, H] compute dtype: LayerNorm output
  void* hid;     // [T, I] compute dtype: activation output
  void* skinny;  // split-k partial sums of the low-rank GEMMs
  size_t skinny_bytes;
};

void plan_forward(const lt_ffn_desc& d, Bump& ws, FwdScratch& s) {
  const size_t e = lt_dtype_size(d.compute_dtype);
  s.u = ws.take((size_t)d.tokens * d.hidden * e);
  s.hid = ws.take((size_t)d.tokens * d.intermediate * e);
  const int r = d.i2h.lowrank > d.h2o.lowrank ? d.i2h.lowrank : d.h2o.lowrank;
  s.skinny_bytes = r > 0 ? lt_gemm_skinny_workspace(d.tokens, r) : 0;
  // dense down-projection of a short batch: room to split its reduction, no more than the saved pre-activation takes
  if (d.h2o.block == 0 && d.h2o.lowrank == 0 && !d.post_ln_weight) {
    const size_t cap = (size_t)d.tokens * (d.gated ? 2 : 1) * d.intermediate * e;
    s.skinny_bytes = std::max(s.skinny_bytes, lt_gemm_out_splitk_workspace(d.tokens, d.hidden, d.intermediate, cap));
  }
  s.skinny = s.skinny_bytes ? ws.take(s.skinny_bytes) : nullptr;
}

struct BwdScratch {
  void* g;           // [T, H] compute dtype: gradient entering the down-projection
  void* g_post;      // [T, H] compute dtype: post-LN only
  float* post_stats; // [T, 2]: post-LN only
  void* hid;         // [T, I]
  void* dpre;        // [T, N1]
  void* u;           // [T, H]
  void* du;          // [T, H] compute dtype (as the reference's autocast matmul leaves it)
  void* ln_ws;
  size_t ln_ws_bytes;
  float* act_colsum;  // [ceil(T / 64), N1]: partial column sums of dpre from the epilogue that writes it
  LinearBwdScratch h2o, i2h;
};

void plan_backward(const lt_ffn_desc& d, Bump& ws, BwdScratch& s) {
  const size_t e = lt_dtype_size(d.compute_dtype);
  const int64_t T = d.tokens;
  const int64_t n1 = d.gated ? 2 * (int64_t)d.intermediate : d.intermediate;
  s.g = ws.take((size_t)T * d.hidden * e);
  s.g_post = d.post_ln_weight ? ws.take((size_t)T * d.hidden * e) : nullptr;
  s.post_stats = d.post_ln_weight ? (float*)ws.take((size_t)T * 2 * sizeof(float)) : nullptr;
  s.hid = ws.take((size_t)T * d.intermediate * e);
  s.dpre = ws.take((size_t)T * n1 * e);
  s.u = ws.take((size_t)T * d.hidden * e);
  s.du = ws.take((size_t)T * d.hidden * e);
  s.ln_ws_bytes = lt_ln_backward_workspace(T, d.hidden);
  s.ln_ws = ws.take(s.ln_ws_bytes);
  s.act_colsum = (float*)ws.take((size_t)((T + 63) / 64) * n1 * sizeof(float));
  plan_linear_backward(d.h2o, T, d.compute_dtype, ws, s.h2o);
  plan_linear_backward(d.i2h, T, d.compute_dtype, ws, s.i2h);
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------------------
// whole FFN block
// ---------------------------------------------------------------------------------------------------------------------
extern "C" size_t lt_ffn_forward_workspace_bytes(const lt_ffn_desc* desc) {
  if (check_ffn_desc(desc) != LT_OK) return 0;
  Bump ws(nullptr);
  FwdScratch s;
  plan_forward(*desc, ws, s);
  return lt_align_up(ws.used, 256);
}

extern "C" size_t lt_ffn_backward_workspace_bytes(const lt_ffn_desc* desc) {
  if (check_ffn_desc(desc) != LT_OK) return 0;
  Bump ws(nullptr);
  BwdScratch s;
  plan_backward(*desc, ws, s);
  return lt_align_up(ws.used, 256);
}

extern "C" int lt_ffn_forward(const lt_ffn_desc* desc, const void* x, void* y, const lt_ffn_saved* saved, void* workspace,
                              size_t workspace_bytes, void* stream_) {
  LT_TRY(check_ffn_desc(desc));
  const lt_ffn_desc& d = *desc;
  hipStream_t stream = (hipStream_t)stream_;
  LT_REQUIRE(x && y && saved && saved->pre_activation && saved->ln_stats, LT_ERR_BAD_ARG, "ffn forward: null tensor");
  LT_REQUIRE(!d.post_ln_weight || saved->post_ln_input, LT_ERR_BAD_ARG, "ffn forward: post_ln_input buffer missing");
  LT_REQUIRE(workspace && lt_aligned(workspace, 256) && workspace_bytes >= lt_ffn_forward_workspace_bytes(desc),
             LT_ERR_WORKSPACE, "ffn forward: needs a 256-byte aligned workspace of %zu bytes",
             lt_ffn_forward_workspace_bytes(desc));
  Bump ws(workspace);
  FwdScratch s;
  plan_forward(d, ws, s);
  const int64_t T = d.tokens, H = d.hidden, I = d.intermediate, N1 = d.gated ? 2 * I : I;
  const int cdt = d.compute_dtype, io = d.io_dtype;
  const DropoutParams drop = make_dropout(d.dropout_p, d.dropout_seed, d.dropout_offset);

  LT_TRY(lt_ln_forward(T, (int)H, d.ln_eps, io, x, d.ln_weight, d.ln_bias, cdt, s.u, saved->ln_stats, io, nullptr,
                       nullptr, false, stream));

  // up-projection + activation
  {
    EpiParams e;
    memset(&e, 0, sizeof(e));
    e.bias = d.i2h.bias; e.pre = saved->pre_activation; e.ld_pre = N1; e.hid = s.hid; e.ld_hid = I;
    e.gated = d.gated; e.act = d.act; e.inter = I;
    LT_TRY(linear_forward_impl(d.i2h, T, cdt, s.u, EPI_ACT_FWD, e, saved->i2h_lowrank_hid, io, stream, s.skinny, s.skinny_bytes));
  }

  // down-projection (+ post-LN) + dropout + residual
  if (d.post_ln_weight) {
    EpiParams e = epi_store_params(saved->post_ln_input, H, cdt, d.h2o.bias);
    LT_TRY(linear_forward_impl(d.h2o, T, cdt, s.hid, EPI_STORE, e, saved->h2o_lowrank_hid, io, stream, s.skinny, s.skinny_bytes));
    LT_TRY(lt_ln_forward(T, (int)H, d.ln_eps, cdt, saved->post_ln_input, d.post_ln_weight, d.post_ln_bias, io, y, nullptr,
                         io, d.residual ? x : nullptr, &drop, true, stream));
  } else {
    EpiParams e;
    memset(&e, 0, sizeof(e));
    e.bias = d.h2o.bias; e.x = d.residual ? x : nullptr; e.y = y; e.ldy = H; e.drop = drop;
    LT_TRY(linear_forward_impl(d.h2o, T, cdt, s.hid, EPI_OUT, e, saved->h2o_lowrank_hid, io, stream, s.skinny, s.skinny_bytes));
  }
  return LT_OK;
}

extern "C" int lt_ffn_backward(const lt_ffn_desc* desc, const void* x, const void* dy, const lt_ffn_saved* saved,
                               const lt_ffn_grads* grads, void* workspace, size_t workspace_bytes, void* stream_) {
  LT_TRY(check_ffn_desc(desc));
  const lt_ffn_desc& d = *desc;
  hipStream_t stream = (hipStream_t)stream_;
  LT_REQUIRE(x && dy && saved && grads && saved->pre_activation && saved->ln_stats, LT_ERR_BAD_ARG, "ffn backward: null tensor");
  LT_REQUIRE(!d.post_ln_weight || saved->post_ln_input, LT_ERR_BAD_ARG, "ffn backward: post_ln_input missing");
  LT_REQUIRE((grads->ln_weight == nullptr) == (grads->ln_bias == nullptr), LT_ERR_BAD_ARG, "ffn backward: pass both LayerNorm gradients or neither");
  LT_REQUIRE((grads->post_ln_weight == nullptr) == (grads->post_ln_bias == nullptr), LT_ERR_BAD_ARG, "ffn backward: pass both post-LN gradients or neither");
  LT_REQUIRE(workspace && lt_aligned(workspace, 256) && workspace_bytes >= lt_ffn_backward_workspace_bytes(desc),
             LT_ERR_WORKSPACE, "ffn backward: needs a 256-byte aligned workspace of %zu bytes",
             lt_ffn_backward_workspace_bytes(desc));
  Bump ws(workspace);
  BwdScratch s;
  plan_backward(d, ws, s);
  const int64_t T = d.tokens, H = d.hidden, I = d.intermediate, N1 = d.gated ? 2 * I : I;
  const int cdt = d.compute_dtype, io = d.io_dtype;
  const DropoutParams drop = make_dropout(d.dropout_p, d.dropout_seed, d.dropout_offset);

  // the small column sums at the end of three passes (two bias gradients, the LayerNorm parameter gradients) wait for one
  // launch at the end of the step
  ColReduceQueue reduces;
  reduces.n = 0;
  // gradient entering the down-projection: dropout replayed on dy, then (optionally) back through the post-LN
  const void* g = s.g;
  lt_linear_grads h2o_grads = grads->h2o;
  if (d.dropout_p == 0.f && io == cdt) {
    g = dy;
  } else if (h2o_grads.bias && !d.post_ln_weight) {
    // the same pass also sums the columns of g: the down-projection's bias gradient
    LT_TRY(lt_dropout_cast_colsum(T, (int)H, io, dy, cdt, s.g, drop, (float*)h2o_grads.bias, s.h2o.colsum, s.h2o.colsum_bytes,
                                  stream, &reduces));
    h2o_grads.bias = nullptr;
  } else {
    LT_TRY(lt_dropout_cast(T * H, io, dy, cdt, s.g, drop, stream));
  }
  if (d.post_ln_weight) {
    LT_TRY(lt_ln_forward(T, (int)H, d.ln_eps, cdt, saved->post_ln_input, nullptr, nullptr, cdt, nullptr, s.post_stats, cdt,
                         nullptr, nullptr, false, stream));
    LT_TRY(lt_ln_backward(T, (int)H, cdt, saved->post_ln_input, s.post_stats, d.post_ln_weight, cdt, g, cdt, nullptr,
                          s.g_post, grads->post_ln_weight, grads->post_ln_bias, s.ln_ws, s.ln_ws_bytes, stream));
    g = s.g_post;
  }

  // down-projection backward; its input-gradient epilogue turns dh into dP and re-materialises h from P
  int bias_rows = 0;  // tokens per partial row of s.act_colsum when the dGeGLU epilogue summed the columns of dP
  {
    EpiParams e;
    memset(&e, 0, sizeof(e));
    e.pre = saved->pre_activation; e.ld_pre = N1; e.dpre = s.dpre; e.hid = s.hid; e.ld_hid = I;
    e.gated = d.gated; e.act = d.act; e.inter = I;
    LT_TRY(linear_backward_impl(d.h2o, T, cdt, s.hid, g, saved->h2o_lowrank_hid, EPI_ACT_BWD, e, h2o_grads, s.h2o, io,
                                stream, grads->i2h.bias ? s.act_colsum : nullptr, &bias_rows));
  }
  lt_linear_grads i2h_grads = grads->i2h;
  if (bias_rows > 0) {  // db1 = column sums of dP, already reduced to one row per bias_rows tokens
    LT_TRY(lt_colreduce((int)((T + bias_rows - 1) / bias_rows), N1, (int)N1, s.act_colsum, (float*)grads->i2h.bias, stream,
                        &reduces));
    i2h_grads.bias = nullptr;
  }

  // up-projection backward on the recomputed LayerNorm output; du in the compute dtype
  LT_TRY(lt_ln_forward(T, (int)H, d.ln_eps, io, x, d.ln_weight, d.ln_bias, cdt, s.u, nullptr, io, nullptr, nullptr, false,
                       stream));
  const bool need_du = grads->dx || grads->ln_weight;
  {
    EpiParams e = epi_store_params(s.du, H, cdt, nullptr);
    LT_TRY(linear_backward_impl(d.i2h, T, cdt, s.u, s.dpre, saved->i2h_lowrank_hid, need_du ? EPI_STORE : -1, e,
                                i2h_grads, s.i2h, io, stream));
  }
  if (need_du) {
    LT_TRY(lt_ln_backward(T, (int)H, io, x, saved->ln_stats, d.ln_weight, cdt, s.du, io, d.residual ? dy : nullptr,
                          grads->dx, grads->ln_weight, grads->ln_bias, s.ln_ws, s.ln_ws_bytes, stream, &reduces));
  }
  return lt_colreduce_flush(reduces, stream);
}

// ---------------------------------------------------------------------------------------------------------------------
// generalized linear layer alone
// ---------------------------------------------------------------------------------------------------------------------
extern "C" size_t lt_linear_backward_workspace_bytes(const lt_linear* lin, int64_t tokens, int32_t dtype) {
  if (!lin || tokens <= 0) return 0;
  Bump ws(nullptr);
  LinearBwdScratch s;
  plan_linear_backward(*lin, tokens, dtype, ws, s);
  return lt_align_up(ws.used, 256);
}

extern "C" int lt_linear_forward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, void* y,
                                 void* lowrank_hid, void* stream) {
  LT_REQUIRE(lin && x && y && tokens > 0, LT_ERR_BAD_ARG, "linear forward: bad arguments");
  LT_TRY(check_dtype(dtype, "linear forward"));
  LT_TRY(check_linear(*lin, "linear", NEED_FWD_TABLE));
  EpiParams e = epi_store_params(y, lin->out_features, dtype, lin->bias);
  return linear_forward_impl(*lin, tokens, dtype, x, EPI_STORE, e, lowrank_hid, dtype, (hipStream_t)stream);
}

extern "C" int lt_linear_backward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, const void* dy,
                                  const void* lowrank_hid, void* dx, const lt_linear_grads* grads, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  LT_REQUIRE(lin && x && dy && grads && tokens > 0, LT_ERR_BAD_ARG, "linear backward: bad arguments");
  LT_TRY(check_dtype(dtype, "linear backward"));
  LT_TRY(check_linear(*lin, "linear", NEED_BWD_TABLE));
  LT_REQUIRE(workspace && lt_aligned(workspace, 256) &&
                 workspace_bytes >= lt_linear_backward_workspace_bytes(lin, tokens, dtype),
             LT_ERR_WORKSPACE, "linear backward: needs a 256-byte aligned workspace of %zu bytes",
             lt_linear_backward_workspace_bytes(lin, tokens, dtype));
  Bump ws(workspace);
  LinearBwdScratch s;
  plan_linear_backward(*lin, tokens, dtype, ws, s);
  EpiParams e = epi_store_params(dx, lin->in_features, dtype, nullptr);
  return linear_backward_impl(*lin, tokens, dtype, x, dy, lowrank_hid, dx ? EPI_STORE : -1, e, *grads, s, dtype,
                              (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------------------------------
// block-sparse matmul alone
// ---------------------------------------------------------------------------------------------------------------------
static lt_linear main_weight_only(const lt_linear& lin) {
  lt_linear l = lin;
  l.bias = nullptr; l.lowrank_first = nullptr; l.lowrank_second = nullptr; l.lowrank = 0;
  return l;
}

extern "C" int lt_blocksparse_forward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, void* y,
                                      void* stream) {
  LT_REQUIRE(lin && x && y && tokens > 0, LT_ERR_BAD_ARG, "blocksparse forward: bad arguments");
  LT_REQUIRE(lin->block > 0, LT_ERR_BAD_ARG, "blocksparse forward: dense weight");
  LT_TRY(check_dtype(dtype, "blocksparse forward"));
  const lt_linear l = main_weight_only(*lin);
  LT_TRY(check_linear(l, "blocksparse", NEED_FWD_TABLE));
  EpiParams e = epi_store_params(y, l.out_features, dtype, nullptr);
  return linear_forward_impl(l, tokens, dtype, x, EPI_STORE, e, nullptr, dtype, (hipStream_t)stream);
}

extern "C" int lt_blocksparse_backward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, const void* dy,
                                       void* dx, void* dweight, void* stream) {
  LT_REQUIRE(lin && x && dy && tokens > 0, LT_ERR_BAD_ARG, "blocksparse backward: bad arguments");
  LT_REQUIRE(lin->block > 0, LT_ERR_BAD_ARG, "blocksparse backward: dense weight");
  LT_TRY(check_dtype(dtype, "blocksparse backward"));
  const lt_linear l = main_weight_only(*lin);
  LT_TRY(check_linear(l, "blocksparse", NEED_BWD_TABLE));
  lt_linear_grads grads;
  memset(&grads, 0, sizeof(grads));
  grads.weight = dweight;
  LinearBwdScratch s;
  memset(&s, 0, sizeof(s));
  EpiParams e = epi_store_params(dx, l.in_features, dtype, nullptr);
  return linear_backward_impl(l, tokens, dtype, x, dy, nullptr, dx ? EPI_STORE : -1, e, grads, s, dtype,
                              (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------------------------------
// LayerNorm, activation, dropout mask, plain GEMM
// ---------------------------------------------------------------------------------------------------------------------
extern "C" int lt_layernorm_forward(int64_t tokens, int32_t hidden, float eps, int32_t x_dtype, const void* x,
                                    const float* weight, const float* bias, int32_t y_dtype, void* y, float* stats,
                                    void* stream) {
  LT_TRY(check_dtype(x_dtype, "layernorm x"));
  LT_TRY(check_dtype(y_dtype, "layernorm y"));
  return lt_ln_forward(tokens, hidden, eps, x_dtype, x, weight, bias, y_dtype, y, stats, y_dtype, nullptr, nullptr, false,
                       (hipStream_t)stream);
}

extern "C" size_t lt_layernorm_backward_workspace_bytes(int64_t tokens, int32_t hidden) {
  if (tokens <= 0 || hidden <= 0) return 0;
  return lt_align_up(lt_ln_backward_workspace(tokens, hidden), 256);
}

extern "C" int lt_layernorm_backward(int64_t tokens, int32_t hidden, int32_t x_dtype, const void* x, const float* stats,
                                     const float* weight, int32_t dy_dtype, const void* dy, int32_t dx_dtype,
                                     const void* residual_grad, void* dx, float* dweight, float* dbias, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  LT_TRY(check_dtype(x_dtype, "layernorm backward x"));
  LT_TRY(check_dtype(dy_dtype, "layernorm backward dy"));
  LT_TRY(check_dtype(dx_dtype, "layernorm backward dx"));
  return lt_ln_backward(tokens, hidden, x_dtype, x, stats, weight, dy_dtype, dy, dx_dtype, residual_grad, dx, dweight,
                        dbias, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int lt_activation_forward(int64_t tokens, int32_t intermediate, int32_t gated, int32_t act, int32_t dtype,
                                     const void* pre, void* hid, void* stream) {
  LT_TRY(check_dtype(dtype, "activation"));
  LT_REQUIRE(act >= 0 && act < LT_ACT_COUNT, LT_ERR_UNSUPPORTED, "unknown activation %d", act);
  return lt_act_forward(tokens, intermediate, gated, act, dtype, pre, hid, (hipStream_t)stream);
}

extern "C" int lt_activation_backward(int64_t tokens, int32_t intermediate, int32_t gated, int32_t act, int32_t dtype,
                                      const void* pre, const void* d_hid, void* d_pre, void* stream) {
  LT_TRY(check_dtype(dtype, "activation backward"));
  LT_REQUIRE(act >= 0 && act < LT_ACT_COUNT, LT_ERR_UNSUPPORTED, "unknown activation %d", act);
  return lt_act_backward(tokens, intermediate, gated, act, dtype, pre, d_hid, d_pre, (hipStream_t)stream);
}

extern "C" int lt_dropout_mask(int64_t tokens, int32_t hidden, float p, uint64_t seed, uint64_t offset, uint8_t* keep,
                               void* stream) {
  LT_REQUIRE(tokens > 0 && hidden > 0 && p >= 0.f && p < 1.f, LT_ERR_BAD_ARG, "dropout mask: bad arguments");
  return lt_dropout_mask_launch(tokens * hidden, keep, make_dropout(p, seed, offset), (hipStream_t)stream);
}

extern "C" int lt_gemm(int32_t dtype, int64_t m, int64_t n, int64_t k, const void* a, int32_t a_kmajor, const void* b,
                       int32_t b_kmajor, int32_t c_dtype, void* c, int32_t force_generic, void* stream) {
  LT_TRY(check_dtype(dtype, "gemm"));
  LT_TRY(check_dtype(c_dtype, "gemm output"));
  LT_REQUIRE(a && b && c && m > 0 && n > 0 && k > 0, LT_ERR_BAD_ARG, "gemm: bad arguments");
  GemmProblem p = blank_problem();
  p.M = m; p.N = n; p.K[0] = k;
  p.A[0] = operand(a, a_kmajor ? k : m, a_kmajor);
  p.B[0] = operand(b, b_kmajor ? k : n, b_kmajor);
  p.epi = epi_store_params(c, n, c_dtype, nullptr);
  p.krot = (force_generic >> 4) & 15;
  p.tile_loop = (force_generic >> 8) & 1;
  force_generic &= 15;
  if (force_generic == 1) return lt_launch_gemm_generic(p, EPI_STORE, dtype, dtype, (hipStream_t)stream);
  p.variant = force_generic == 2 ? 1 : 0;  // 2: the register-staged tiled kernel instead of the copy-based one
  return lt_launch_gemm(p, EPI_STORE, dtype, dtype, (hipStream_t)stream);
}
