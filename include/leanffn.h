/*
 * libleanffn -- C ABI of the MI355X (gfx950) LeanFFN kernels.
 *
 * Everything here takes plain device pointers and sizes.  The library never allocates or frees device memory, keeps no
 * pointer after a call returns, launches asynchronously on the stream it is given and never synchronises.  Every function
 * that returns int returns LT_OK (0) or an lt_status error; lt_last_error() gives the message for the calling thread.
 * No C++ exception crosses this boundary.
 *
 * Reference interfaces replaced (paths relative to the learning-at-home/lean_transformer checkout):
 *   lt_ffn_forward / lt_ffn_backward   _LeanFFN.forward  lean_transformer/ffn.py:146-217,
 *                                      _LeanFFN.backward lean_transformer/ffn.py:233-306
 *   lt_linear_forward / _backward      _GeneralizedLinear.forward_functional / backward_functional
 *                                      lean_transformer/blocksparse/linear.py:161-230, :237-328
 *   lt_blocksparse_forward / _backward blocksparse_matmul / blocksparse_matmul_backward
 *                                      lean_transformer/blocksparse/native_backend.py:9-35, :38-76
 *                                      (also the role of the matmul_op plug-in slot, blocksparse/triton_backend.py:37-79)
 *   lt_layernorm_forward / _backward   the F.layer_norm calls and their autograd, lean_transformer/ffn.py:184,283,290-293
 *   lt_activation_forward / _backward  gelu_fused / gelu_fused_grad lean_transformer/utils.py:24-38 and
 *                                      _LeanFFN._apply_activation   lean_transformer/ffn.py:138-144
 *   lt_dropout_mask                    the mask torch.dropout draws at lean_transformer/ffn.py:204 and replays at :245
 */
#ifndef LEANFFN_H
#define LEANFFN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum lt_status {
  LT_OK = 0,
  LT_ERR_BAD_ARG = 1,     /* null pointer, non-positive size, misaligned pointer */
  LT_ERR_UNSUPPORTED = 2, /* a combination the kernels do not implement */
  LT_ERR_WORKSPACE = 3,   /* workspace smaller than lt_*_workspace_bytes() */
  LT_ERR_HIP = 4          /* a HIP runtime call or kernel launch failed */
} lt_status;

/* Element types.  The 16-bit type is fixed when the library is compiled: libleanffn.so computes in bfloat16 and accepts
 * LT_F32 and LT_BF16; libleanffn_f16.so is the same sources compiled with -DLT_HALF_IS_FP16 (IEEE binary16 operands on
 * v_mfma_f32_32x32x16_f16, the same kernels otherwise) and accepts LT_F32 and LT_F16.  Either library refuses the other's
 * 16-bit code with LT_ERR_BAD_ARG; a process may load both (they share no state).  Accumulation is fp32 in both; fp16's
 * range is the caller's to manage (loss scaling), as under torch.autocast(float16) in the reference. */
typedef enum lt_dtype { LT_F32 = 0, LT_BF16 = 1, LT_F16 = 2 } lt_dtype;

/* Activations evaluated in registers, value and derivative: the reference's gelu_fused (tanh form, lean_transformer/utils.py:24-38)
 * and the closed-form entries of transformers.activations.ACT2FN, the table the reference's ACT2FN extends (utils.py:80).
 * LT_ACT_GELU is the erf form; leaky_relu has slope 0.01.  Entries with learned parameters (prelu, xielu) have no kind. */
typedef enum lt_act {
  LT_ACT_GELU_FUSED = 0,
  LT_ACT_GELU = 1,
  LT_ACT_RELU = 2,
  LT_ACT_SILU = 3,
  LT_ACT_QUICK_GELU = 4,
  LT_ACT_GELU_10 = 5,
  LT_ACT_RELU6 = 6,
  LT_ACT_RELU2 = 7,
  LT_ACT_LEAKY_RELU = 8,
  LT_ACT_MISH = 9,
  LT_ACT_SIGMOID = 10,
  LT_ACT_TANH = 11,
  LT_ACT_LINEAR = 12,
  LT_ACT_HARDSWISH = 13,
  LT_ACT_LAPLACE = 14,
  LT_ACT_SQRT_SOFTPLUS = 15,
  LT_ACT_COUNT = 16
} lt_act;

/* One projection in the reference's "generalized linear" form: main weight (dense or native block-sparse), optional bias,
 * optional low-rank pair.  Weights and low-rank factors are in the compute dtype; the bias is always fp32. */
typedef struct lt_linear {
  const void* weight;              /* dense: [out_features, in_features]; sparse: [in_features, blocks_per_in, block] */
  const float* bias;               /* [out_features] or NULL */
  const void* lowrank_first;       /* [lowrank, in_features] or NULL */
  const void* lowrank_second;      /* [out_features, lowrank] or NULL */
  const int32_t* forward_indices;  /* sparse: [out_features / block, blocks_per_out]; dense: NULL */
  const int64_t* backward_indices; /* sparse: [in_features / block, blocks_per_in]; dense: NULL */
  int32_t in_features;
  int32_t out_features;
  int32_t lowrank;        /* 0 when there is no low-rank term */
  int32_t block;          /* sparse block size, 0 when dense */
  int32_t blocks_per_out; /* K: active blocks per output block row */
  int32_t blocks_per_in;  /* A: active blocks per input block column */
  int32_t out_group;      /* sparse: every aligned run of this many consecutive output blocks has the same list of input
                             blocks, and under each of them the run's weight blocks are adjacent (forward_indices of output
                             block ob0 + j = those of ob0, + j).  PixelFly with stretch=True on a tall matrix: out_blocks /
                             in_blocks.  A promise by the caller that only selects faster forward and weight-gradient
                             kernels; 0 or 1 when not known, which is always safe.  Must divide the number of output blocks.
                             A false promise computes with the wrong weight blocks (it cannot make a kernel read outside
                             the weight); lt_linear_check_out_group tests it on the device.
                             Low 16 bits: the run length.  High 16 bits, when above 1: the members of a run are not
                             consecutive but that many blocks apart (blocks r, r + s, r + 2 s, ...: PixelFly with stretch=False
                             on a tall matrix tiles a square pattern s blocks wide; length x s must equal the number of
                             output blocks).  Such a run promises equal lists of input blocks only and serves the
                             weight-gradient kernel only. */
  int32_t in_group;       /* sparse: every aligned run of this many consecutive input blocks has the same list of output
                             blocks (backward_indices of input block ib0 + i = those of ib0).  PixelFly with stretch=True on
                             a wide matrix: in_blocks / out_blocks.  A promise like out_group: it only selects a faster
                             weight-gradient kernel, 0 or 1 is always safe, it must divide the number of input blocks, a false
                             one puts wrong values into the weight gradient (never an access outside it), and
                             lt_linear_check_in_group tests it on the device.  Low / high 16 bits as in out_group. */
} lt_linear;

/* Where lt_linear_backward / lt_ffn_backward write parameter gradients; a NULL member skips that gradient.
 * weight / lowrank_* are in the compute dtype and shaped like the parameter, bias is fp32. */
typedef struct lt_linear_grads {
  void* weight;
  float* bias;
  void* lowrank_first;
  void* lowrank_second;
} lt_linear_grads;

typedef struct lt_ffn_desc {
  int64_t tokens;       /* T: rows of the flattened input */
  int32_t hidden;       /* H */
  int32_t intermediate; /* I; the up-projection has 2*I outputs when gated (first half = gate) */
  int32_t gated;
  int32_t act;           /* lt_act */
  int32_t residual;      /* add the input to the output */
  int32_t io_dtype;      /* lt_dtype of x, y, dy, dx */
  int32_t compute_dtype; /* lt_dtype of weights, GEMM operands, the saved pre-activation and weight gradients */
  float ln_eps;
  float dropout_p;        /* 0 disables dropout (also pass 0 in eval mode) */
  uint64_t dropout_seed;  /* Philox key */
  uint64_t dropout_offset;/* Philox stream offset; forward and backward of one call must pass the same pair */
  const float* ln_weight; /* [H] fp32 */
  const float* ln_bias;   /* [H] fp32 */
  const float* post_ln_weight; /* [H] fp32 or NULL: optional LayerNorm after the down-projection */
  const float* post_ln_bias;
  lt_linear i2h; /* H -> (gated ? 2I : I) */
  lt_linear h2o; /* I -> H */
} lt_ffn_desc;

/* Activations kept between forward and backward (all caller-allocated).  This is the reference's save-set
 * (lean_transformer/ffn.py:210-216) plus the LayerNorm row statistics (8 bytes per token). */
typedef struct lt_ffn_saved {
  void* pre_activation;  /* [T, 2I or I] compute dtype */
  float* ln_stats;       /* [T, 2] (mean, rstd) of the pre-LayerNorm */
  void* post_ln_input;   /* [T, H] compute dtype; only with post-LN, else NULL */
  void* i2h_lowrank_hid; /* [T, i2h.lowrank] compute dtype or NULL */
  void* h2o_lowrank_hid; /* [T, h2o.lowrank] compute dtype or NULL */
} lt_ffn_saved;

typedef struct lt_ffn_grads {
  void* dx;               /* [T, H] io dtype, or NULL */
  float* ln_weight;       /* [H] fp32 (both or neither of ln_weight / ln_bias) */
  float* ln_bias;
  float* post_ln_weight;
  float* post_ln_bias;
  lt_linear_grads i2h;
  lt_linear_grads h2o;
} lt_ffn_grads;

const char* lt_version(void);
const char* lt_last_error(void);

/* ---- whole FFN block ------------------------------------------------------------------------------------------------ */
size_t lt_ffn_forward_workspace_bytes(const lt_ffn_desc* desc);
size_t lt_ffn_backward_workspace_bytes(const lt_ffn_desc* desc);
/* y = [x +] dropout([postLN](act(LN(x) W1^T + b1) W2^T + b2)); fills *saved. */
int lt_ffn_forward(const lt_ffn_desc* desc, const void* x, void* y, const lt_ffn_saved* saved, void* workspace,
                   size_t workspace_bytes, void* stream);
/* gradients of the above given dy, recomputing LayerNorm output and activation from x and saved->pre_activation */
int lt_ffn_backward(const lt_ffn_desc* desc, const void* x, const void* dy, const lt_ffn_saved* saved,
                    const lt_ffn_grads* grads, void* workspace, size_t workspace_bytes, void* stream);

/* ---- generalized linear: y = x W^T (+ bias) (+ (x L1^T) L2^T) ------------------------------------------------------- */
size_t lt_linear_backward_workspace_bytes(const lt_linear* lin, int64_t tokens, int32_t dtype);
/* x [T, in], y [T, out], lowrank_hid [T, lowrank] (written when lin->lowrank > 0), all in `dtype` */
int lt_linear_forward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, void* y, void* lowrank_hid,
                      void* stream);
/* dx may be NULL; dy [T, out]; lowrank_hid as written by lt_linear_forward */
int lt_linear_backward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, const void* dy,
                       const void* lowrank_hid, void* dx, const lt_linear_grads* grads, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Tests lin->out_group against lin->forward_indices on the device: writes 1 to *flag (device memory, 4 bytes) when every
 * aligned run of out_group output blocks shares one list of input blocks with adjacent weight blocks, else 0.  Asynchronous
 * like everything else: the caller reads the flag when it chooses (once per index table is enough).  No counterpart in the
 * reference, whose matmul takes no such hint. */
int lt_linear_check_out_group(const lt_linear* lin, int32_t* flag, void* stream);
/* The same for lin->in_group against lin->backward_indices.  No counterpart in the reference either. */
int lt_linear_check_in_group(const lt_linear* lin, int32_t* flag, void* stream);

/* ---- block-sparse matmul alone (weight in the native [in_features, A, block] format) ----------------------------------- */
int lt_blocksparse_forward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, void* y, void* stream);
/* dx and/or dweight may be NULL */
int lt_blocksparse_backward(const lt_linear* lin, int64_t tokens, int32_t dtype, const void* x, const void* dy, void* dx,
                            void* dweight, void* stream);

/* ---- LayerNorm over the last dimension -------------------------------------------------------------------------------- */
/* x [T, H] in x_dtype -> y [T, H] in y_dtype; stats [T, 2] = (mean, rstd) written when non-NULL */
int lt_layernorm_forward(int64_t tokens, int32_t hidden, float eps, int32_t x_dtype, const void* x, const float* weight,
                         const float* bias, int32_t y_dtype, void* y, float* stats, void* stream);
size_t lt_layernorm_backward_workspace_bytes(int64_t tokens, int32_t hidden);
/* dx = LN'(dy) [+ residual_grad]; dweight / dbias fp32 [H]; stats from the forward */
int lt_layernorm_backward(int64_t tokens, int32_t hidden, int32_t x_dtype, const void* x, const float* stats,
                          const float* weight, int32_t dy_dtype, const void* dy, int32_t dx_dtype,
                          const void* residual_grad, void* dx, float* dweight, float* dbias, void* workspace,
                          size_t workspace_bytes, void* stream);

/* lt_layernorm_backward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid allocation).  No counterpart in the reference.  Same arguments and results as
 * lt_layernorm_backward without the workspace: the partial parameter-gradient rows go to a buffer of
 * lt_layernorm_backward_static_scratch_bytes() (8 MiB) that the library holds in static device memory, one copy per GPU,
 * looked up on the first call on each device.  The device that owns `stream` must be the current device.  Rows of a
 * multiple of 4 elements with 16-byte aligned pointers fit for every tokens / hidden <= 8192; other shapes are refused
 * with LT_ERR_UNSUPPORTED once tokens * hidden * 8 bytes (tokens capped at 1024) exceed the buffer.  Calls no allocator.
 * All calls on one GPU share the buffer: calls that overlap in time on the same GPU (different streams, or two captured
 * graphs replayed side by side) race.  The buffer's address is looked up on the first call on each device, which must
 * therefore happen outside stream capture (one warm-up call per device): a first call on a capturing stream is refused with
 * LT_ERR_UNSUPPORTED and leaves the capture intact. */
size_t lt_layernorm_backward_static_scratch_bytes(void);
int lt_layernorm_backward_static(int64_t tokens, int32_t hidden, int32_t x_dtype, const void* x, const float* stats,
                                 const float* weight, int32_t dy_dtype, const void* dy, int32_t dx_dtype,
                                 const void* residual_grad, void* dx, float* dweight, float* dbias, void* stream);

/* ---- activation alone (for tests of the in-register maths) ------------------------------------------------------------ */
/* pre [T, 2I or I] -> hid [T, I] */
int lt_activation_forward(int64_t tokens, int32_t intermediate, int32_t gated, int32_t act, int32_t dtype,
                          const void* pre, void* hid, void* stream);
/* d_hid [T, I], pre -> d_pre [T, 2I or I] */
int lt_activation_backward(int64_t tokens, int32_t intermediate, int32_t gated, int32_t act, int32_t dtype,
                           const void* pre, const void* d_hid, void* d_pre, void* stream);

/* ---- dropout mask of a [T, H] output: keep[t*H + h] in {0,1}, the mask the fused kernels apply for (seed, offset) ------- */
int lt_dropout_mask(int64_t tokens, int32_t hidden, float p, uint64_t seed, uint64_t offset, uint8_t* keep, void* stream);

/* ---- plain GEMM on the library's kernels (tests and benchmarks of the MFMA core) -------------------------------------- */
/* C[M,N] = op(A) op(B): a_kmajor != 0: A is [M,K] row-major, else [K,M]; b_kmajor != 0: B is [N,K] row-major, else [K,N].
 * force_generic (low 4 bits): 0 the library's own choice; 1 the any-shape kernel even when a tiled bf16 kernel applies;
 * 2 the register-staged tiled kernel instead of the copy-based one.  Bits 4..7, when non-zero, choose how workgroups stagger
 * their walk over k in the copy-based kernel (15: not at all) instead of the default for the layout.  Bit 8: one workgroup
 * per tile in the copy-based kernel even when there are more tiles than compute units (by default one workgroup per compute
 * unit then loops over its tiles; both give the same bits).  The choice travels with the call (no process-wide state): lt_gemm
 * may run concurrently with every other entry point. */
int lt_gemm(int32_t dtype, int64_t m, int64_t n, int64_t k, const void* a, int32_t a_kmajor, const void* b,
            int32_t b_kmajor, int32_t c_dtype, void* c, int32_t force_generic, void* stream);

/* ---- per-kernel timing (no counterpart in the reference: measurement only) ----------------------------------------------
 * While enabled, every kernel launch of the library is bracketed by two HIP events recorded on the launch stream.
 * lt_profile_read waits for the recorded events and returns one aggregated entry per kernel tag: launches, total device
 * milliseconds, and the algorithmic flops / bytes the launches stand for (0 where not applicable). */
typedef struct lt_profile_entry {
  char name[64];
  int64_t launches;
  double ms;
  double flops;
  double bytes;
} lt_profile_entry;

int lt_profile_enable(int32_t enable);
int lt_profile_reset(void);
/* fills at most max_entries entries, returns the number of distinct tags (negative lt_status on error) */
int lt_profile_read(lt_profile_entry* entries, int32_t max_entries);

#ifdef __cplusplus
}
#endif
#endif /* LEANFFN_H */
