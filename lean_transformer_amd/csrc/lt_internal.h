// Internal launchers shared between the translation units of libleanffn.
#pragma once
#include "lt_gemm.h"

// LayerNorm forward.  y may be null (statistics only).  tail: apply dropout, then add `residual` (dtype res_dtype).
int lt_ln_forward(int64_t T, int H, float eps, int x_dtype, const void* x, const float* w, const float* b, int y_dtype,
                  void* y, float* stats, int res_dtype, const void* residual, const DropoutParams* drop, bool tail,
                  hipStream_t stream);
size_t lt_ln_backward_workspace(int64_t T, int H);
int lt_ln_backward(int64_t T, int H, int x_dtype, const void* x, const float* stats, const float* w, int dy_dtype,
                   const void* dy, int dx_dtype, const void* residual_grad, void* dx, float* dweight, float* dbias,
                   void* workspace, size_t workspace_bytes, hipStream_t stream, ColReduceQueue* defer = nullptr);
size_t lt_colsum_workspace(int64_t rows, int cols);
int lt_colsum(int64_t rows, int cols, int64_t ld, int dtype, const void* in, float* out, void* workspace,
              size_t workspace_bytes, hipStream_t stream);
int lt_act_forward(int64_t T, int64_t I, int gated, int act, int dtype, const void* pre, void* hid, hipStream_t stream);
int lt_act_backward(int64_t T, int64_t I, int gated, int act, int dtype, const void* pre, const void* dhid, void* dpre,
                    hipStream_t stream);
int lt_dropout_cast_colsum(int64_t rows, int cols, int in_dtype, const void* in, int out_dtype, void* out,
                           const DropoutParams& drop, float* colsum, void* workspace, size_t workspace_bytes,
                           hipStream_t stream, ColReduceQueue* defer = nullptr);
int lt_dropout_cast(int64_t n, int in_dtype, const void* in, int out_dtype, void* out, const DropoutParams& drop,
                    hipStream_t stream);
int lt_dropout_mask_launch(int64_t n, uint8_t* keep, const DropoutParams& drop, hipStream_t stream);
