// Instantiates the tiled bf16 GEMM kernels with the EPI_OUT epilogue (dense layouts and block-sparse walks).
#include "gemm_mfma_kernels.h"

int lt_mfma_launch_dense_kind3(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  return launch_layout<EPI_OUT>(p, io_dtype, stream);
}

int lt_mfma_launch_sparse_kind3(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  return launch_sparse<EPI_OUT>(p, io_dtype, stream);
}
