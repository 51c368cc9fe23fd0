// Instantiates the tiled bf16 GEMM kernels with the EPI_STORE epilogue (dense layouts and block-sparse walks).
#include "gemm_mfma_kernels.h"

int lt_mfma_launch_dense_kind0(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  return launch_layout<EPI_STORE>(p, io_dtype, stream);
}

int lt_mfma_launch_sparse_kind0(const GemmProblem& p, int io_dtype, hipStream_t stream) {
  return launch_sparse<EPI_STORE>(p, io_dtype, stream);
}

namespace {
template <bool A_KM, bool B_KM> int launch_skinny(const GemmProblem& p, int slices, hipStream_t stream) {
  const int tiles_m = (int)((p.M + 127) / 128), tiles_n = (int)(p.N / 128);
  dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)slices), block(256);
  // these products stream one large operand once against a small one: operand tiles are requested two k-steps ahead
  hipLaunchKernelGGL((gemm_bf16_kernel<128, 128, 2, 2, A_KM, B_KM, EPI_STORE, float, SPARSE_NONE, 1, 2>), grid, block, 0, stream, p, tiles_m, tiles_n);
  LT_LAUNCH_CHECK();
  return LT_OK;
}
}  // namespace

int lt_mfma_launch_skinny(const GemmProblem& p, int slices, hipStream_t stream) {
  const bool a_km = p.A[0].kmajor, b_km = p.B[0].kmajor;
  if (a_km && b_km) return launch_skinny<true, true>(p, slices, stream);
  if (a_km) return launch_skinny<true, false>(p, slices, stream);
  return launch_skinny<false, false>(p, slices, stream);
}
