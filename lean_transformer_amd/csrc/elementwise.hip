// HBM-bound kernels of the FFN path: LayerNorm forward / backward with wavefront-shuffle row reductions, column sums for
// bias / LayerNorm-parameter gradients, stand-alone activation forward / backward, dropout replay and the dropout mask.
#include <mutex>

#include "lt_internal.h"

namespace {

constexpr int LN_MAXV = 32;  // float4 per lane held in registers: rows up to 64 * 4 * 32 = 8192 elements stay on chip
// The row kernels are instantiated for 8, 16 and 32 vectors per lane (hidden <= 2048, 4096, 8192): the register arrays are
// sized by the template argument, so a narrower row leaves room for more wavefronts per SIMD.
static int ln_vectors_per_lane(int H) { return H <= 2048 ? 8 : H <= 4096 ? 16 : 32; }

// ---------------------------------------------------------------------------------------------------------------------
// LayerNorm forward: one wavefront per row.  The row is read once into registers (when hidden % 4 == 0 and it fits), the
// mean and the centred second moment are reduced across the 64 lanes with shuffles, and the normalised row is written in
// the GEMM operand dtype.  TAIL fuses what follows a post-LayerNorm: dropout, then the residual add.
// ---------------------------------------------------------------------------------------------------------------------
template <typename TX, typename TY, typename TR, bool TAIL, int MAXV>
__global__ __launch_bounds__(256) void ln_fwd_kernel(int64_t T, int H, float eps, const TX* __restrict__ x,
                                                      const float* __restrict__ w, const float* __restrict__ b,
                                                      TY* __restrict__ y, float* __restrict__ stats,
                                                      const TR* __restrict__ residual, DropoutParams drop, int vec) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  const TX* xr = x + row * H;
  const float inv_h = 1.0f / (float)H;
  float mean, rstd;
  if (vec) {
    // W elements per lane per piece: 8 where the row length allows it, so that a bf16 output leaves in 16-byte stores
    auto row_in_registers = [&](auto W_c) {
      constexpr int W = decltype(W_c)::value, PIECES = MAXV * 4 / W;
      float v[PIECES][W];
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < PIECES; i++) {
        const int c = (i * 64 + lane) * W;
        if (c < H) {
          if constexpr (W == 8) load8(xr + c, v[i]);
          else load4(xr + c, v[i]);
#pragma unroll
          for (int e = 0; e < W; e++) s += v[i][e];
        }
      }
      mean = wave_sum(s) * inv_h;
      float q = 0.f;
#pragma unroll
      for (int i = 0; i < PIECES; i++) {
        const int c = (i * 64 + lane) * W;
        if (c < H) {
#pragma unroll
          for (int e = 0; e < W; e++) {
            const float d = v[i][e] - mean;
            q += d * d;
          }
        }
      }
      rstd = 1.0f / sqrtf(wave_sum(q) * inv_h + eps);
      if (y) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
          const int c = (i * 64 + lane) * W;
          if (c < H) {
            float wv[W], bv[W], o[W];
            if constexpr (W == 8) {
              load8(w + c, wv);
              load8(b + c, bv);
            } else {
              load4(w + c, wv);
              load4(b + c, bv);
            }
#pragma unroll
            for (int e = 0; e < W; e++) o[e] = (v[i][e] - mean) * rstd * wv[e] + bv[e];
            if constexpr (TAIL) {
              if (drop.p > 0.f) {
#pragma unroll
                for (int h = 0; h < W / 4; h++) {
                  bool keep[4];
                  dropout_keep4(drop, row * H + c + 4 * h, keep);
#pragma unroll
                  for (int e = 0; e < 4; e++) o[4 * h + e] = keep[e] ? o[4 * h + e] * drop.scale : 0.f;
                }
              }
              if (residual) {
                float rv[W];
                if constexpr (W == 8) load8(residual + row * H + c, rv);
                else load4(residual + row * H + c, rv);
#pragma unroll
                for (int e = 0; e < W; e++) o[e] += rv[e];
              }
            }
            if constexpr (W == 8) store8(y + row * H + c, o);
            else store4(y + row * H + c, o);
          }
        }
      }
    };
    if (vec == 2) row_in_registers(std::integral_constant<int, 8>{});
    else row_in_registers(std::integral_constant<int, 4>{});
  } else {
    float s = 0.f;
    for (int c = lane; c < H; c += 64) s += ldf(xr, c);
    mean = wave_sum(s) * inv_h;
    float q = 0.f;
    for (int c = lane; c < H; c += 64) {
      const float d = ldf(xr, c) - mean;
      q += d * d;
    }
    rstd = 1.0f / sqrtf(wave_sum(q) * inv_h + eps);
    if (y) {
      for (int c = lane; c < H; c += 64) {
        float o = (ldf(xr, c) - mean) * rstd * w[c] + b[c];
        if constexpr (TAIL) {
          if (drop.p > 0.f) o = dropout_keep(drop, row * H + c) ? o * drop.scale : 0.f;
          if (residual) o += ldf(residual, row * H + c);
        }
        stf(y, row * H + c, o);
      }
    }
  }
  if (stats && lane == 0) {
    stats[row * 2] = mean;
    stats[row * 2 + 1] = rstd;
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// LayerNorm backward.  A workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ...; its 256 threads split the columns.
//   dxhat = dy * w;  c1 = mean(dxhat);  c2 = mean(dxhat * xhat);  dx = rstd * (dxhat - c1 - xhat * c2) [+ residual grad]
// Column sums of dy * xhat (-> dweight) and dy (-> dbias) are kept per thread across the rows of the workgroup and written
// as one partial row per workgroup; lt_colreduce sums the partial rows.
// ---------------------------------------------------------------------------------------------------------------------
constexpr int LNB_MAXC = 32;  // columns per thread (hidden <= 256 * 32 = 8192) for the register-resident partial sums

__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();  // protect `red` against the previous use
  if (lane == 0) {
    red[wave * 2] = a;
    red[wave * 2 + 1] = b;
  }
  __syncthreads();
  a = red[0] + red[2] + red[4] + red[6];
  b = red[1] + red[3] + red[5] + red[7];
}

template <typename TX, typename TDY, typename TDX>
__global__ __launch_bounds__(256) void ln_bwd_kernel(int64_t T, int H, const TX* __restrict__ x,
                                                      const float* __restrict__ stats, const float* __restrict__ w,
                                                      const TDY* __restrict__ dy, const TDX* __restrict__ residual_grad,
                                                      TDX* __restrict__ dx, float* __restrict__ partial) {
  __shared__ float red[8];
  const int tid = threadIdx.x;
  float pw[LNB_MAXC], pb[LNB_MAXC];
#pragma unroll
  for (int i = 0; i < LNB_MAXC; i++) pw[i] = pb[i] = 0.f;
  const float inv_h = 1.0f / (float)H;
  for (int64_t row = blockIdx.x; row < T; row += gridDim.x) {
    const float mean = stats[row * 2], rstd = stats[row * 2 + 1];
    const TX* xr = x + row * H;
    const TDY* dyr = dy + row * H;
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < LNB_MAXC; i++) {
      const int c = tid + i * 256;
      if (c < H) {
        const float xh = (ldf(xr, c) - mean) * rstd, g = ldf(dyr, c);
        const float dxh = g * w[c];
        s1 += dxh;
        s2 += dxh * xh;
        pw[i] += g * xh;
        pb[i] += g;
      }
    }
    block_sum2(s1, s2, red);
    const float c1 = s1 * inv_h, c2 = s2 * inv_h;
    if (dx) {
#pragma unroll
      for (int i = 0; i < LNB_MAXC; i++) {
        const int c = tid + i * 256;
        if (c < H) {
          const float xh = (ldf(xr, c) - mean) * rstd;
          float v = rstd * (ldf(dyr, c) * w[c] - c1 - xh * c2);
          if (residual_grad) v += ldf(residual_grad, row * H + c);
          stf(dx, row * H + c, v);
        }
      }
    }
  }
  if (partial) {
#pragma unroll
    for (int i = 0; i < LNB_MAXC; i++) {
      const int c = tid + i * 256;
      if (c < H) {
        partial[((int64_t)blockIdx.x * 2) * H + c] = pw[i];
        partial[((int64_t)blockIdx.x * 2 + 1) * H + c] = pb[i];
      }
    }
  }
}

// Rows wider than the register-resident kernels take (hidden > 8192), any alignment: the same arithmetic with the columns in
// a loop.  dx: a workgroup per row (grid-stride), two passes over the row; parameter gradients: one column per thread over a
// slice of rows, one partial (dweight, dbias) row per slice.
template <typename TX, typename TDY, typename TDX>
__global__ __launch_bounds__(256) void ln_bwd_dx_wide_kernel(int64_t T, int H, const TX* __restrict__ x,
                                                              const float* __restrict__ stats, const float* __restrict__ w,
                                                              const TDY* __restrict__ dy,
                                                              const TDX* __restrict__ residual_grad, TDX* __restrict__ dx) {
  __shared__ float red[8];
  const float inv_h = 1.0f / (float)H;
  for (int64_t row = blockIdx.x; row < T; row += gridDim.x) {
    const float mean = stats[row * 2], rstd = stats[row * 2 + 1];
    const TX* xr = x + row * H;
    const TDY* dyr = dy + row * H;
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) {
      const float dxh = ldf(dyr, c) * w[c];
      s1 += dxh;
      s2 += dxh * ((ldf(xr, c) - mean) * rstd);
    }
    block_sum2(s1, s2, red);
    const float c1 = s1 * inv_h, c2 = s2 * inv_h;
    for (int c = threadIdx.x; c < H; c += 256) {
      const float xh = (ldf(xr, c) - mean) * rstd;
      float v = rstd * (ldf(dyr, c) * w[c] - c1 - xh * c2);
      if (residual_grad) v += ldf(residual_grad, row * H + c);
      stf(dx, row * H + c, v);
    }
  }
}

template <typename TX, typename TDY>
__global__ __launch_bounds__(256) void ln_bwd_param_wide_kernel(int64_t T, int H, const TX* __restrict__ x,
                                                                 const float* __restrict__ stats, const TDY* __restrict__ dy,
                                                                 int64_t rows_per_slice, float* __restrict__ partial) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= H) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice, r1 = min(T, r0 + rows_per_slice);
  float pw = 0.f, pb = 0.f;
  for (int64_t r = r0; r < r1; r++) {
    const float g = ldf(dy, r * H + c);
    pw += g * ((ldf(x, r * H + c) - stats[r * 2]) * stats[r * 2 + 1]);
    pb += g;
  }
  partial[((int64_t)blockIdx.y * 2) * H + c] = pw;
  partial[((int64_t)blockIdx.y * 2 + 1) * H + c] = pb;
}

// Vectorised LayerNorm backward (hidden % 4 == 0, hidden <= 8192, 16-byte aligned rows), split in two so that neither half
// has to keep per-column partial sums next to a cached row:
//   ln_bwd_dx_kernel      one wavefront per row; dy and x of the row live in registers, the two row sums go through
//                         shuffles, dx (+ residual gradient) is written with 16-byte stores
//   ln_bwd_param_kernel   column-parallel: 64 lanes x 4 columns per workgroup and 4 row lanes walking a slice of rows;
//                         writes one partial (dweight, dbias) row per slice, summed by colreduce_kernel
template <typename TX, typename TDY, typename TDX, int MAXV>
__global__ __launch_bounds__(256) void ln_bwd_dx_kernel(int64_t T, int H, const TX* __restrict__ x,
                                                         const float* __restrict__ stats, const float* __restrict__ w,
                                                         const TDY* __restrict__ dy, const TDX* __restrict__ residual_grad,
                                                         TDX* __restrict__ dx) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  const float mean = stats[row * 2], rstd = stats[row * 2 + 1];
  const TX* xr = x + row * H;
  const TDY* dyr = dy + row * H;
  float xh[MAXV][4], dxh[MAXV][4];
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int c = (i * 64 + lane) * 4;
    if (c < H) {
      float wv[4];
      load4(xr + c, xh[i]);
      load4(dyr + c, dxh[i]);
      load4(w + c, wv);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        xh[i][e] = (xh[i][e] - mean) * rstd;
        dxh[i][e] *= wv[e];
        s1 += dxh[i][e];
        s2 += dxh[i][e] * xh[i][e];
      }
    }
  }
  const float inv_h = 1.0f / (float)H;
  const float c1 = wave_sum(s1) * inv_h, c2 = wave_sum(s2) * inv_h;
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int c = (i * 64 + lane) * 4;
    if (c < H) {
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; e++) o[e] = rstd * (dxh[i][e] - c1 - xh[i][e] * c2);
      if (residual_grad) {
        float rv[4];
        load4(residual_grad + row * H + c, rv);
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] += rv[e];
      }
      store4(dx + row * H + c, o);
    }
  }
}

template <typename TX, typename TDY>
__global__ __launch_bounds__(256) void ln_bwd_param_kernel(int64_t T, int H, const TX* __restrict__ x,
                                                            const float* __restrict__ stats, const TDY* __restrict__ dy,
                                                            int64_t rows_per_slice, float* __restrict__ partial) {
  __shared__ float red[4][64][8];
  const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + cl) * 4;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice, r1 = min(T, r0 + rows_per_slice);
  float pw[4] = {0.f, 0.f, 0.f, 0.f}, pb[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < H) {
    for (int64_t r = r0 + rl; r < r1; r += 4) {
      const float mean = stats[r * 2], rstd = stats[r * 2 + 1];
      float xv[4], g[4];
      load4(x + r * H + c, xv);
      load4(dy + r * H + c, g);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        pw[e] += g[e] * ((xv[e] - mean) * rstd);
        pb[e] += g[e];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 4; e++) {
    red[rl][cl][e] = pw[e];
    red[rl][cl][4 + e] = pb[e];
  }
  __syncthreads();
  if (rl == 0 && c < H) {
    float ow[4], ob[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      ow[e] = red[0][cl][e] + red[1][cl][e] + red[2][cl][e] + red[3][cl][e];
      ob[e] = red[0][cl][4 + e] + red[1][cl][4 + e] + red[2][cl][4 + e] + red[3][cl][4 + e];
    }
    store4(partial + ((int64_t)blockIdx.y * 2) * H + c, ow);
    store4(partial + ((int64_t)blockIdx.y * 2 + 1) * H + c, ob);
  }
}

// out[c] = sum_r partial[r * stride + c], one thread per column (rows are few)
__global__ void colreduce_kernel(int rows, int64_t stride, int cols, const float* __restrict__ partial,
                                 float* __restrict__ out) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  float s = 0.f;
  for (int r = 0; r < rows; r++) s += partial[(int64_t)r * stride + c];
  out[c] = s;
}

// same, 16 row lanes x 16 column lanes of 4 columns per workgroup: short dependent chains, 16-byte loads
__global__ __launch_bounds__(256) void colreduce4_kernel(int rows, int64_t stride, int cols, const float* __restrict__ partial,
                                                         float* __restrict__ out) {
  __shared__ float red[16][16][5];
  const int cl = threadIdx.x & 15, rl = threadIdx.x >> 4;
  const int c = (blockIdx.x * 16 + cl) * 4;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {
    for (int r = rl; r < rows; r += 16) {
      float v[4];
      load4(partial + (int64_t)r * stride + c, v);
#pragma unroll
      for (int e = 0; e < 4; e++) s[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 4; e++) red[rl][cl][e] = s[e];
  __syncthreads();
  if (rl == 0 && c < cols) {
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      o[e] = 0.f;
#pragma unroll
      for (int q = 0; q < 16; q++) o[e] += red[q][cl][e];
    }
    store4(out + c, o);
  }
}

// several such sums in one launch: blockIdx.y picks the job; the same arithmetic in the same order as colreduce4_kernel
__global__ __launch_bounds__(256) void colreduce4_multi_kernel(ColReduceQueue q) {
  __shared__ float red[16][16][5];
  const ColReduceJob& job = q.job[blockIdx.y];
  const int cl = threadIdx.x & 15, rl = threadIdx.x >> 4;
  const int c = (blockIdx.x * 16 + cl) * 4;
  if (blockIdx.x * 64 >= job.cols) return;  // (the whole workgroup)
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < job.cols) {
    for (int r = rl; r < job.rows; r += 16) {
      float v[4];
      load4(job.partial + (int64_t)r * job.stride + c, v);
#pragma unroll
      for (int e = 0; e < 4; e++) s[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 4; e++) red[rl][cl][e] = s[e];
  __syncthreads();
  if (rl == 0 && c < job.cols) {
    float o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      o[e] = 0.f;
#pragma unroll
      for (int k = 0; k < 16; k++) o[e] += red[k][cl][e];
    }
    store4(job.out + c, o);
  }
}

// out[c] = sum of `rows` rows of partial: picks the vector kernel when the layout allows; with a queue that has room, the
// vector form waits for the queue's flush
static void launch_colreduce(int rows, int64_t stride, int cols, const float* partial, float* out, hipStream_t stream,
                             ColReduceQueue* defer = nullptr) {
  const bool vec = (cols & 3) == 0 && (stride & 3) == 0 && lt_aligned(partial, 16) && lt_aligned(out, 16);
  if (vec && defer && defer->n < 4) {
    defer->job[defer->n++] = ColReduceJob{partial, out, rows, cols, stride};
    return;
  }
  if (vec)
    hipLaunchKernelGGL(colreduce4_kernel, dim3((unsigned)((cols + 63) / 64)), dim3(256), 0, stream, rows, stride, cols, partial, out);
  else
    hipLaunchKernelGGL(colreduce_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, stream, rows, stride, cols, partial, out);
}


// partial[blockIdx.y][c] = sum over this row-slice of in[t, c]; 64 column lanes x 4 row lanes per workgroup
template <typename T>
__global__ __launch_bounds__(256) void colsum_partial_kernel(int64_t rows, int cols, int64_t ld, const T* __restrict__ in,
                                                              int64_t rows_per_slice, float* __restrict__ partial) {
  __shared__ float red[4][64];
  const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + cl;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice, r1 = min(rows, r0 + rows_per_slice);
  float s = 0.f;
  if (c < cols)
    for (int64_t r = r0 + rl; r < r1; r += 4) s += ldf(in, r * ld + c);
  red[rl][cl] = s;
  __syncthreads();
  if (rl == 0 && c < cols) partial[(int64_t)blockIdx.y * cols + c] = red[0][cl] + red[1][cl] + red[2][cl] + red[3][cl];
}

// same with 8 consecutive columns per thread (16-byte loads for bf16): 32 column lanes x 8 row lanes per workgroup
template <typename T>
__global__ __launch_bounds__(256) void colsum_partial8_kernel(int64_t rows, int cols, int64_t ld, const T* __restrict__ in,
                                                               int64_t rows_per_slice, float* __restrict__ partial) {
  __shared__ float red[8][32][9];
  const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + cl) * 8;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice, r1 = min(rows, r0 + rows_per_slice);
  float s[8];
#pragma unroll
  for (int e = 0; e < 8; e++) s[e] = 0.f;
  if (c < cols) {
#pragma unroll 4
    for (int64_t r = r0 + rl; r < r1; r += 8) {
      float v[8];
      load8(in + r * ld + c, v);
#pragma unroll
      for (int e = 0; e < 8; e++) s[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++) red[rl][cl][e] = s[e];
  __syncthreads();
  if (rl == 0 && c < cols) {
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      o[e] = 0.f;
#pragma unroll
      for (int q = 0; q < 8; q++) o[e] += red[q][cl][e];
    }
    store8(partial + (int64_t)blockIdx.y * cols + c, o);
  }
}

// dropout replay + cast of a [rows, cols] gradient with the column sums of what it writes (the bias gradient of the layer
// the result feeds), in the work decomposition of colsum_partial8_kernel
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void dropout_cast_colsum_kernel(int64_t rows, int cols, const TI* __restrict__ in,
                                                                  TO* __restrict__ out, DropoutParams drop,
                                                                  int64_t rows_per_slice, float* __restrict__ partial) {
  __shared__ float red[8][32][9];
  const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + cl) * 8;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice, r1 = min(rows, r0 + rows_per_slice);
  float s[8];
#pragma unroll
  for (int e = 0; e < 8; e++) s[e] = 0.f;
  if (c < cols) {
#pragma unroll 4
    for (int64_t r = r0 + rl; r < r1; r += 8) {
      const int64_t idx = r * cols + c;
      float v[8];
      load8(in + idx, v);
      if (drop.p > 0.f) {
        bool k0[4], k1[4];
        dropout_keep4(drop, idx, k0);
        dropout_keep4(drop, idx + 4, k1);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[e] = k0[e] ? v[e] * drop.scale : 0.f;
          v[4 + e] = k1[e] ? v[4 + e] * drop.scale : 0.f;
        }
      }
      store8(out + idx, v);
#pragma unroll
      for (int e = 0; e < 8; e++) s[e] += (float)(TO)v[e];  // sums of the values as stored
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++) red[rl][cl][e] = s[e];
  __syncthreads();
  if (rl == 0 && c < cols) {
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      o[e] = 0.f;
#pragma unroll
      for (int q = 0; q < 8; q++) o[e] += red[q][cl][e];
    }
    store8(partial + (int64_t)blockIdx.y * cols + c, o);
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// stand-alone (gated) activation forward / backward on a saved pre-activation
// ---------------------------------------------------------------------------------------------------------------------
template <typename TC>
__global__ void act_fwd_kernel(int64_t T, int64_t I, int gated, int act, const TC* __restrict__ pre, TC* __restrict__ hid) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * I) return;
  const int64_t t = idx / I, i = idx % I;
  const int64_t ldp = gated ? 2 * I : I;
  float a = act_value<PRECISE>(act, ldf(pre, t * ldp + i));
  if (gated) a *= ldf(pre, t * ldp + I + i);
  stf(hid, idx, a);
}

// 8 consecutive features per thread (16-byte accesses for bf16); I % 8 == 0 and 16-byte aligned rows
template <typename TC>
__global__ void act_fwd8_kernel(int64_t T, int64_t I, int gated, int act, const TC* __restrict__ pre, TC* __restrict__ hid) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (idx >= T * I) return;
  const int64_t t = idx / I, i = idx % I;
  const int64_t ldp = gated ? 2 * I : I;
  float g[8], h[8];
  load8(pre + t * ldp + i, g);
#pragma unroll
  for (int e = 0; e < 8; e++) h[e] = act_value<PRECISE>(act, g[e]);
  if (gated) {
    float l[8];
    load8(pre + t * ldp + I + i, l);
#pragma unroll
    for (int e = 0; e < 8; e++) h[e] *= l[e];
  }
  store8(hid + idx, h);
}

template <typename TC>
__global__ void act_bwd8_kernel(int64_t T, int64_t I, int gated, int act, const TC* __restrict__ pre,
                                const TC* __restrict__ dhid, TC* __restrict__ dpre) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (idx >= T * I) return;
  const int64_t t = idx / I, i = idx % I;
  const int64_t ldp = gated ? 2 * I : I;
  float g[8], a[8], da[8], dh[8], o[8];
  load8(pre + t * ldp + i, g);
  load8(dhid + idx, dh);
#pragma unroll
  for (int e = 0; e < 8; e++) act_eval<PRECISE>(act, g[e], a[e], da[e]);
  if (gated) {
    float l[8];
    load8(pre + t * ldp + I + i, l);
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = dh[e] * l[e] * da[e];
    store8(dpre + t * ldp + i, o);
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = dh[e] * a[e];
    store8(dpre + t * ldp + I + i, o);
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = dh[e] * da[e];
    store8(dpre + t * ldp + i, o);
  }
}

template <typename TC>
__global__ void act_bwd_kernel(int64_t T, int64_t I, int gated, int act, const TC* __restrict__ pre,
                               const TC* __restrict__ dhid, TC* __restrict__ dpre) {
  constexpr bool PRECISE = sizeof(TC) == 4;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * I) return;
  const int64_t t = idx / I, i = idx % I;
  const int64_t ldp = gated ? 2 * I : I;
  float a, da;
  act_eval<PRECISE>(act, ldf(pre, t * ldp + i), a, da);
  const float dh = ldf(dhid, idx);
  if (gated) {
    const float pl = ldf(pre, t * ldp + I + i);
    stf(dpre, t * ldp + i, dh * pl * da);
    stf(dpre, t * ldp + I + i, dh * a);
  } else {
    stf(dpre, t * ldp + i, dh * da);
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// dropout replay on the incoming gradient (and conversion to the GEMM operand dtype); mask bytes for tests
// ---------------------------------------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void dropout_cast_kernel(int64_t n, const TI* __restrict__ in, TO* __restrict__ out, DropoutParams drop) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  float v = ldf(in, idx);
  if (drop.p > 0.f) v = dropout_keep(drop, idx) ? v * drop.scale : 0.f;
  stf(out, idx, v);
}

__global__ void dropout_mask_kernel(int64_t n, uint8_t* __restrict__ keep, DropoutParams drop) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  keep[idx] = drop.p > 0.f ? (dropout_keep(drop, idx) ? 1 : 0) : 1;
}

// sum of split-k partial results in slice order, 4 elements per thread
template <typename TO>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, int slices, int64_t stride, int64_t count, int cols,
                                     const float* __restrict__ bias, TO* __restrict__ out) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= count) return;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < slices; s++) {
    float v[4];
    load4(partial + (int64_t)s * stride + i, v);
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] += v[e];
  }
  if (bias) {
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] += bias[(i + e) % cols];
  }
  store4(out + i, acc);
}

inline unsigned blocks_for(int64_t n, int threads) { return (unsigned)((n + threads - 1) / threads); }

}  // namespace

// ---------------------------------------------------------------------------------------------------------------------
// host-side launchers
// ---------------------------------------------------------------------------------------------------------------------
int lt_ln_forward(int64_t T, int H, float eps, int x_dtype, const void* x, const float* w, const float* b, int y_dtype,
                  void* y, float* stats, int res_dtype, const void* residual, const DropoutParams* drop, bool tail,
                  hipStream_t stream) {
  LT_REQUIRE(T > 0 && H > 0 && x, LT_ERR_BAD_ARG, "layernorm: bad arguments");
  LT_REQUIRE(!y || (w && b), LT_ERR_BAD_ARG, "layernorm: weight and bias are required when an output is requested");
  // rows are held in registers and moved 4 elements at a time when the size and every pointer allow it
  int vec = (H & 3) == 0 && H <= 64 * 4 * LN_MAXV && lt_aligned(x, 16) && (!y || lt_aligned(y, 16)) &&
            (!w || lt_aligned(w, 16)) && (!b || lt_aligned(b, 16)) && (!residual || lt_aligned(residual, 16));
  if (vec && (H & 7) == 0) vec = 2;  // 8 elements per lane per piece: 16-byte stores of a bf16 output
  dim3 grid(blocks_for(T, 4)), block(256);
  DropoutParams d = drop ? *drop : make_dropout(0.f, 0, 0);
  LtProfileScope scope(tail ? "layernorm_fwd_tail" : (y ? "layernorm_fwd" : "layernorm_stats"), 0.0,
                       (double)T * H * (lt_dtype_size(x_dtype) + (y ? lt_dtype_size(y_dtype) : 0) +
                                        (residual ? lt_dtype_size(res_dtype) : 0)) + (stats ? 8.0 * T : 0.0),
                       stream);
  const int maxv = ln_vectors_per_lane(H);
#define LT_LN_LAUNCH_V(TX, TY, TR, TAILV, MAXV)                                                                             \
  hipLaunchKernelGGL((ln_fwd_kernel<TX, TY, TR, TAILV, MAXV>), grid, block, 0, stream, T, H, eps, (const TX*)x, w, b, (TY*)y, \
                     stats, (const TR*)residual, d, vec)
#define LT_LN_LAUNCH(TX, TY, TR, TAILV)                     \
  do {                                                      \
    if (maxv == 8) LT_LN_LAUNCH_V(TX, TY, TR, TAILV, 8);    \
    else if (maxv == 16) LT_LN_LAUNCH_V(TX, TY, TR, TAILV, 16); \
    else LT_LN_LAUNCH_V(TX, TY, TR, TAILV, 32);             \
  } while (0)
  if (!tail) {
    if (x_dtype == LT_F32 && y_dtype == LT_F32) LT_LN_LAUNCH(float, float, float, false);
    else if (x_dtype == LT_F32) LT_LN_LAUNCH(float, bf16, float, false);
    else if (y_dtype == LT_F32) LT_LN_LAUNCH(bf16, float, float, false);
    else LT_LN_LAUNCH(bf16, bf16, float, false);
  } else {
    // post-LayerNorm tail: input in the compute dtype, output and residual in the io dtype (res_dtype == y_dtype)
    LT_REQUIRE(res_dtype == y_dtype, LT_ERR_BAD_ARG, "layernorm tail: residual and output dtypes differ");
    if (x_dtype == LT_F32 && y_dtype == LT_F32) LT_LN_LAUNCH(float, float, float, true);
    else if (x_dtype == LT_F32) LT_LN_LAUNCH(float, bf16, bf16, true);
    else if (y_dtype == LT_F32) LT_LN_LAUNCH(bf16, float, float, true);
    else LT_LN_LAUNCH(bf16, bf16, bf16, true);
  }
#undef LT_LN_LAUNCH
#undef LT_LN_LAUNCH_V
  LT_LAUNCH_CHECK();
  return LT_OK;
}

static int ln_bwd_blocks(int64_t T) { return (int)(T < 1024 ? T : 1024); }
static int ln_bwd_slices(int64_t T) {
  int64_t s = (T + 63) / 64;
  return (int)(s < 1 ? 1 : (s > 128 ? 128 : s));
}

// partial (dweight, dbias) rows: one pair per workgroup of the any-shape kernel or per row slice of the vectorised one
size_t lt_ln_backward_workspace(int64_t T, int H) {
  const int rows = ln_bwd_blocks(T) > ln_bwd_slices(T) ? ln_bwd_blocks(T) : ln_bwd_slices(T);
  return (size_t)rows * 2 * (size_t)H * sizeof(float);
}

int lt_ln_backward(int64_t T, int H, int x_dtype, const void* x, const float* stats, const float* w, int dy_dtype,
                   const void* dy, int dx_dtype, const void* residual_grad, void* dx, float* dweight, float* dbias,
                   void* workspace, size_t workspace_bytes, hipStream_t stream, ColReduceQueue* defer) {
  LT_REQUIRE(T > 0 && H > 0 && x && stats && w && dy, LT_ERR_BAD_ARG, "layernorm backward: bad arguments");
  LT_REQUIRE((dweight == nullptr) == (dbias == nullptr), LT_ERR_BAD_ARG, "layernorm backward: pass both dweight and dbias or neither");
  float* partial = dweight ? (float*)workspace : nullptr;
  LtProfileScope scope("layernorm_bwd", 0.0,
                       (double)T * H * ((dx ? 1 : 0) + (dweight ? 1 : 0)) * (lt_dtype_size(x_dtype) + lt_dtype_size(dy_dtype)) +
                           (double)T * H * ((dx ? lt_dtype_size(dx_dtype) : 0) + (dx && residual_grad ? lt_dtype_size(dx_dtype) : 0)),
                       stream);
  const int key = (x_dtype == LT_BF16) * 4 + (dy_dtype == LT_BF16) * 2 + (dx_dtype == LT_BF16);
  const bool vec = (H & 3) == 0 && H <= 64 * 4 * LN_MAXV && lt_aligned(x, 16) && lt_aligned(dy, 16) && lt_aligned(w, 16) &&
                   (!dx || lt_aligned(dx, 16)) && (!residual_grad || lt_aligned(residual_grad, 16)) &&
                   (!partial || lt_aligned(partial, 16));
  const bool wide = H > 256 * LNB_MAXC;  // wider than the register-resident kernels take
  // partial (dweight, dbias) rows of the path taken: one pair per row slice (vectorised, wide) or per workgroup (any-shape)
  int partial_rows = (vec || wide) ? ln_bwd_slices(T) : ln_bwd_blocks(T);
  if (dweight) {
    const size_t need = (size_t)partial_rows * 2 * (size_t)H * sizeof(float);
    LT_REQUIRE(workspace && workspace_bytes >= need, LT_ERR_WORKSPACE,
               "layernorm backward: %zu bytes of scratch needed for the parameter gradients, %zu given", need, workspace_bytes);
  }
  if (vec) {
    if (dx) {
      dim3 grid(blocks_for(T, 4)), block(256);
      const int maxv = ln_vectors_per_lane(H);
#define LT_LNB_DX_V(TX, TDY, TDX, MAXV)                                                                                       \
  hipLaunchKernelGGL((ln_bwd_dx_kernel<TX, TDY, TDX, MAXV>), grid, block, 0, stream, T, H, (const TX*)x, stats, w, (const TDY*)dy, \
                     (const TDX*)residual_grad, (TDX*)dx)
#define LT_LNB_DX(TX, TDY, TDX)                        \
  do {                                                 \
    if (maxv == 8) LT_LNB_DX_V(TX, TDY, TDX, 8);       \
    else if (maxv == 16) LT_LNB_DX_V(TX, TDY, TDX, 16); \
    else LT_LNB_DX_V(TX, TDY, TDX, 32);                \
  } while (0)
      switch (key) {
        case 0: LT_LNB_DX(float, float, float); break;
        case 1: LT_LNB_DX(float, float, bf16); break;
        case 2: LT_LNB_DX(float, bf16, float); break;
        case 3: LT_LNB_DX(float, bf16, bf16); break;
        case 4: LT_LNB_DX(bf16, float, float); break;
        case 5: LT_LNB_DX(bf16, float, bf16); break;
        case 6: LT_LNB_DX(bf16, bf16, float); break;
        default: LT_LNB_DX(bf16, bf16, bf16); break;
      }
#undef LT_LNB_DX
#undef LT_LNB_DX_V
      LT_LAUNCH_CHECK();
    }
    if (partial) {
      const int64_t rps = (T + partial_rows - 1) / partial_rows;
      dim3 grid(blocks_for(H, 256), partial_rows), block(256);
#define LT_LNB_PARAM(TX, TDY)                                                                                            \
  hipLaunchKernelGGL((ln_bwd_param_kernel<TX, TDY>), grid, block, 0, stream, T, H, (const TX*)x, stats, (const TDY*)dy, rps, \
                     partial)
      switch (key >> 1) {
        case 0: LT_LNB_PARAM(float, float); break;
        case 1: LT_LNB_PARAM(float, bf16); break;
        case 2: LT_LNB_PARAM(bf16, float); break;
        default: LT_LNB_PARAM(bf16, bf16); break;
      }
#undef LT_LNB_PARAM
      LT_LAUNCH_CHECK();
    }
  } else if (wide) {
    if (dx) {
      dim3 grid((unsigned)ln_bwd_blocks(T)), block(256);
#define LT_LNB_WIDE(TX, TDY, TDX)                                                                                          \
  hipLaunchKernelGGL((ln_bwd_dx_wide_kernel<TX, TDY, TDX>), grid, block, 0, stream, T, H, (const TX*)x, stats, w, (const TDY*)dy, \
                     (const TDX*)residual_grad, (TDX*)dx)
      switch (key) {
        case 0: LT_LNB_WIDE(float, float, float); break;
        case 1: LT_LNB_WIDE(float, float, bf16); break;
        case 2: LT_LNB_WIDE(float, bf16, float); break;
        case 3: LT_LNB_WIDE(float, bf16, bf16); break;
        case 4: LT_LNB_WIDE(bf16, float, float); break;
        case 5: LT_LNB_WIDE(bf16, float, bf16); break;
        case 6: LT_LNB_WIDE(bf16, bf16, float); break;
        default: LT_LNB_WIDE(bf16, bf16, bf16); break;
      }
#undef LT_LNB_WIDE
      LT_LAUNCH_CHECK();
    }
    if (partial) {
      const int64_t rps = (T + partial_rows - 1) / partial_rows;
      dim3 grid(blocks_for(H, 256), partial_rows), block(256);
#define LT_LNB_WIDE_PARAM(TX, TDY)                                                                                         \
  hipLaunchKernelGGL((ln_bwd_param_wide_kernel<TX, TDY>), grid, block, 0, stream, T, H, (const TX*)x, stats, (const TDY*)dy, \
                     rps, partial)
      switch (key >> 1) {
        case 0: LT_LNB_WIDE_PARAM(float, float); break;
        case 1: LT_LNB_WIDE_PARAM(float, bf16); break;
        case 2: LT_LNB_WIDE_PARAM(bf16, float); break;
        default: LT_LNB_WIDE_PARAM(bf16, bf16); break;
      }
#undef LT_LNB_WIDE_PARAM
      LT_LAUNCH_CHECK();
    }
  } else {
    dim3 grid(partial_rows), block(256);
#define LT_LNB_LAUNCH(TX, TDY, TDX)                                                                                      \
  hipLaunchKernelGGL((ln_bwd_kernel<TX, TDY, TDX>), grid, block, 0, stream, T, H, (const TX*)x, stats, w, (const TDY*)dy, \
                     (const TDX*)residual_grad, (TDX*)dx, partial)
    switch (key) {
      case 0: LT_LNB_LAUNCH(float, float, float); break;
      case 1: LT_LNB_LAUNCH(float, float, bf16); break;
      case 2: LT_LNB_LAUNCH(float, bf16, float); break;
      case 3: LT_LNB_LAUNCH(float, bf16, bf16); break;
      case 4: LT_LNB_LAUNCH(bf16, float, float); break;
      case 5: LT_LNB_LAUNCH(bf16, float, bf16); break;
      case 6: LT_LNB_LAUNCH(bf16, bf16, float); break;
      default: LT_LNB_LAUNCH(bf16, bf16, bf16); break;
    }
#undef LT_LNB_LAUNCH
    LT_LAUNCH_CHECK();
  }
  if (dweight) {
    // partial rows alternate (dweight, dbias): stride 2 * H between them
    launch_colreduce(partial_rows, (int64_t)2 * H, H, partial, dweight, stream, defer);
    launch_colreduce(partial_rows, (int64_t)2 * H, H, partial + H, dbias, stream, defer);
    LT_LAUNCH_CHECK();
  }
  return LT_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// LayerNorm backward for callers that cannot allocate device memory.  The partial (dweight, dbias) rows live in a
// file-scope device array instead of a caller workspace.  Each GPU holds its own copy of the array at its own address,
// looked up once per device; host code only ever uses that looked-up address, never the array's name.
// ---------------------------------------------------------------------------------------------------------------------
constexpr size_t LT_LN_STATIC_SCRATCH_BYTES = (size_t)8 << 20;  // 128 row slices x (dweight, dbias) x 8192 columns x 4 bytes
static __device__ __align__(256) unsigned char scratch[LT_LN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int LT_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[LT_MAX_DEVICES] = {};

// device address of `scratch` on the device `stream` belongs to, which must be the current device
int static_scratch_for(hipStream_t stream, void** out) {
  int current = -1, owner = -1;
  LT_HIP(hipGetDevice(&current));
  LT_HIP(hipStreamGetDevice(stream, &owner));
  LT_REQUIRE(owner == current, LT_ERR_BAD_ARG,
             "layernorm backward (static scratch): the stream belongs to device %d but device %d is current", owner, current);
  LT_REQUIRE(current >= 0 && current < LT_MAX_DEVICES, LT_ERR_UNSUPPORTED, "device index %d above %d", current, LT_MAX_DEVICES - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[current]) {
    // the look-up is not a stream operation: under capture it could invalidate the caller's capture, so it is refused there
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    LT_HIP(hipStreamIsCapturing(stream, &capture));
    LT_REQUIRE(capture == hipStreamCaptureStatusNone, LT_ERR_UNSUPPORTED,
               "layernorm backward (static scratch): the first call on a device must happen outside stream capture");
    void* ptr = nullptr;
    LT_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    LT_REQUIRE(ptr != nullptr, LT_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch");
    g_scratch_ptr[current] = ptr;
  }
  *out = g_scratch_ptr[current];
  return LT_OK;
}
}  // namespace

extern "C" size_t lt_layernorm_backward_static_scratch_bytes(void) { return LT_LN_STATIC_SCRATCH_BYTES; }

extern "C" int lt_layernorm_backward_static(int64_t tokens, int32_t hidden, int32_t x_dtype, const void* x, const float* stats,
                                            const float* weight, int32_t dy_dtype, const void* dy, int32_t dx_dtype,
                                            const void* residual_grad, void* dx, float* dweight, float* dbias,
                                            void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  for (int d : {x_dtype, dy_dtype, dx_dtype})
    LT_REQUIRE(d == LT_F32 || d == LT_BF16, LT_ERR_BAD_ARG,
               "layernorm backward (static scratch): dtype code %d is not one of this library's (fp32 = %d, " LT_HALF_NAME " = %d)", d,
               (int)LT_F32, (int)LT_BF16);
  void* ptr = nullptr;
  if (dweight) LT_TRY(static_scratch_for(stream, &ptr));
  const int status = lt_ln_backward(tokens, hidden, x_dtype, x, stats, weight, dy_dtype, dy, dx_dtype, residual_grad, dx,
                                    dweight, dbias, ptr, LT_LN_STATIC_SCRATCH_BYTES, stream);
  if (status == LT_ERR_WORKSPACE)
    LT_FAIL(LT_ERR_UNSUPPORTED,
            "layernorm backward (static scratch): tokens=%lld hidden=%d needs more than the %zu-byte static buffer "
            "(rows of a multiple of 4 elements with 16-byte aligned pointers always fit); use lt_layernorm_backward",
            (long long)tokens, hidden, LT_LN_STATIC_SCRATCH_BYTES);
  return status;
}

// slices of 64 rows (8 per thread), at most 64 of them: 16 x 64 workgroups at 4096 columns, enough to keep every CU's
// memory pipeline full (slices of 256 rows left one workgroup per CU: 2.9 TB/s)
static int colsum_slices(int64_t rows) {
  int64_t s = (rows + 63) / 64;
  return (int)(s < 1 ? 1 : (s > 64 ? 64 : s));
}

size_t lt_colsum_workspace(int64_t rows, int cols) { return (size_t)colsum_slices(rows) * (size_t)cols * sizeof(float); }

int lt_colsum(int64_t rows, int cols, int64_t ld, int dtype, const void* in, float* out, void* workspace,
              size_t workspace_bytes, hipStream_t stream) {
  LT_REQUIRE(rows > 0 && cols > 0 && in && out, LT_ERR_BAD_ARG, "colsum: bad arguments");
  LT_REQUIRE(workspace && workspace_bytes >= lt_colsum_workspace(rows, cols), LT_ERR_WORKSPACE,
             "colsum: workspace of %zu bytes needed", lt_colsum_workspace(rows, cols));
  LtProfileScope scope("colsum", 0.0, (double)rows * cols * lt_dtype_size(dtype), stream);
  const int slices = colsum_slices(rows);
  const int64_t rps = (rows + slices - 1) / slices;
  float* partial = (float*)workspace;
  if ((cols & 7) == 0 && (ld & 7) == 0 && lt_aligned(in, 16) && lt_aligned(partial, 16)) {
    dim3 grid(blocks_for(cols, 256), slices), block(256);
    if (dtype == LT_F32)
      hipLaunchKernelGGL((colsum_partial8_kernel<float>), grid, block, 0, stream, rows, cols, ld, (const float*)in, rps, partial);
    else
      hipLaunchKernelGGL((colsum_partial8_kernel<bf16>), grid, block, 0, stream, rows, cols, ld, (const bf16*)in, rps, partial);
  } else {
    dim3 grid(blocks_for(cols, 64), slices), block(256);
    if (dtype == LT_F32)
      hipLaunchKernelGGL((colsum_partial_kernel<float>), grid, block, 0, stream, rows, cols, ld, (const float*)in, rps, partial);
    else
      hipLaunchKernelGGL((colsum_partial_kernel<bf16>), grid, block, 0, stream, rows, cols, ld, (const bf16*)in, rps, partial);
  }
  launch_colreduce(slices, (int64_t)cols, cols, partial, out, stream);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_act_forward(int64_t T, int64_t I, int gated, int act, int dtype, const void* pre, void* hid, hipStream_t stream) {
  LT_REQUIRE(T > 0 && I > 0 && pre && hid, LT_ERR_BAD_ARG, "activation: bad arguments");
  LtProfileScope scope("activation_fwd", 0.0, (double)T * I * lt_dtype_size(dtype) * (gated ? 3 : 2), stream);
  dim3 grid(blocks_for(T * I, 256)), block(256);
  const bool vec = (I & 7) == 0 && lt_aligned(pre, 16) && lt_aligned(hid, 16);
  if (vec) grid = dim3(blocks_for(T * I / 8, 256));
  if (dtype == LT_F32 && vec)
    hipLaunchKernelGGL((act_fwd8_kernel<float>), grid, block, 0, stream, T, I, gated, act, (const float*)pre, (float*)hid);
  else if (vec)
    hipLaunchKernelGGL((act_fwd8_kernel<bf16>), grid, block, 0, stream, T, I, gated, act, (const bf16*)pre, (bf16*)hid);
  else if (dtype == LT_F32)
    hipLaunchKernelGGL((act_fwd_kernel<float>), grid, block, 0, stream, T, I, gated, act, (const float*)pre, (float*)hid);
  else
    hipLaunchKernelGGL((act_fwd_kernel<bf16>), grid, block, 0, stream, T, I, gated, act, (const bf16*)pre, (bf16*)hid);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_act_backward(int64_t T, int64_t I, int gated, int act, int dtype, const void* pre, const void* dhid, void* dpre,
                    hipStream_t stream) {
  LT_REQUIRE(T > 0 && I > 0 && pre && dhid && dpre, LT_ERR_BAD_ARG, "activation backward: bad arguments");
  LtProfileScope scope("activation_bwd", 0.0, (double)T * I * lt_dtype_size(dtype) * (gated ? 5 : 3), stream);
  dim3 grid(blocks_for(T * I, 256)), block(256);
  const bool vec = (I & 7) == 0 && lt_aligned(pre, 16) && lt_aligned(dhid, 16) && lt_aligned(dpre, 16);
  if (vec) grid = dim3(blocks_for(T * I / 8, 256));
  if (dtype == LT_F32 && vec)
    hipLaunchKernelGGL((act_bwd8_kernel<float>), grid, block, 0, stream, T, I, gated, act, (const float*)pre,
                       (const float*)dhid, (float*)dpre);
  else if (vec)
    hipLaunchKernelGGL((act_bwd8_kernel<bf16>), grid, block, 0, stream, T, I, gated, act, (const bf16*)pre,
                       (const bf16*)dhid, (bf16*)dpre);
  else if (dtype == LT_F32)
    hipLaunchKernelGGL((act_bwd_kernel<float>), grid, block, 0, stream, T, I, gated, act, (const float*)pre,
                       (const float*)dhid, (float*)dpre);
  else
    hipLaunchKernelGGL((act_bwd_kernel<bf16>), grid, block, 0, stream, T, I, gated, act, (const bf16*)pre,
                       (const bf16*)dhid, (bf16*)dpre);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_dropout_cast(int64_t n, int in_dtype, const void* in, int out_dtype, void* out, const DropoutParams& drop,
                    hipStream_t stream) {
  LT_REQUIRE(n > 0 && in && out, LT_ERR_BAD_ARG, "dropout: bad arguments");
  LtProfileScope scope("dropout_replay_cast", 0.0, (double)n * (lt_dtype_size(in_dtype) + lt_dtype_size(out_dtype)), stream);
  dim3 grid(blocks_for(n, 256)), block(256);
  const int key = (in_dtype == LT_BF16) * 2 + (out_dtype == LT_BF16);
  switch (key) {
    case 0: hipLaunchKernelGGL((dropout_cast_kernel<float, float>), grid, block, 0, stream, n, (const float*)in, (float*)out, drop); break;
    case 1: hipLaunchKernelGGL((dropout_cast_kernel<float, bf16>), grid, block, 0, stream, n, (const float*)in, (bf16*)out, drop); break;
    case 2: hipLaunchKernelGGL((dropout_cast_kernel<bf16, float>), grid, block, 0, stream, n, (const bf16*)in, (float*)out, drop); break;
    default: hipLaunchKernelGGL((dropout_cast_kernel<bf16, bf16>), grid, block, 0, stream, n, (const bf16*)in, (bf16*)out, drop); break;
  }
  LT_LAUNCH_CHECK();
  return LT_OK;
}

// lt_dropout_cast of a [rows, cols] tensor plus colsum[c] = sum over rows of the result; workspace as for lt_colsum
int lt_dropout_cast_colsum(int64_t rows, int cols, int in_dtype, const void* in, int out_dtype, void* out,
                           const DropoutParams& drop, float* colsum, void* workspace, size_t workspace_bytes,
                           hipStream_t stream, ColReduceQueue* defer) {
  LT_REQUIRE(rows > 0 && cols > 0 && in && out && colsum, LT_ERR_BAD_ARG, "dropout + column sums: bad arguments");
  LT_REQUIRE(workspace && workspace_bytes >= lt_colsum_workspace(rows, cols), LT_ERR_WORKSPACE,
             "dropout + column sums: workspace of %zu bytes needed", lt_colsum_workspace(rows, cols));
  if ((cols & 7) != 0 || !lt_aligned(in, 16) || !lt_aligned(out, 16) || !lt_aligned(workspace, 16)) {
    LT_TRY(lt_dropout_cast(rows * cols, in_dtype, in, out_dtype, out, drop, stream));
    return lt_colsum(rows, cols, cols, out_dtype, out, colsum, workspace, workspace_bytes, stream);
  }
  LtProfileScope scope("dropout_replay_cast", 0.0, (double)rows * cols * (lt_dtype_size(in_dtype) + lt_dtype_size(out_dtype)),
                       stream);
  const int slices = colsum_slices(rows);
  const int64_t rps = (rows + slices - 1) / slices;
  float* partial = (float*)workspace;
  dim3 grid(blocks_for(cols, 256), slices), block(256);
  const int key = (in_dtype == LT_BF16) * 2 + (out_dtype == LT_BF16);
  switch (key) {
    case 0: hipLaunchKernelGGL((dropout_cast_colsum_kernel<float, float>), grid, block, 0, stream, rows, cols, (const float*)in, (float*)out, drop, rps, partial); break;
    case 1: hipLaunchKernelGGL((dropout_cast_colsum_kernel<float, bf16>), grid, block, 0, stream, rows, cols, (const float*)in, (bf16*)out, drop, rps, partial); break;
    case 2: hipLaunchKernelGGL((dropout_cast_colsum_kernel<bf16, float>), grid, block, 0, stream, rows, cols, (const bf16*)in, (float*)out, drop, rps, partial); break;
    default: hipLaunchKernelGGL((dropout_cast_colsum_kernel<bf16, bf16>), grid, block, 0, stream, rows, cols, (const bf16*)in, (bf16*)out, drop, rps, partial); break;
  }
  launch_colreduce(slices, (int64_t)cols, cols, partial, colsum, stream, defer);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_dropout_mask_launch(int64_t n, uint8_t* keep, const DropoutParams& drop, hipStream_t stream) {
  LT_REQUIRE(n > 0 && keep, LT_ERR_BAD_ARG, "dropout mask: bad arguments");
  hipLaunchKernelGGL(dropout_mask_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream, n, keep, drop);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_splitk_reduce(const float* partial, int slices, int64_t stride, int64_t count, int cols, const float* bias,
                     int out_dtype, void* out, hipStream_t stream) {
  LT_REQUIRE(partial && out && slices > 0 && count > 0 && (count & 3) == 0 && (stride & 3) == 0, LT_ERR_BAD_ARG,
             "split-k reduce: bad arguments");
  LtProfileScope scope("splitk_reduce", 0.0, (double)count * (4.0 * slices + lt_dtype_size(out_dtype)), stream);
  dim3 grid(blocks_for(count / 4, 256)), block(256);
  if (out_dtype == LT_F32)
    hipLaunchKernelGGL((splitk_reduce_kernel<float>), grid, block, 0, stream, partial, slices, stride, count, cols, bias, (float*)out);
  else
    hipLaunchKernelGGL((splitk_reduce_kernel<bf16>), grid, block, 0, stream, partial, slices, stride, count, cols, bias, (bf16*)out);
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_colreduce_flush(ColReduceQueue& queue, hipStream_t stream) {
  if (queue.n == 0) return LT_OK;
  int blocks = 1;
  double bytes = 0.0;
  for (int i = 0; i < queue.n; i++) {
    blocks = std::max(blocks, (queue.job[i].cols + 63) / 64);
    bytes += (double)queue.job[i].cols * 4.0 * (queue.job[i].rows + 1);
  }
  LtProfileScope scope("colreduce", 0.0, bytes, stream);
  hipLaunchKernelGGL(colreduce4_multi_kernel, dim3((unsigned)blocks, (unsigned)queue.n), dim3(256), 0, stream, queue);
  queue.n = 0;
  LT_LAUNCH_CHECK();
  return LT_OK;
}

int lt_colreduce(int rows, int64_t stride, int cols, const float* partial, float* out, hipStream_t stream,
                 ColReduceQueue* defer) {
  LT_REQUIRE(rows > 0 && cols > 0 && partial && out, LT_ERR_BAD_ARG, "colreduce: bad arguments");
  if (defer && defer->n < 4 && (cols & 3) == 0 && (stride & 3) == 0 && lt_aligned(partial, 16) && lt_aligned(out, 16)) {
    launch_colreduce(rows, stride, cols, partial, out, stream, defer);
    return LT_OK;
  }
  LtProfileScope scope("colreduce", 0.0, (double)cols * 4.0 * (rows + 1), stream);
  launch_colreduce(rows, stride, cols, partial, out, stream);
  LT_LAUNCH_CHECK();
  return LT_OK;
}
