// Shared device / host helpers of libleanffn (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/leanffn.h"

// The 16-bit element type of this build.  The sources name it bf16 throughout; compiled with -DLT_HALF_IS_FP16 the same
// name stands for IEEE binary16, the dtype code the library accepts for it is LT_F16 instead of LT_BF16, and the matrix
// instruction is the f16 one of the same shape.  Nothing else depends on the format: conversions are casts, the LDS and
// copy paths move 16-bit words, every accumulator is fp32.
#ifdef LT_HALF_IS_FP16
typedef _Float16 bf16;
#define LT_BF16 LT_F16
#define LT_HALF_NAME "fp16"
#define LT_MFMA_32X32X16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0)
#else
typedef __bf16 bf16;
#define LT_HALF_NAME "bf16"
#define LT_MFMA_32X32X16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
#endif
typedef __attribute__((__vector_size__(8 * sizeof(bf16)))) bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

// ---------------------------------------------------------------------------------------------------------------------
// error reporting: thread-local message, int status across the C ABI
// ---------------------------------------------------------------------------------------------------------------------
void lt_set_error(const char* fmt, ...);

#define LT_FAIL(code, ...)     \
  do {                         \
    lt_set_error(__VA_ARGS__); \
    return (code);             \
  } while (0)

#define LT_REQUIRE(cond, code, ...)            \
  do {                                         \
    if (!(cond)) LT_FAIL(code, __VA_ARGS__);   \
  } while (0)

#define LT_HIP(expr)                                                                                   \
  do {                                                                                                 \
    hipError_t e_ = (expr);                                                                            \
    if (e_ != hipSuccess) LT_FAIL(LT_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),   \
                                  __FILE__, __LINE__);                                                 \
  } while (0)

#define LT_LAUNCH_CHECK()                                                                                     \
  do {                                                                                                        \
    hipError_t e_ = hipGetLastError();                                                                        \
    if (e_ != hipSuccess) LT_FAIL(LT_ERR_HIP, "kernel launch failed: %s (%s:%d)", hipGetErrorString(e_),      \
                                  __FILE__, __LINE__);                                                        \
  } while (0)

#define LT_TRY(expr)            \
  do {                          \
    int s_ = (expr);            \
    if (s_ != LT_OK) return s_; \
  } while (0)

// ---------------------------------------------------------------------------------------------------------------------
// optional per-kernel timing: a scope object brackets the launches issued while it lives with two events on `stream`
// ---------------------------------------------------------------------------------------------------------------------
bool lt_profile_active();
void lt_profile_begin(const char* tag, double flops, double bytes, hipStream_t stream);
void lt_profile_end(hipStream_t stream);
struct LtProfileScope {
  hipStream_t stream;
  bool on;
  LtProfileScope(const char* tag, double flops, double bytes, hipStream_t s) : stream(s), on(lt_profile_active()) {
    if (on) lt_profile_begin(tag, flops, bytes, s);
  }
  ~LtProfileScope() {
    if (on) lt_profile_end(stream);
  }
};

static inline size_t lt_dtype_size(int dtype) { return dtype == LT_F32 ? 4 : 2; }
static inline size_t lt_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline bool lt_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---------------------------------------------------------------------------------------------------------------------
// scalar conversions
// ---------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i) { return to_f32(p[i]); }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v) { p[i] = from_f32<T>(v); }

// 4 consecutive elements <-> 4 floats (pointers must be aligned to 4 elements)
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16* p, float (&v)[4]) {
  union { uint2 u; bf16 h[4]; } t;
  t.u = *reinterpret_cast<const uint2*>(p);
#pragma unroll
  for (int i = 0; i < 4; i++) v[i] = (float)t.h[i];
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16* p, const float (&v)[4]) {
  union { uint2 u; bf16 h[4]; } t;
#pragma unroll
  for (int i = 0; i < 4; i++) t.h[i] = (bf16)v[i];
  *reinterpret_cast<uint2*>(p) = t.u;
}

// 8 consecutive elements <-> 8 floats (pointers must be aligned to 8 elements for bf16, 4 for fp32)
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float (&v)[8]) {
  union { uint4 u; bf16 h[8]; } t;
  t.u = *reinterpret_cast<const uint4*>(p);
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = (float)t.h[i];
}
__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float (&v)[8]) {
  union { uint4 u; bf16 h[8]; } t;
#pragma unroll
  for (int i = 0; i < 8; i++) t.h[i] = (bf16)v[i];
  *reinterpret_cast<uint4*>(p) = t.u;
}

// ---------------------------------------------------------------------------------------------------------------------
// wavefront (64 lanes) reductions through cross-lane shuffles
// ---------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---------------------------------------------------------------------------------------------------------------------
// activations and their derivatives, evaluated in fp32 registers.  PRECISE selects libm-grade tanh/exp for the fp32 path;
// the bf16 path uses the hardware exp2 / reciprocal approximations (error far below one bf16 ulp).
// gelu_fused follows lean_transformer/utils.py:24-38, including its truncated constants.
// ---------------------------------------------------------------------------------------------------------------------
template <bool PRECISE> __device__ __forceinline__ float lt_tanh(float z) {
  if constexpr (PRECISE) {
    return tanhf(z);
  } else {
    // tanh z = 1 - 2 / (1 + e^{2z}); saturates correctly when e^{2z} over/underflows
    float e = __expf(2.0f * z);
    return 1.0f - __fdividef(2.0f, 1.0f + e);
  }
}
template <bool PRECISE> __device__ __forceinline__ float lt_sigmoid(float z) {
  if constexpr (PRECISE) {
    return 1.0f / (1.0f + expf(-z));
  } else {
    return __fdividef(1.0f, 1.0f + __expf(-z));
  }
}

// value and derivative in one go (they share the transcendental)
template <bool PRECISE> __device__ __forceinline__ void act_eval(int act, float x, float& value, float& deriv) {
  switch (act) {
    case LT_ACT_GELU_FUSED: {
      if constexpr (PRECISE) {
        float t = lt_tanh<PRECISE>(0.79788456f * x * (1.0f + 0.044715f * x * x));
        value = x * 0.5f * (1.0f + t);
        deriv = 0.5f * x * ((1.0f - t * t) * (0.79788456f + 0.1070322243f * x * x)) + 0.5f * (1.0f + t);
      } else {
        // The same function with fewer instructions (the fused GEMM epilogues are bound by them): with u the tanh argument,
        // 0.5 (1 + tanh u) = s = 1 / (1 + e^{-2u}), 2u = x (1.59576912 + 0.071354816 x^2), so gelu = x s and
        // gelu' = s + x s (1 - s) (2u)' with (2u)' = 1.59576912 + 0.214064448 x^2.  The exponent is formed directly as the
        // base-2 argument (constants times -log2 e); e^{-2u} = inf gives s = 0, e^{-2u} = 0 gives s = 1.
        const float x2 = x * x;
        const float w = x * fmaf(x2, -0.102943241f, -2.302208198f);
        const float s = __fdividef(1.0f, 1.0f + __builtin_amdgcn_exp2f(w));
        value = x * s;
        deriv = fmaf(value * (1.0f - s), fmaf(x2, 0.214064448f, 1.59576912f), s);
      }
      break;
    }
    case LT_ACT_GELU: {
      float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
      float pdf = (PRECISE ? expf(-0.5f * x * x) : __expf(-0.5f * x * x)) * 0.39894228040143268f;
      value = x * cdf;
      deriv = cdf + x * pdf;
      break;
    }
    case LT_ACT_RELU:
      value = x > 0.0f ? x : 0.0f;
      deriv = x > 0.0f ? 1.0f : 0.0f;
      break;
    case LT_ACT_SILU: {
      float s = lt_sigmoid<PRECISE>(x);
      value = x * s;
      deriv = s * (1.0f + x * (1.0f - s));
      break;
    }
    // The remaining closed-form entries of the Hugging Face activation table (the table the reference extends,
    // lean_transformer/utils.py:80).  They run through the general epilogue strips; libm-grade functions throughout.
    case LT_ACT_QUICK_GELU: {
      float s = lt_sigmoid<PRECISE>(1.702f * x);
      value = x * s;
      deriv = s + 1.702f * x * s * (1.0f - s);
      break;
    }
    case LT_ACT_GELU_10: {  // clip(gelu(x), -10, 10): the clip passes gradients where gelu(x) lies inside the interval
      float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
      float g = x * cdf;
      value = fminf(fmaxf(g, -10.0f), 10.0f);
      deriv = (g >= -10.0f && g <= 10.0f) ? cdf + x * expf(-0.5f * x * x) * 0.39894228040143268f : 0.0f;
      break;
    }
    case LT_ACT_RELU6:
      value = fminf(fmaxf(x, 0.0f), 6.0f);
      deriv = (x > 0.0f && x < 6.0f) ? 1.0f : 0.0f;
      break;
    case LT_ACT_RELU2: {
      float r = x > 0.0f ? x : 0.0f;
      value = r * r;
      deriv = 2.0f * r;
      break;
    }
    case LT_ACT_LEAKY_RELU:  // negative slope 0.01 (torch.nn.LeakyReLU's default, the table's entry)
      value = x > 0.0f ? x : 0.01f * x;
      deriv = x > 0.0f ? 1.0f : 0.01f;
      break;
    case LT_ACT_MISH: {  // x tanh(softplus(x)); softplus(x) = x beyond 20 like torch's
      float sp = x > 20.0f ? x : log1pf(expf(x));
      float t = tanhf(sp);
      value = x * t;
      deriv = t + x * (1.0f - t * t) * lt_sigmoid<true>(x);
      break;
    }
    case LT_ACT_SIGMOID: {
      float s = lt_sigmoid<true>(x);
      value = s;
      deriv = s * (1.0f - s);
      break;
    }
    case LT_ACT_TANH: {
      float t = tanhf(x);
      value = t;
      deriv = 1.0f - t * t;
      break;
    }
    case LT_ACT_LINEAR:
      value = x;
      deriv = 1.0f;
      break;
    case LT_ACT_HARDSWISH:
      value = x * fminf(fmaxf(x + 3.0f, 0.0f), 6.0f) * (1.0f / 6.0f);
      deriv = x < -3.0f ? 0.0f : (x <= 3.0f ? x * (1.0f / 3.0f) + 0.5f : 1.0f);
      break;
    case LT_ACT_LAPLACE: {  // 0.5 (1 + erf((x - mu) / (sigma sqrt 2))), mu = 0.707107, sigma = 0.282095
      const float inv = 1.0f / (0.282095f * 1.41421356237f);
      float z = (x - 0.707107f) * inv;
      value = 0.5f * (1.0f + erff(z));
      deriv = expf(-z * z) * inv * 0.56418958354775629f;  // 1 / sqrt(pi)
      break;
    }
    default: {  // LT_ACT_SQRT_SOFTPLUS
      float sp = x > 20.0f ? x : log1pf(expf(x));
      value = sqrtf(sp);
      deriv = value > 0.0f ? lt_sigmoid<true>(x) / (2.0f * value) : 0.0f;  // softplus underflows to 0 far in the negative tail
      break;
    }
  }
}
template <bool PRECISE> __device__ __forceinline__ float act_value(int act, float x) {
  float v, d;
  act_eval<PRECISE>(act, x, v, d);
  return v;
}

// ---------------------------------------------------------------------------------------------------------------------
// Philox4x32-10 counter-based generator: element e of a [T, H] tensor uses word (e & 3) of block counter (e >> 2) in the
// stream (seed, offset).  Forward epilogue and backward replay evaluate the same function, so no mask is stored.
// ---------------------------------------------------------------------------------------------------------------------
struct DropoutParams {
  float p;            // drop probability, 0 = off
  float scale;        // 1 / (1 - p)
  uint32_t threshold; // keep iff random word >= threshold  (threshold = p * 2^32)
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
};

static inline DropoutParams make_dropout(float p, uint64_t seed, uint64_t offset) {
  DropoutParams d;
  d.p = p;
  d.scale = p > 0.f ? 1.0f / (1.0f - p) : 1.0f;
  double t = (double)p * 4294967296.0;
  d.threshold = t >= 4294967295.0 ? 4294967295u : (uint32_t)t;
  d.seed_lo = (uint32_t)seed;
  d.seed_hi = (uint32_t)(seed >> 32);
  d.off_lo = (uint32_t)offset;
  d.off_hi = (uint32_t)(offset >> 32);
  return d;
}

__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                              uint32_t (&out)[4]) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// keep decision of one element
__device__ __forceinline__ bool dropout_keep(const DropoutParams& d, int64_t elem) {
  uint64_t blk = (uint64_t)elem >> 2;
  uint32_t r[4];
  philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi, r);
  return r[elem & 3] >= d.threshold;
}
// keep decisions of 4 consecutive elements starting at a multiple of 4
__device__ __forceinline__ void dropout_keep4(const DropoutParams& d, int64_t elem4, bool (&keep)[4]) {
  uint64_t blk = (uint64_t)elem4 >> 2;
  uint32_t r[4];
  philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi, r);
#pragma unroll
  for (int i = 0; i < 4; i++) keep[i] = r[i] >= d.threshold;
}
