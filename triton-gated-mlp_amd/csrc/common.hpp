// Shared device helpers for the gfx950 gated-MLP kernels: storage types, MFMA wrappers,
// fp32 SiLU, and the Philox4x32-10 counter RNG that defines the dropout mask.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gmlp {

typedef _Float16 f16;
typedef __bf16 bf16;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Per-dtype traits.  mfma = v_mfma_f32_32x32x16, mfma16 = v_mfma_f32_16x16x32 (4 accumulator floats
// per lane: column l % 16, rows 4*(l/16) .. +3).  An operand fragment of v_mfma_f32_32x32x16_{f16,bf16} is 8 consecutive
// reduction elements per lane: lane l carries row (l % 32), reduction slots 8*(l / 32) .. +7.
// The 16 accumulator floats of lane l sit at column (l % 32), rows 8*(i/4) + 4*(l/32) + (i%4).
template <typename T>
struct Traits;

template <>
struct Traits<f16> {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(f16 v) { return (float)v; }
  static __device__ __forceinline__ f16 from_f32(float v) { return (f16)v; }
};

template <>
struct Traits<bf16> {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }
  static __device__ __forceinline__ bf16 from_f32(float v) { return (bf16)v; }
};

template <>
struct Traits<float> {
  typedef float vec8 __attribute__((ext_vector_type(8)));
  typedef float vec4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ float to_f32(float v) { return v; }
  static __device__ __forceinline__ float from_f32(float v) { return v; }
};

// sigma(x) = 1/(1+e^-x), silu(x) = x*sigma(x), silu'(x) = sigma*(1 + x*(1-sigma)); all fp32.
// Same forms as the reference's _compute_sigma/_silu_fwd/_silu_bwd (src/triton_gated_mlp/ops/act.py:28-45).
// Reciprocals are the hardware's v_rcp_f32 (1 ulp): a plain `1.0f / y` compiles to the IEEE division
// sequence of eleven instructions, which made the activation arithmetic the longest part of the
// fused epilogues.
__device__ __forceinline__ float rcp_f32(float y) { return __builtin_amdgcn_rcpf(y); }
__device__ __forceinline__ float sigmoid_f32(float x) { return rcp_f32(1.0f + __expf(-x)); }
__device__ __forceinline__ float silu_f32(float x) { return x * sigmoid_f32(x); }
__device__ __forceinline__ float silu_grad_f32(float x) {
  float s = sigmoid_f32(x);
  return s * (1.0f + x * (1.0f - s));
}

// Phi(x) = (1 + erf(x/sqrt 2))/2 through Abramowitz & Stegun 7.1.26, erfc(z) = poly(t) e^{-z^2} with
// t = 1/(1 + p z) for z >= 0 (|error| <= 1.5e-7 on erf, so <= 3e-7 on Phi with fp32 rounding: three
// orders below fp16/bf16 resolution).  One exp and one reciprocal per value instead of libm's
// two-branch erff, and e^{-x^2/2} is shared with the normal density the derivative needs.  The
// lower tail comes out as a product rather than as 1 + erf, so it does not cancel.
struct NormalCdf {
  float cdf, e;  // Phi(x), e^{-x^2/2}
};
__device__ __forceinline__ NormalCdf normal_cdf_f32(float x) {
  const float ax = fabsf(x);
  const float t = rcp_f32(1.0f + 0.23164189f * ax);  // p / sqrt 2, p = 0.3275911
  const float e = __expf(-0.5f * x * x);
  float poly = 1.061405429f;
  poly = poly * t - 1.453152027f;
  poly = poly * t + 1.421413741f;
  poly = poly * t - 0.284496736f;
  poly = poly * t + 0.254829592f;
  const float q = 0.5f * poly * t * e;
  return {x < 0.f ? q : 1.0f - q, e};
}
// tanh(x) = sign(x) (1 - e)/(1 + e), e = e^{-2|x|}; below 1/4 the odd series to x^7 (next term
// 62/2835 x^9 < 2e-7 relative) replaces the cancelling 1 - e.  Relative error < 5e-7.
__device__ __forceinline__ float tanh_f32(float x) {
  const float ax = fabsf(x), x2 = x * x;
  const float e = __expf(-2.0f * ax);
  const float big = (1.0f - e) * rcp_f32(1.0f + e);
  const float small = ax * (1.0f + x2 * (-0.33333333f + x2 * (0.13333333f - x2 * 0.053968254f)));
  return copysignf(ax < 0.25f ? small : big, x);
}

// Gate activations.  The codes are the GMLP_ACT_* values of the C interface; the functions are the
// ones the reference's eager module offers for hidden_act (ACT2CLS / ACT_FWD,
// src/triton_gated_mlp/gated_mlp.py:17-37) with torch's default parameters: exact (erf) GELU,
// LeakyReLU slope 0.01.  Derivatives follow torch.autograd at the kinks: relu'(0) = 0,
// leaky_relu'(0) = 0.01.  Everything is evaluated in fp32.
enum Act : int {
  ACT_SILU = 0,
  ACT_GELU = 1,
  ACT_RELU = 2,
  ACT_LEAKY_RELU = 3,
  ACT_SIGMOID = 4,
  ACT_TANH = 5,
  ACT_IDENTITY = 6,
  ACT_COUNT = 7
};
constexpr float LEAKY_SLOPE = 0.01f;

// y[r] = act(x[r]) for W values; `act` is uniform over the wavefront, so the switch is a scalar
// branch taken once per call.  ACT >= 0 fixes the activation at compile time (`act` is ignored and
// the other cases are not emitted); ACT_RUNTIME keeps the switch.
constexpr int ACT_RUNTIME = -1;
template <int W, int ACT = ACT_RUNTIME>
__device__ __forceinline__ void act_fwd_w(int act, const float* x, float* y) {
  switch (ACT >= 0 ? ACT : act) {
    case ACT_SILU:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = silu_f32(x[r]);
      break;
    case ACT_GELU:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = x[r] * normal_cdf_f32(x[r]).cdf;
      break;
    case ACT_RELU:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = x[r] < 0.f ? 0.f : x[r];
      break;
    case ACT_LEAKY_RELU:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = x[r] < 0.f ? LEAKY_SLOPE * x[r] : x[r];
      break;
    case ACT_SIGMOID:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = sigmoid_f32(x[r]);
      break;
    case ACT_TANH:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = tanh_f32(x[r]);
      break;
    default:
#pragma unroll
      for (int r = 0; r < W; ++r) y[r] = x[r];
      break;
  }
}

// y[r] = act(x[r]) and d[r] = act'(x[r]).
template <int W, int ACT = ACT_RUNTIME>
__device__ __forceinline__ void act_fwd_grad_w(int act, const float* x, float* y, float* d) {
  switch (ACT >= 0 ? ACT : act) {
    case ACT_SILU:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        float s = sigmoid_f32(x[r]);
        y[r] = x[r] * s;
        d[r] = s * (1.0f + x[r] * (1.0f - s));
      }
      break;
    case ACT_GELU:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        NormalCdf n = normal_cdf_f32(x[r]);
        y[r] = x[r] * n.cdf;
        d[r] = n.cdf + x[r] * (0.39894228040143268f * n.e);
      }
      break;
    case ACT_RELU:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        y[r] = x[r] < 0.f ? 0.f : x[r];
        d[r] = x[r] > 0.f ? 1.f : 0.f;
      }
      break;
    case ACT_LEAKY_RELU:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        y[r] = x[r] < 0.f ? LEAKY_SLOPE * x[r] : x[r];
        d[r] = x[r] > 0.f ? 1.f : LEAKY_SLOPE;
      }
      break;
    case ACT_SIGMOID:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        float s = sigmoid_f32(x[r]);
        y[r] = s;
        d[r] = s * (1.0f - s);
      }
      break;
    case ACT_TANH:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        float t = tanh_f32(x[r]);
        y[r] = t;
        d[r] = 1.0f - t * t;
      }
      break;
    default:
#pragma unroll
      for (int r = 0; r < W; ++r) {
        y[r] = x[r];
        d[r] = 1.0f;
      }
      break;
  }
}

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11).
__host__ __device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2,
                                                        uint32_t c3, uint32_t k0, uint32_t k1,
                                                        uint32_t out[4]) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)M0 * c0;
    uint64_t p1 = (uint64_t)M1 * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

struct DropoutParams {
  uint32_t threshold;  // keep iff word >= threshold; threshold = floor(p * 2^32)
  float scale;         // 1/(1-p)
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  int enabled;
};

// Keep bits for the 4 consecutive elements e4*4 .. e4*4+3 of the flattened [M,N] tensor.
__host__ __device__ __forceinline__ void dropout_keep4(const DropoutParams& d, uint64_t e4,
                                                        bool keep[4]) {
  uint32_t w[4];
  philox4x32_10((uint32_t)e4, (uint32_t)(e4 >> 32), d.off_lo, d.off_hi, d.seed_lo, d.seed_hi, w);
#pragma unroll
  for (int i = 0; i < 4; ++i) keep[i] = w[i] >= d.threshold;
}

}  // namespace gmlp
