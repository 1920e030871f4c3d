// Shared device helpers for the gfx950 MoE-FFN kernels: element-type traits, bf16 conversion with
// PyTorch's rounding (round-to-nearest-even, canonical NaN), activations, wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/d2dmoe.h"

namespace d2dmoe {

constexpr int kWave = 64;  // CDNA wavefront width

// ---------------------------------------------------------------- bf16 <-> f32 -----------------
typedef uint16_t bf16_t;  // raw bits

__host__ __device__ inline float bf16_to_f32(bf16_t v) {
  union { uint32_t u; float f; } c;
  c.u = ((uint32_t)v) << 16;
  return c.f;
}

// round-to-nearest-even; NaN -> 0x7FC0 (what c10::BFloat16 produces)
__host__ __device__ inline bf16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7FC0;
  uint32_t bias = 0x7fffu + ((c.u >> 16) & 1u);
  return (bf16_t)((c.u + bias) >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int dtype = D2DMOE_F32;
  __device__ static inline float load(const float* p) { return *p; }
  __device__ static inline void store(float* p, float v) { *p = v; }
  __device__ static inline float round(float v) { return v; }
};
template <> struct Elem<bf16_t> {
  static constexpr int dtype = D2DMOE_BF16;
  __device__ static inline float load(const bf16_t* p) { return bf16_to_f32(*p); }
  __device__ static inline void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  __device__ static inline float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};
// IEEE half precision (the reference benches float32 and float16, test_moe_implementations.py:223-228): a type of its
// own, so that it selects its own kernels; conversions round to nearest even, as torch.float16 does
typedef _Float16 f16_t;
template <> struct Elem<f16_t> {
  static constexpr int dtype = D2DMOE_F16;
  __device__ static inline float load(const f16_t* p) { return (float)*p; }
  __device__ static inline void store(f16_t* p, float v) { *p = (f16_t)v; }
  __device__ static inline float round(float v) { return (float)(f16_t)v; }
};
// two values rounded to the 16-bit storage type and packed, low half first
template <typename T> __device__ inline uint32_t pack2_16(float lo, float hi);

// ---------------------------------------------------------------- activations ------------------
// Definitions follow the reference's kernel-side helpers (utils.py:730-756).
__device__ inline float apply_act(int act, float x) {
  switch (act) {
    case D2DMOE_ACT_RELU: return fmaxf(x, 0.f);   // == (x >= 0 ? x : 0), NaN -> 0 as well
    case D2DMOE_ACT_GELU: {
      // erf by the rational approximation of Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7, on the order of
      // float32 rounding): one exp, one reciprocal, five multiply-adds
      const float z = fabsf(x) * 0.70710678118654752440f;
      const float t = __builtin_amdgcn_rcpf(1.f + 0.3275911f * z);
      const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
      const float erf_abs = 1.f - poly * __expf(-z * z);
      return x * 0.5f * (1.f + copysignf(erf_abs, x));
    }
    case D2DMOE_ACT_TANH: return tanhf(x);
    case D2DMOE_ACT_LEAKY_RELU: return x >= 0.f ? x : 0.01f * x;
    case D2DMOE_ACT_GELU_TANH: {
      // 0.5 x (1 + tanh(u)) == x * sigmoid(2u),  u = sqrt(2/pi) (x + 0.044715 x^3): one exp and one reciprocal
      const float k2 = 2.f * 0.79788456080286535588f;
      const float u2 = k2 * (x + 0.044715f * x * x * x);
      return x * __builtin_amdgcn_rcpf(1.f + __expf(-u2));
    }
    case D2DMOE_ACT_SILU: return x * __builtin_amdgcn_rcpf(1.f + __expf(-x));
    case D2DMOE_ACT_ABS: return fabsf(x);
    default: return x;
  }
}

template <int ACT> __device__ inline float act_fn(float x) { return apply_act(ACT, x); }

// ---------------------------------------------------------------- wave64 helpers ---------------
// NaN-propagating maximum (torch.max semantics).
__device__ inline float nanmax(float a, float b) { return (a > b || a != a) ? a : b; }

__device__ inline float wave_nanmax(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = nanmax(v, __shfl_xor(v, off, kWave));
  return v;
}

__device__ inline int wave_sum_i32(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace d2dmoe
