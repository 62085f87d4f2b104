// Device helpers shared by the translation units of libgbx_mixers.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "gbx_mixers.h"

namespace gbxm {

typedef unsigned short bf16_t;          // storage type of a bf16 element

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(static_cast<unsigned>(v) << 16); }
// round to nearest even (values here are finite)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const unsigned u = __float_as_uint(f);
  return static_cast<bf16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) { return f32_to_bf16(f); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// sum over a workgroup of NW waves; every thread gets the result; `red` is NW floats of LDS.  Fixed order: deterministic.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();                       // red may still be read from an earlier call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) s += red[i];
  return s;
}

// Transcendentals: exact library forms for fp32 models, hardware approximations (a few ulp) where activations are bf16.
template <bool FAST> __device__ __forceinline__ float exp_(float x) { if constexpr (FAST) return __expf(x); else return expf(x); }
template <bool FAST> __device__ __forceinline__ float sigmoid_(float x) {
  if constexpr (FAST) return __fdividef(1.f, 1.f + __expf(-x)); else return 1.f / (1.f + expf(-x));
}
template <bool FAST> __device__ __forceinline__ float tanh_(float x) {
  if constexpr (FAST) { const float e = __expf(2.f * x); return 1.f - __fdividef(2.f, e + 1.f); } else return tanhf(x);
}
// Gated activations of feed-forwards (GBXM_GLU_*): silu(g) u, gelu(g) u in the tanh form, sigmoid(g) u, or the clamped form
// g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit).
template <bool FAST> __device__ __forceinline__ float glu_act(float g, float u, int kind, float limit, float alpha) {
  if (kind == GBXM_GLU_CLAMPED_SWISH) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_<FAST>(alpha * g) * (u + 1.f);
  }
  if (kind == GBXM_GLU_GELU_TANH) return 0.5f * g * (1.f + tanh_<FAST>(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
  if (kind == GBXM_GLU_SIGMOID) return sigmoid_<FAST>(g) * u;
  return g * sigmoid_<FAST>(g) * u;
}
template <bool FAST> __device__ __forceinline__ float log1p_(float x) { if constexpr (FAST) return __logf(1.f + x); else return log1pf(x); }

// floats per (split, row, head) of the key-split partial sums of softmax attention: dv sums padded to a multiple of four (rows stay
// 16-byte aligned), then two more pairs of which the last holds (running maximum, denominator)
__host__ __device__ __forceinline__ int partial_width(int dv) { return (dv + 3) / 4 * 4 + 4; }

extern thread_local char g_err[512];
int fail(int code, const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);
inline int after_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? GBXM_OK : hip_fail(e, what);
}

}  // namespace gbxm
