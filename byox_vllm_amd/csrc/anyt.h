// Element access for kernels that run in either 16-bit or true 32-bit storage (dtype NV_BF16 / NV_F32): loads widen
// to float, stores round to nearest even.  The arithmetic of these kernels is fp32 in both cases.
#pragma once
#include "common.h"

template <typename T> __device__ __forceinline__ float ld_f32(const T* p);
template <> __device__ __forceinline__ float ld_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_f32<bf16_t>(const bf16_t* p) {
  return __uint_as_float(((uint32_t) * reinterpret_cast<const uint16_t*>(p)) << 16);
}
template <typename T> __device__ __forceinline__ void st_f32(T* p, float v);
template <> __device__ __forceinline__ void st_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f32<bf16_t>(bf16_t* p, float v) { *p = (bf16_t)v; }

// value rounded to the storage type and widened again (what a consumer of a stored T would read)
template <typename T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<bf16_t>(float v) { return (float)(bf16_t)v; }

__device__ __forceinline__ float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f32(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f32(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// Gated unit act(gate) * up.  act 0: SiLU, 1: tanh-form GELU, 2: the clamped form with limit c,
// g = min(gate, c), u = clamp(up, -c, c), g * sigmoid(1.702 g) * (u + 1).
__device__ __forceinline__ float glu_act(float g, float u, int act, float c) {
  if (act == 2) {
    g = fminf(g, c);
    u = fminf(fmaxf(u, -c), c);
    return g * sigmoid_f32(1.702f * g) * (u + 1.0f);
  }
  return (act == 1 ? gelu_tanh_f32(g) : silu_f32(g)) * u;
}
// log(sigmoid(z)) without cancellation: -softplus(-z)
__device__ __forceinline__ float log_sigmoid_f32(float z) {
  return z >= 0.0f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

// Sum / maximum over a workgroup of up to 1024 threads; `red` holds at least 32 floats of LDS.  Every thread gets
// the result; the routine ends with the LDS free for reuse.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.0f;
  for (int i = 0; i < nw; ++i) s += red[i];
  return s;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = red[0];
  for (int i = 1; i < nw; ++i) s = fmaxf(s, red[i]);
  return s;
}

#define NV_DISPATCH_T(dtype, ...)                      \
  do {                                                 \
    if ((dtype) == NV_BF16) {                          \
      typedef bf16_t T;                                \
      __VA_ARGS__;                                     \
    } else {                                           \
      typedef float T;                                 \
      __VA_ARGS__;                                     \
    }                                                  \
  } while (0)
