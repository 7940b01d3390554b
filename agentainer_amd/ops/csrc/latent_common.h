// Typed element access shared by the grouped-norm, latent-attention and
// routed-expert kernels: every kernel is written once over an element
// type T (short = bf16 bits, float = fp32) and does its math in fp32.
#pragma once

#include "common.h"

__device__ __forceinline__ float ldf(const float* p, long i) { return p[i]; }
__device__ __forceinline__ float ldf(const short* p, long i) {
  return bits2f(p[i]);
}
__device__ __forceinline__ void stf(float* p, long i, float v) { p[i] = v; }
__device__ __forceinline__ void stf(short* p, long i, float v) {
  p[i] = f2bits(v);
}

// 4 consecutive elements (caller guarantees 4-element alignment)
__device__ __forceinline__ void ld4(const float* p, long i, float* v) {
  const float4 t = *reinterpret_cast<const float4*>(p + i);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void ld4(const short* p, long i, float* v) {
  const bf16x4 t = *reinterpret_cast<const bf16x4*>(p + i);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = bits2f(t[j]);
}
__device__ __forceinline__ void st4(float* p, long i, const float* v) {
  *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(short* p, long i, const float* v) {
  bf16x4 t;
#pragma unroll
  for (int j = 0; j < 4; ++j) t[j] = f2bits(v[j]);
  *reinterpret_cast<bf16x4*>(p + i) = t;
}

// sum over a 256-thread block (4 waves); red = 4 floats of LDS
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = v;
  __syncthreads();
  const float t = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return t;
}

#define LATENT_DISPATCH_T(tensor, ...)                                         \
  do {                                                                         \
    if ((tensor).scalar_type() == at::kBFloat16) {                             \
      using T = short;                                                         \
      __VA_ARGS__;                                                             \
    } else {                                                                   \
      TORCH_CHECK((tensor).scalar_type() == at::kFloat,                        \
                  "expected a bf16 or fp32 tensor");                           \
      using T = float;                                                         \
      __VA_ARGS__;                                                             \
    }                                                                          \
  } while (0)
