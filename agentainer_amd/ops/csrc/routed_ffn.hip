// Gated feed-forward activations and the sigmoid top-k router (gfx950).
//
//   act_mul:                out = act(gate) * up, act in {relu, silu}
//   sigmoid_topk_route:     weight[t, e] = sigmoid(z[t, e]) for the `top`
//                           largest scores of row t, 0 elsewhere (fp32)
//   routed_scaled_silu_mul: stacked-expert activation with the routing
//                           weight on the expert INPUT: the gate|up GEMM
//                           ran on the unscaled input, so the projections
//                           of the scaled input are w*g and w*u:
//                           out[t, e, f] = silu(w g) * (w u); experts with
//                           w == 0 write 0 without reading their columns.
//
// All three are memory-bound elementwise passes, 4 elements per lane.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

template <typename T, int VEC>
__global__ void act_mul_kernel(T* __restrict__ out, const T* __restrict__ gate,
                               const T* __restrict__ up, long n, int Hc,
                               long gs, long us, int act) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long row = i / Hc;
  const int col = (int)(i % Hc);
  float g[VEC], u[VEC], o[VEC];
  if constexpr (VEC == 4) {
    ld4(gate, row * gs + col, g);
    ld4(up, row * us + col, u);
  } else {
    g[0] = ldf(gate, row * gs + col);
    u[0] = ldf(up, row * us + col);
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const float a = act == 0 ? fmaxf(g[j], 0.f) : g[j] / (1.0f + expf(-g[j]));
    o[j] = a * u[j];
  }
  if constexpr (VEC == 4) {
    st4(out, i, o);
  } else {
    stf(out, i, o[0]);
  }
}

constexpr int ROUTE_PER_LANE = 16;  // experts <= 64 * 16

// one wave per token row
__global__ __launch_bounds__(64) void sigmoid_topk_kernel(
    float* __restrict__ weight, const float* __restrict__ logits, int E,
    int top) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  float s[ROUTE_PER_LANE];
  bool taken[ROUTE_PER_LANE];
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    taken[k] = false;
    s[k] = e < E ? 1.0f / (1.0f + expf(-logits[t * E + e])) : -1.0f;
  }
  for (int r = 0; r < top; ++r) {
    // lane-local best (lowest index wins ties), then across the wave
    float bv = -2.0f;
    int be = 0x7fffffff;
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) {
      const int e = k * WAVE + lane;
      if (e < E && !taken[k] && s[k] > bv) { bv = s[k]; be = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, WAVE);
      const int oe = __shfl_xor(be, off, WAVE);
      if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
    }
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k)
      if (k * WAVE + lane == be) taken[k] = true;
  }
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    if (e < E) weight[t * E + e] = taken[k] ? s[k] : 0.f;
  }
}

template <typename T, int VEC>
__global__ void routed_silu_kernel(T* __restrict__ out,
                                   const T* __restrict__ gu,
                                   const float* __restrict__ weight, long n,
                                   int E, int F, long gu_rs) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long t = i / ((long)E * F);
  const int rem = (int)(i % ((long)E * F));
  const int e = rem / F, f = rem % F;
  const float w = weight[t * E + e];
  float o[VEC];
  if (w == 0.f) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = 0.f;
  } else {
    float g[VEC], u[VEC];
    const long base = t * gu_rs + (long)e * 2 * F + f;
    if constexpr (VEC == 4) {
      ld4(gu, base, g);
      ld4(gu, base + F, u);
    } else {
      g[0] = ldf(gu, base);
      u[0] = ldf(gu, base + F);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float gs = w * g[j];
      o[j] = gs / (1.0f + expf(-gs)) * (w * u[j]);
    }
  }
  if constexpr (VEC == 4) {
    st4(out, i, o);
  } else {
    stf(out, i, o[0]);
  }
}

}  // namespace

void act_mul(torch::Tensor out, torch::Tensor gate, torch::Tensor up,
             long act) {
  TORCH_CHECK(out.is_contiguous() && gate.dim() == 2 && up.dim() == 2);
  TORCH_CHECK(gate.stride(1) == 1 && up.stride(1) == 1);
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() &&
              up.scalar_type() == out.scalar_type());
  const int T_ = gate.size(0), Hc = gate.size(1);
  TORCH_CHECK(up.size(0) == T_ && up.size(1) == Hc && out.numel() == (long)T_ * Hc);
  TORCH_CHECK(act == 0 || act == 1);
  const long n = (long)T_ * Hc;
  if (n == 0) return;
  const bool vec = Hc % 4 == 0 && gate.stride(0) % 4 == 0 &&
                   up.stride(0) % 4 == 0 && gate.storage_offset() % 4 == 0 &&
                   up.storage_offset() % 4 == 0;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((act_mul_kernel<T, 4>), dim3((n / 4 + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gate.data_ptr(), (const T*)up.data_ptr(), n,
                         Hc, (long)gate.stride(0), (long)up.stride(0), (int)act);
    } else {
      hipLaunchKernelGGL((act_mul_kernel<T, 1>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gate.data_ptr(), (const T*)up.data_ptr(), n,
                         Hc, (long)gate.stride(0), (long)up.stride(0), (int)act);
    }
  });
}

void sigmoid_topk_route(torch::Tensor weight, torch::Tensor logits, long top) {
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.is_contiguous());
  TORCH_CHECK(logits.scalar_type() == at::kFloat && logits.is_contiguous() &&
              logits.dim() == 2);
  const int T_ = logits.size(0), E = logits.size(1);
  TORCH_CHECK(weight.numel() == (long)T_ * E);
  TORCH_CHECK(E <= WAVE * ROUTE_PER_LANE, "too many experts");
  TORCH_CHECK(top >= 1 && top <= E, "top out of range");
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL(sigmoid_topk_kernel, dim3(T_), dim3(64), 0, stream,
                     weight.data_ptr<float>(), logits.data_ptr<float>(), E,
                     (int)top);
}

void routed_scaled_silu_mul(torch::Tensor out, torch::Tensor gu,
                            torch::Tensor weight) {
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && gu.dim() == 2 &&
              gu.stride(1) == 1 && gu.scalar_type() == out.scalar_type());
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.is_contiguous() &&
              weight.dim() == 2);
  const int T_ = out.size(0), E = weight.size(1);
  TORCH_CHECK(weight.size(0) == T_ && gu.size(0) == T_);
  TORCH_CHECK(out.size(1) % E == 0);
  const int F = out.size(1) / E;
  TORCH_CHECK(gu.size(1) == (long)2 * E * F, "gate|up width mismatch");
  const long n = (long)T_ * E * F;
  if (n == 0) return;
  const bool vec = F % 4 == 0 && gu.stride(0) % 4 == 0 &&
                   gu.storage_offset() % 4 == 0;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((routed_silu_kernel<T, 4>), dim3((n / 4 + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(), n,
                         E, F, (long)gu.stride(0));
    } else {
      hipLaunchKernelGGL((routed_silu_kernel<T, 1>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(), n,
                         E, F, (long)gu.stride(0));
    }
  });
}
