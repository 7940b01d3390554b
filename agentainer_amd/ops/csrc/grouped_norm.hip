// Residual update fused with grouped RMS norms (gfx950), fp32 residual.
//
//   x      <- x + mult * (a + b)            (a, b optional)
//   out_k  <- x / sqrt(mean_g(x^2) + eps) * w_k      k = 1 (, 2)
//
// mean_g runs over each of `groups` equal consecutive parts of the row on
// its own. The residual x stays fp32 in HBM; a, b and the outputs carry
// the compute dtype T. One 256-thread workgroup per row walks the groups
// in turn: pass 1 updates x and accumulates the group's sum of squares,
// a block reduction yields the group's 1/rms, pass 2 re-reads the values
// the SAME threads just wrote (L1/L2 hits) and emits both normed outputs —
// the two norms a parallel-residual layer needs cost one read of x.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

template <typename T, int VEC>
__global__ __launch_bounds__(256) void residual_gnorm_kernel(
    float* __restrict__ x, const T* __restrict__ a, long a_rs,
    const T* __restrict__ b, long b_rs, float mult,
    const float* __restrict__ w1, T* __restrict__ o1,
    const float* __restrict__ w2, T* __restrict__ o2, int W, int groups,
    float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int Wg = W / groups;
  float* xr = x + row * W;
  for (int g = 0; g < groups; ++g) {
    const int c0 = g * Wg;
    float ss = 0.f;
    for (int i = threadIdx.x * VEC; i < Wg; i += 256 * VEC) {
      float v[VEC];
      if constexpr (VEC == 4) {
        ld4(xr, c0 + i, v);
      } else {
        v[0] = xr[c0 + i];
      }
      if (a != nullptr) {
        float s[VEC];
        if constexpr (VEC == 4) {
          ld4(a, row * a_rs + c0 + i, s);
        } else {
          s[0] = ldf(a, row * a_rs + c0 + i);
        }
        if (b != nullptr) {
          float t[VEC];
          if constexpr (VEC == 4) {
            ld4(b, row * b_rs + c0 + i, t);
          } else {
            t[0] = ldf(b, row * b_rs + c0 + i);
          }
#pragma unroll
          for (int j = 0; j < VEC; ++j) s[j] += t[j];
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = fmaf(mult, s[j], v[j]);
        if constexpr (VEC == 4) {
          st4(xr, c0 + i, v);
        } else {
          xr[c0 + i] = v[0];
        }
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
    }
    const float tot = block_sum_256(ss, red);
    const float r = 1.0f / sqrtf(tot / (float)Wg + eps);
    for (int i = threadIdx.x * VEC; i < Wg; i += 256 * VEC) {
      float v[VEC], wv[VEC], o[VEC];
      if constexpr (VEC == 4) {
        ld4(xr, c0 + i, v);
        ld4(w1, c0 + i, wv);
      } else {
        v[0] = xr[c0 + i];
        wv[0] = w1[c0 + i];
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = v[j] * r * wv[j];
      if constexpr (VEC == 4) {
        st4(o1, row * W + c0 + i, o);
      } else {
        stf(o1, row * W + c0 + i, o[0]);
      }
      if (o2 != nullptr) {
        if constexpr (VEC == 4) {
          ld4(w2, c0 + i, wv);
        } else {
          wv[0] = w2[c0 + i];
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = v[j] * r * wv[j];
        if constexpr (VEC == 4) {
          st4(o2, row * W + c0 + i, o);
        } else {
          stf(o2, row * W + c0 + i, o[0]);
        }
      }
    }
  }
}

}  // namespace

void residual_grouped_rmsnorm(torch::Tensor x, c10::optional<torch::Tensor> a,
                              c10::optional<torch::Tensor> b, double mult,
                              torch::Tensor w1, torch::Tensor o1,
                              c10::optional<torch::Tensor> w2,
                              c10::optional<torch::Tensor> o2, long groups,
                              double eps) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2, "residual stream must be contiguous fp32 [T, W]");
  const int T_ = x.size(0), W = x.size(1);
  TORCH_CHECK(groups >= 1 && W % groups == 0, "width % groups != 0");
  TORCH_CHECK(w1.scalar_type() == at::kFloat && w1.numel() == W &&
              w1.is_contiguous());
  TORCH_CHECK(o1.is_contiguous() && o1.size(0) == T_ && o1.size(1) == W);
  TORCH_CHECK(!b.has_value() || a.has_value(), "b without a");
  TORCH_CHECK(w2.has_value() == o2.has_value());
  if (o2.has_value()) {
    TORCH_CHECK(o2->is_contiguous() && o2->scalar_type() == o1.scalar_type() &&
                o2->size(0) == T_ && o2->size(1) == W);
    TORCH_CHECK(w2->scalar_type() == at::kFloat && w2->numel() == W &&
                w2->is_contiguous());
  }
  long a_rs = 0, b_rs = 0;
  if (a.has_value()) {
    TORCH_CHECK(a->scalar_type() == o1.scalar_type() && a->dim() == 2 &&
                a->size(0) == T_ && a->size(1) == W && a->stride(1) == 1);
    a_rs = a->stride(0);
  }
  if (b.has_value()) {
    TORCH_CHECK(b->scalar_type() == o1.scalar_type() && b->dim() == 2 &&
                b->size(0) == T_ && b->size(1) == W && b->stride(1) == 1);
    b_rs = b->stride(0);
  }
  if (T_ == 0) return;
  const int Wg = W / groups;
  const bool vec = (Wg % 4 == 0) && (a_rs % 4 == 0) && (b_rs % 4 == 0);
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(o1, {
    const T* ap = a.has_value() ? (const T*)a->data_ptr() : nullptr;
    const T* bp = b.has_value() ? (const T*)b->data_ptr() : nullptr;
    const float* w2p = w2.has_value() ? w2->data_ptr<float>() : nullptr;
    T* o2p = o2.has_value() ? (T*)o2->data_ptr() : nullptr;
    if (vec) {
      hipLaunchKernelGGL((residual_gnorm_kernel<T, 4>), dim3(T_), dim3(256), 0,
                         stream, x.data_ptr<float>(), ap, a_rs, bp, b_rs,
                         (float)mult, w1.data_ptr<float>(), (T*)o1.data_ptr(),
                         w2p, o2p, W, (int)groups, (float)eps);
    } else {
      hipLaunchKernelGGL((residual_gnorm_kernel<T, 1>), dim3(T_), dim3(256), 0,
                         stream, x.data_ptr<float>(), ap, a_rs, bp, b_rs,
                         (float)mult, w1.data_ptr<float>(), (T*)o1.data_ptr(),
                         w2p, o2p, W, (int)groups, (float)eps);
    }
  });
}
