// Scalar-gain RMS norms and the PolyNorm activation (gfx950).
//
//   scalar_postnorm_residual   x(fp32) += g * y / sqrt(mean(y^2) + eps);
//                              h = T(x)           (post-norm residual step)
//   scalar_rmsnorm             out = T(g * x / sqrt(mean(x^2) + eps))
//   poly_norm                  out = a U(z) + b U(z^2) + c U(z^3) + e,
//                              U(v) = v / sqrt(mean(v^2) + eps) per row
//
// g is ONE number per norm and lives in device memory (no host read). All
// statistics and the residual are fp32; y, z, h and out carry the compute
// dtype T. One 256-thread workgroup per row: pass 1 accumulates the sums,
// pass 2 re-reads the row the same threads just read (L1/L2 hits) and
// writes. The residual update, the norm, the gain and the cast that feeds
// the next GEMM are one kernel, one read of y and one read+write of x.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

template <typename T, int VEC>
__device__ __forceinline__ void ldv(const T* p, long i, float* v) {
  if constexpr (VEC == 4) {
    ld4(p, i, v);
  } else {
    v[0] = ldf(p, i);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void stv(T* p, long i, const float* v) {
  if constexpr (VEC == 4) {
    st4(p, i, v);
  } else {
    stf(p, i, v[0]);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void scalar_postnorm_residual_kernel(
    float* __restrict__ x, const T* __restrict__ y, long y_rs,
    const float* __restrict__ gain, float eps, T* __restrict__ h, int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const T* yr = y + row * y_rs;
  float ss = 0.f;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float v[VEC];
    ldv<T, VEC>(yr, i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
  }
  const float r = gain[0] / sqrtf(block_sum_256(ss, red) / (float)W + eps);
  float* xr = x + row * W;
  T* hr = h + row * W;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float v[VEC], xv[VEC];
    ldv<T, VEC>(yr, i, v);
    ldv<float, VEC>(xr, i, xv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) xv[j] = fmaf(v[j], r, xv[j]);
    stv<float, VEC>(xr, i, xv);
    stv<T, VEC>(hr, i, xv);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void scalar_rmsnorm_kernel(
    T* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ gain, float eps, int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const float* xr = x + row * W;
  float ss = 0.f;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float v[VEC];
    ldv<float, VEC>(xr, i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
  }
  const float r = gain[0] / sqrtf(block_sum_256(ss, red) / (float)W + eps);
  T* orow = out + row * W;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float v[VEC];
    ldv<float, VEC>(xr, i, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] *= r;
    stv<T, VEC>(orow, i, v);
  }
}

// MAXC > 0: the row (F <= 256 * VEC * MAXC values) is held in registers
// between the two passes, so z is read from memory once; MAXC == 0 re-reads.
template <typename T, int VEC, int MAXC>
__global__ __launch_bounds__(256) void poly_norm_kernel(
    T* __restrict__ out, const T* __restrict__ z, long z_rs,
    const float* __restrict__ coef, float eps, int F) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const T* zr = z + row * z_rs;
  constexpr int NC = MAXC > 0 ? MAXC : 1;
  float keep[NC][VEC];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  if constexpr (MAXC > 0) {
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int i = (c * 256 + threadIdx.x) * VEC;
      if (i < F) {
        ldv<T, VEC>(zr, i, keep[c]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float q = keep[c][j] * keep[c][j];
          s2 += q;
          s4 = fmaf(q, q, s4);
          s6 = fmaf(q * keep[c][j], q * keep[c][j], s6);
        }
      }
    }
  } else {
    for (int i = threadIdx.x * VEC; i < F; i += 256 * VEC) {
      float v[VEC];
      ldv<T, VEC>(zr, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float q = v[j] * v[j];
        s2 += q;
        s4 = fmaf(q, q, s4);
        s6 = fmaf(q * v[j], q * v[j], s6);
      }
    }
  }
  const float n = (float)F;
  const float r1 = coef[0] / sqrtf(block_sum_256(s2, red) / n + eps);
  const float r2 = coef[1] / sqrtf(block_sum_256(s4, red) / n + eps);
  const float r3 = coef[2] / sqrtf(block_sum_256(s6, red) / n + eps);
  const float e = coef[3];
  T* orow = out + row * F;
  if constexpr (MAXC > 0) {
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int i = (c * 256 + threadIdx.x) * VEC;
      if (i < F) {
        float v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float x = keep[c][j], q = x * x;
          v[j] = fmaf(x, r1, fmaf(q, r2, fmaf(q * x, r3, e)));
        }
        stv<T, VEC>(orow, i, v);
      }
    }
  } else {
    for (int i = threadIdx.x * VEC; i < F; i += 256 * VEC) {
      float v[VEC];
      ldv<T, VEC>(zr, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float q = v[j] * v[j];
        v[j] = fmaf(v[j], r1, fmaf(q, r2, fmaf(q * v[j], r3, e)));
      }
      stv<T, VEC>(orow, i, v);
    }
  }
}

bool aligned16(const torch::Tensor& t) {
  return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0;
}

}  // namespace

void scalar_postnorm_residual(torch::Tensor x, torch::Tensor y,
                              torch::Tensor gain, double eps, torch::Tensor h) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2, "residual stream must be contiguous fp32 [T, W]");
  const int T_ = x.size(0), W = x.size(1);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == T_ && y.size(1) == W &&
              y.stride(1) == 1, "y must be [T, W] with unit column stride");
  TORCH_CHECK(h.is_contiguous() && h.dim() == 2 && h.size(0) == T_ &&
              h.size(1) == W && h.scalar_type() == y.scalar_type());
  TORCH_CHECK(gain.scalar_type() == at::kFloat && gain.numel() == 1 &&
              gain.is_cuda(), "gain: one fp32 number on the device");
  if (T_ == 0) return;
  const bool vec = W % 4 == 0 && y.stride(0) % 4 == 0 && aligned16(x) &&
                   aligned16(y) && aligned16(h);
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(y, {
    if (vec) {
      hipLaunchKernelGGL((scalar_postnorm_residual_kernel<T, 4>), dim3(T_),
                         dim3(256), 0, stream, x.data_ptr<float>(),
                         (const T*)y.data_ptr(), (long)y.stride(0),
                         gain.data_ptr<float>(), (float)eps, (T*)h.data_ptr(),
                         W);
    } else {
      hipLaunchKernelGGL((scalar_postnorm_residual_kernel<T, 1>), dim3(T_),
                         dim3(256), 0, stream, x.data_ptr<float>(),
                         (const T*)y.data_ptr(), (long)y.stride(0),
                         gain.data_ptr<float>(), (float)eps, (T*)h.data_ptr(),
                         W);
    }
  });
}

void scalar_rmsnorm(torch::Tensor out, torch::Tensor x, torch::Tensor gain,
                    double eps) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2, "x must be contiguous fp32 [T, W]");
  const int T_ = x.size(0), W = x.size(1);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
              out.size(1) == W);
  TORCH_CHECK(gain.scalar_type() == at::kFloat && gain.numel() == 1 &&
              gain.is_cuda(), "gain: one fp32 number on the device");
  if (T_ == 0) return;
  const bool vec = W % 4 == 0 && aligned16(x) && aligned16(out);
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((scalar_rmsnorm_kernel<T, 4>), dim3(T_), dim3(256), 0,
                         stream, (T*)out.data_ptr(), x.data_ptr<float>(),
                         gain.data_ptr<float>(), (float)eps, W);
    } else {
      hipLaunchKernelGGL((scalar_rmsnorm_kernel<T, 1>), dim3(T_), dim3(256), 0,
                         stream, (T*)out.data_ptr(), x.data_ptr<float>(),
                         gain.data_ptr<float>(), (float)eps, W);
    }
  });
}

void poly_norm(torch::Tensor out, torch::Tensor z, torch::Tensor coef,
               double eps) {
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1);
  const int T_ = z.size(0), F = z.size(1);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
              out.size(1) == F && out.scalar_type() == z.scalar_type());
  TORCH_CHECK(coef.scalar_type() == at::kFloat && coef.numel() == 4 &&
              coef.is_contiguous() && coef.is_cuda(),
              "coef: four fp32 numbers on the device");
  if (T_ == 0) return;
  const bool vec = F % 4 == 0 && z.stride(0) % 4 == 0 && aligned16(z) &&
                   aligned16(out);
  auto stream = at::hip::getCurrentHIPStream();
#define LAUNCH_POLY(VEC_, MAXC_)                                              \
  hipLaunchKernelGGL((poly_norm_kernel<T, VEC_, MAXC_>), dim3(T_), dim3(256), \
                     0, stream, (T*)out.data_ptr(), (const T*)z.data_ptr(),   \
                     (long)z.stride(0), coef.data_ptr<float>(), (float)eps, F)
  LATENT_DISPATCH_T(z, {
    if (vec && F <= 256 * 4 * 4) {
      LAUNCH_POLY(4, 4);
    } else if (vec && F <= 256 * 4 * 16) {
      LAUNCH_POLY(4, 16);
    } else if (vec) {
      LAUNCH_POLY(4, 0);
    } else {
      LAUNCH_POLY(1, 0);
    }
  });
#undef LAUNCH_POLY
}
