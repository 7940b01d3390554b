// Query/key preparation fused with the paged K/V append (gfx950).
//
// For every new token and head, in fp32:
//
//   norm_first : u <- u / sqrt(mean(u^2) + eps) * w ;  u <- rotate(u)
//   otherwise  : u <- rotate(u) ;  u <- u / sqrt(mean(u^2) + eps)
//
// rotate() turns the first 2*half coordinates of the head: coordinate i is
// paired with i + half, angle = position * freq[i] (fp32 product, exact
// cosf/sinf), and cos/sin are scaled by `amp` (1 unless the frequencies
// are YaRN-stretched). Coordinates from 2*half on pass through.
//
// q [T, H, D] is rewritten in place (a strided view of the fused
// projection's output); k [T, G, D] goes straight into the pool
// k_cache[P, G, PS, D] at the token's slot and v [T, G, Dv] is copied into
// v_cache[P, G, PS, Dv] — rotated keys never travel through HBM twice.
// slot < 0 skips the append. A workgroup serves one token and a slice of
// its heads (grid.y slices; few slices for long prompts, one head per wave
// for decode steps): its threads first fill the token's cos/sin table in
// LDS (the exact, range-reduced cosf/sinf are the expensive part and the
// heads of a slice share them), then each of the 4 waves takes its heads
// in turn; a head vector sits in the wave's private LDS patch so the pair
// partner may live in any lane.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <algorithm>
#include "latent_common.h"

namespace {

constexpr int RN_WAVES = 4;

__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T>
__global__ __launch_bounds__(64 * RN_WAVES) void rotary_norm_append_kernel(
    T* __restrict__ q, long q_ts, long q_hs, const T* __restrict__ k,
    long k_ts, long k_hs, const T* __restrict__ v, long v_ts, long v_hs,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const float* __restrict__ freqs, float amp, int half,
    const int* __restrict__ positions, const long* __restrict__ slots,
    float eps, const float* __restrict__ q_w, const float* __restrict__ k_w,
    int norm_first, int heads_per_wave, int H, int G, int D, int Dv, int PS) {
  extern __shared__ float smem[];
  float* cs = smem;                            // [2 * half]: cos | sin
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < half; i += WAVE * RN_WAVES) {
    const float ang = pos * freqs[i];
    cs[i] = cosf(ang) * amp;
    cs[half + i] = sinf(ang) * amp;
  }
  __syncthreads();
  const long slot = slots[t];
  float* s = smem + 2 * half + wave * D;
  const int j0 = (blockIdx.y * RN_WAVES + wave) * heads_per_wave;
  const int j1 = min(j0 + heads_per_wave, H + 2 * G);
  for (int j = j0; j < j1; ++j) {              // wave-uniform
    if (j >= H + G) {                          // value head: plain copy
      if (slot < 0) continue;
      const int g = j - H - G;
      const T* src = v + (long)t * v_ts + (long)g * v_hs;
      T* dst = v_cache + (((slot / PS) * G + g) * PS + slot % PS) * Dv;
      for (int i = lane; i < Dv; i += WAVE) dst[i] = src[i];
      continue;
    }
    const bool is_q = j < H;
    if (!is_q && slot < 0) continue;
    const T* src = is_q ? q + (long)t * q_ts + (long)j * q_hs
                        : k + (long)t * k_ts + (long)(j - H) * k_hs;
    const float* w = is_q ? q_w : k_w;
    wave_lds_sync();                           // patch free again
    float ss = 0.f;
    for (int i = lane; i < D; i += WAVE) {
      const float u = ldf(src, i);
      s[i] = u;
      ss = fmaf(u, u, ss);
    }
    if (norm_first) {
      const float r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
      for (int i = lane; i < D; i += WAVE)
        s[i] = s[i] * r * (w != nullptr ? w[i] : 1.0f);
    }
    wave_lds_sync();
    for (int i = lane; i < half; i += WAVE) {
      const float c = cs[i], sn = cs[half + i];
      const float a = s[i], b = s[i + half];
      s[i] = a * c - b * sn;
      s[i + half] = b * c + a * sn;
    }
    wave_lds_sync();
    float r = 1.0f;
    if (!norm_first) {
      ss = 0.f;
      for (int i = lane; i < D; i += WAVE) ss = fmaf(s[i], s[i], ss);
      r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    }
    T* dst = is_q ? q + (long)t * q_ts + (long)j * q_hs
                  : k_cache +
                        (((slot / PS) * G + (j - H)) * PS + slot % PS) * D;
    for (int i = lane; i < D; i += WAVE) stf(dst, i, s[i] * r);
  }
}

}  // namespace

void rotary_norm_append(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                        torch::Tensor k_cache, torch::Tensor v_cache,
                        torch::Tensor freqs, double amp,
                        torch::Tensor positions, torch::Tensor slot_mapping,
                        double eps, c10::optional<torch::Tensor> q_w,
                        c10::optional<torch::Tensor> k_w, bool norm_first) {
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 &&
              q.stride(2) == 1 && k.stride(2) == 1 && v.stride(2) == 1);
  const int T_ = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Dv = v.size(2);
  TORCH_CHECK(k.size(0) == T_ && v.size(0) == T_ && k.size(2) == D &&
              v.size(1) == G, "q/k/v shapes disagree");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
              k_cache.size(1) == G && k_cache.size(3) == D,
              "k_cache must be contiguous [P, G, PS, D]");
  TORCH_CHECK(v_cache.dim() == 4 && v_cache.is_contiguous() &&
              v_cache.size(1) == G && v_cache.size(3) == Dv &&
              v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(2) == k_cache.size(2),
              "v_cache must be contiguous [P, G, PS, Dv]");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type(),
              "q, k, v and the pools share one element type");
  TORCH_CHECK(freqs.scalar_type() == at::kFloat && freqs.is_contiguous() &&
              freqs.is_cuda());
  const int half = freqs.numel();
  TORCH_CHECK(2 * half <= D, "rotary dims exceed the head size");
  TORCH_CHECK(positions.scalar_type() == at::kInt && positions.numel() == T_ &&
              positions.is_contiguous());
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong &&
              slot_mapping.numel() == T_ && slot_mapping.is_contiguous());
  const float* qw = nullptr;
  const float* kw = nullptr;
  if (q_w.has_value()) {
    TORCH_CHECK(q_w->scalar_type() == at::kFloat && q_w->numel() == D &&
                q_w->is_contiguous());
    qw = q_w->data_ptr<float>();
  }
  if (k_w.has_value()) {
    TORCH_CHECK(k_w->scalar_type() == at::kFloat && k_w->numel() == D &&
                k_w->is_contiguous());
    kw = k_w->data_ptr<float>();
  }
  if (T_ == 0) return;
  const size_t smem = ((size_t)RN_WAVES * D + 2 * half) * sizeof(float);
  TORCH_CHECK(smem <= 64 * 1024, "head size too large");
  // long prompts: several heads per wave share one cos/sin table; short
  // steps: one head per wave so the launch still fills the chip
  const int per_tok = H + 2 * G;
  const int hpw = T_ >= 1024 ? std::min(4, (per_tok + RN_WAVES - 1) / RN_WAVES)
                             : 1;
  const int slices = (per_tok + RN_WAVES * hpw - 1) / (RN_WAVES * hpw);
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(q, {
    hipLaunchKernelGGL(
        rotary_norm_append_kernel<T>,
        dim3((unsigned)T_, (unsigned)slices), dim3(64 * RN_WAVES), smem, stream, (T*)q.data_ptr(), (long)q.stride(0),
        (long)q.stride(1), (const T*)k.data_ptr(), (long)k.stride(0),
        (long)k.stride(1), (const T*)v.data_ptr(), (long)v.stride(0),
        (long)v.stride(1), (T*)k_cache.data_ptr(), (T*)v_cache.data_ptr(),
        freqs.data_ptr<float>(), (float)amp, half, positions.data_ptr<int>(),
        slot_mapping.data_ptr<long>(), (float)eps, qw, kw,
        norm_first ? 1 : 0, hpw, H, G, D, Dv, (int)k_cache.size(2));
  });
}
