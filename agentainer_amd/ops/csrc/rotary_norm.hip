// Rotary tables and query/key preparation fused with the paged K/V append
// (gfx950).
//
//   rotary_table         cs[t] = (cos(a) * amp | sin(a) * amp), a = position
//                        * freq[i] (fp32 product, exact range-reduced
//                        cosf/sinf), once per engine step and rotary setting:
//                        every layer and head with that setting reads it.
//   rotary_norm_append   for every new token and head, in fp32:
//
//     norm_first : u <- u / sqrt(mean(u^2) + eps) * w ;  u <- rotate(u)
//     otherwise  : u <- rotate(u) ;  u <- u / sqrt(mean(u^2) + eps)
//
// rotate() turns the first 2*half coordinates of the head, coordinate i
// paired with i + half; coordinates from 2*half on pass through. `amp` is 1
// unless the frequencies are YaRN-stretched.
//
// q [T, H, D] is rewritten in place (a strided view of the fused
// projection's output); k [T, G, D] goes straight into the pool
// k_cache[P, G, PS, D] at the token's slot and v [T, G, Dv] is copied into
// v_cache[P, G, PS, Dv] — rotated keys never travel through HBM twice.
// slot < 0 skips the append. One wave per (token, head): a lane owns whole
// rotation pairs (i, i + half) plus a strided share of the pass-through
// coordinates, so a head lives in registers from its load to its store and
// only the sums of squares cross lanes.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <algorithm>
#include "latent_common.h"

namespace {

constexpr int RN_WAVES = 4;
constexpr int RN_PAIRS = 2;   // rotation pairs per lane: rotary dims <= 256
constexpr int RN_PASS = 4;    // pass-through values per lane: <= 256

__global__ __launch_bounds__(256) void rotary_table_kernel(
    float* __restrict__ cs, const int* __restrict__ positions,
    const float* __restrict__ freqs, float amp, int half, long n) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const long t = idx / half;
  const int i = (int)(idx % half);
  const float ang = (float)positions[t] * freqs[i];
  cs[t * 2 * half + i] = cosf(ang) * amp;
  cs[t * 2 * half + half + i] = sinf(ang) * amp;
}

template <typename T>
__global__ __launch_bounds__(64 * RN_WAVES) void rotary_norm_append_kernel(
    T* __restrict__ q, long q_ts, long q_hs, const T* __restrict__ k,
    long k_ts, long k_hs, const T* __restrict__ v, long v_ts, long v_hs,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const float* __restrict__ cos_sin, int half,
    const long* __restrict__ slots, float eps, const float* __restrict__ q_w,
    const float* __restrict__ k_w, int norm_first, int n_tok, int H, int G,
    int D, int Dv, int PS) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int per_tok = H + 2 * G;
  const unsigned item = blockIdx.x * RN_WAVES + wave;
  if (item >= (unsigned)n_tok * per_tok) return;   // whole wave leaves
  const int t = (int)(item / (unsigned)per_tok);
  const float* cs = cos_sin + (long)t * 2 * half;
  const long slot = slots[t];
  const int rot = 2 * half;
  const int j0 = (int)(item % (unsigned)per_tok);
  for (int j = j0; j == j0; ++j) {             // one item; `continue` leaves
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
    // every load of the head is issued before the first use: head values,
    // the token's cos/sin and (norm_first) the norm weights
    float a[RN_PAIRS], b[RN_PAIRS], c[RN_PASS];
    float cc[RN_PAIRS], sn[RN_PAIRS];
    float wa[RN_PAIRS], wb[RN_PAIRS], wc[RN_PASS];
    const bool use_w = norm_first && w != nullptr;
#pragma unroll
    for (int n = 0; n < RN_PAIRS; ++n) {
      const int i = lane + n * WAVE;
      const bool ok = i < half;
      a[n] = ok ? ldf(src, i) : 0.f;
      b[n] = ok ? ldf(src, i + half) : 0.f;
      cc[n] = ok ? cs[i] : 1.f;
      sn[n] = ok ? cs[half + i] : 0.f;
      wa[n] = (ok && use_w) ? w[i] : 1.f;
      wb[n] = (ok && use_w) ? w[i + half] : 1.f;
    }
#pragma unroll
    for (int n = 0; n < RN_PASS; ++n) {
      const int i = rot + lane + n * WAVE;
      c[n] = i < D ? ldf(src, i) : 0.f;
      wc[n] = (i < D && use_w) ? w[i] : 1.f;
    }
    float ss = 0.f;
    if (norm_first) {
#pragma unroll
      for (int n = 0; n < RN_PAIRS; ++n)
        ss = fmaf(a[n], a[n], fmaf(b[n], b[n], ss));
#pragma unroll
      for (int n = 0; n < RN_PASS; ++n) ss = fmaf(c[n], c[n], ss);
      const float r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
#pragma unroll
      for (int n = 0; n < RN_PAIRS; ++n) {
        a[n] *= r * wa[n];
        b[n] *= r * wb[n];
      }
#pragma unroll
      for (int n = 0; n < RN_PASS; ++n) c[n] *= r * wc[n];
    }
    ss = 0.f;
#pragma unroll
    for (int n = 0; n < RN_PAIRS; ++n) {
      const float x = a[n], y = b[n];
      a[n] = x * cc[n] - y * sn[n];
      b[n] = y * cc[n] + x * sn[n];
      ss = fmaf(a[n], a[n], fmaf(b[n], b[n], ss));
    }
    float r = 1.0f;
    if (!norm_first) {
#pragma unroll
      for (int n = 0; n < RN_PASS; ++n) ss = fmaf(c[n], c[n], ss);
      r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    }
    T* dst = is_q ? q + (long)t * q_ts + (long)j * q_hs
                  : k_cache +
                        (((slot / PS) * G + (j - H)) * PS + slot % PS) * D;
#pragma unroll
    for (int n = 0; n < RN_PAIRS; ++n) {
      const int i = lane + n * WAVE;
      if (i < half) {
        stf(dst, i, a[n] * r);
        stf(dst, i + half, b[n] * r);
      }
    }
#pragma unroll
    for (int n = 0; n < RN_PASS; ++n) {
      const int i = rot + lane + n * WAVE;
      if (i < D) stf(dst, i, c[n] * r);
    }
  }
}


// bf16 heads of exactly 64 * EPL coordinates (EPL = 1, 2, 4; rotary half a
// multiple of EPL): lane l owns coordinates [l*EPL, (l+1)*EPL), moved with
// ONE load and ONE store per head, and takes its rotation partner from lane
// l +- half/EPL by a shuffle. The kernel is bound by vector-memory
// instructions per wave, and this form issues 4-5 of them instead of 11.
template <int EPL>
struct VecOf;
template <>
struct VecOf<1> { typedef short S; typedef float F; };
template <>
struct VecOf<2> {
  typedef short S __attribute__((ext_vector_type(2)));
  typedef float F __attribute__((ext_vector_type(2)));
};
template <>
struct VecOf<4> {
  typedef short S __attribute__((ext_vector_type(4)));
  typedef float F __attribute__((ext_vector_type(4)));
};

template <int EPL>
__device__ __forceinline__ void ld_bf(const short* p, float* v) {
  typename VecOf<EPL>::S t = *reinterpret_cast<const typename VecOf<EPL>::S*>(p);
  if constexpr (EPL == 1) {
    v[0] = bits2f(t);
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = bits2f(t[e]);
  }
}
template <int EPL>
__device__ __forceinline__ void st_bf(short* p, const float* v) {
  typename VecOf<EPL>::S t;
  if constexpr (EPL == 1) {
    t = f2bits(v[0]);
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) t[e] = f2bits(v[e]);
  }
  *reinterpret_cast<typename VecOf<EPL>::S*>(p) = t;
}
template <int EPL>
__device__ __forceinline__ void ld_f(const float* p, float* v) {
  typename VecOf<EPL>::F t = *reinterpret_cast<const typename VecOf<EPL>::F*>(p);
  if constexpr (EPL == 1) {
    v[0] = t;
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) v[e] = t[e];
  }
}

template <int EPL>
__global__ __launch_bounds__(64 * RN_WAVES) void rotary_norm_append_vec_kernel(
    short* __restrict__ q, long q_ts, long q_hs, const short* __restrict__ k,
    long k_ts, long k_hs, const short* __restrict__ v, long v_ts, long v_hs,
    short* __restrict__ k_cache, short* __restrict__ v_cache,
    const float* __restrict__ cos_sin, int half,
    const long* __restrict__ slots, float eps, const float* __restrict__ q_w,
    const float* __restrict__ k_w, int norm_first, int n_tok, int H, int G,
    int Dv, int PS) {
  constexpr int D = WAVE * EPL;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int per_tok = H + 2 * G;
  const unsigned item = blockIdx.x * RN_WAVES + wave;
  if (item >= (unsigned)n_tok * per_tok) return;   // whole wave leaves
  const int t = (int)(item / (unsigned)per_tok);
  const int j = (int)(item % (unsigned)per_tok);
  const long slot = slots[t];
  if (j >= H + G) {                            // value head: plain copy
    if (slot < 0) return;
    const int g = j - H - G;
    const short* src = v + (long)t * v_ts + (long)g * v_hs;
    short* dst = v_cache + (((slot / PS) * G + g) * PS + slot % PS) * Dv;
    for (int i = lane; i < Dv; i += WAVE) dst[i] = src[i];
    return;
  }
  const bool is_q = j < H;
  if (!is_q && slot < 0) return;
  const short* src = is_q ? q + (long)t * q_ts + (long)j * q_hs
                          : k + (long)t * k_ts + (long)(j - H) * k_hs;
  const float* w = is_q ? q_w : k_w;
  const int e0 = lane * EPL;
  const int rot = 2 * half;
  const bool low = e0 < half, turns = e0 < rot;
  const float* cs = cos_sin + (long)t * rot;
  float x[EPL], cc[EPL], sn[EPL], wv[EPL];
  ld_bf<EPL>(src + e0, x);
#pragma unroll
  for (int e = 0; e < EPL; ++e) { cc[e] = 1.f; sn[e] = 0.f; wv[e] = 1.f; }
  if (turns) {
    const int i0 = low ? e0 : e0 - half;
    ld_f<EPL>(cs + i0, cc);
    ld_f<EPL>(cs + half + i0, sn);
  }
  if (norm_first && w != nullptr) ld_f<EPL>(w + e0, wv);
  if (norm_first) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) ss = fmaf(x[e], x[e], ss);
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
#pragma unroll
    for (int e = 0; e < EPL; ++e) x[e] *= r * wv[e];
  }
  // partner coordinate e +- half lives half/EPL lanes away
  const int hop = half / EPL;
  const int partner = low ? lane + hop : lane - hop;
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const float y = __shfl(x[e], turns ? partner : lane, WAVE);
    const float rx = low ? x[e] * cc[e] - y * sn[e] : x[e] * cc[e] + y * sn[e];
    x[e] = turns ? rx : x[e];
    ss = fmaf(x[e], x[e], ss);
  }
  if (!norm_first) {
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
#pragma unroll
    for (int e = 0; e < EPL; ++e) x[e] *= r;
  }
  short* dst = is_q ? q + (long)t * q_ts + (long)j * q_hs
                    : k_cache +
                          (((slot / PS) * G + (j - H)) * PS + slot % PS) * D;
  st_bf<EPL>(dst + e0, x);
}

}  // namespace

torch::Tensor rotary_table(torch::Tensor positions, torch::Tensor freqs,
                           double amp) {
  TORCH_CHECK(positions.scalar_type() == at::kInt && positions.is_contiguous() &&
              positions.is_cuda());
  TORCH_CHECK(freqs.scalar_type() == at::kFloat && freqs.is_contiguous() &&
              freqs.device() == positions.device());
  const long T_ = positions.numel();
  const int half = freqs.numel();
  auto cs = torch::empty({T_, 2L * half},
                         torch::TensorOptions().dtype(torch::kFloat).device(
                             positions.device()));
  const long n = T_ * half;
  if (n == 0) return cs;
  hipLaunchKernelGGL(rotary_table_kernel, dim3((unsigned)((n + 255) / 256)),
                     dim3(256), 0, at::hip::getCurrentHIPStream(),
                     cs.data_ptr<float>(), positions.data_ptr<int>(),
                     freqs.data_ptr<float>(), (float)amp, half, n);
  return cs;
}

void rotary_norm_append(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                        torch::Tensor k_cache, torch::Tensor v_cache,
                        torch::Tensor cos_sin, torch::Tensor slot_mapping,
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
  TORCH_CHECK(cos_sin.scalar_type() == at::kFloat && cos_sin.is_contiguous() &&
              cos_sin.dim() == 2 && cos_sin.size(0) == T_ &&
              cos_sin.size(1) % 2 == 0 && cos_sin.is_cuda(),
              "cos_sin must be contiguous fp32 [T, 2 * half]");
  const int half = cos_sin.size(1) / 2;
  TORCH_CHECK(2 * half <= D, "rotary dims exceed the head size");
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
  TORCH_CHECK(half <= WAVE * RN_PAIRS && D - 2 * half <= WAVE * RN_PASS,
              "head size too large");
  const long items = (long)T_ * (H + 2 * G);
  TORCH_CHECK(items < (1L << 31), "too many (token, head) items");
  auto stream = at::hip::getCurrentHIPStream();
  const dim3 grid((unsigned)((items + RN_WAVES - 1) / RN_WAVES));
  const int epl = D / WAVE;
  auto al = [&](const torch::Tensor& x, long bytes) {
    return reinterpret_cast<uintptr_t>(x.data_ptr()) % bytes == 0;
  };
  if (q.scalar_type() == at::kBFloat16 && D % WAVE == 0 &&
      (epl == 1 || epl == 2 || epl == 4) && half % epl == 0 &&
      q.stride(0) % epl == 0 && q.stride(1) % epl == 0 &&
      k.stride(0) % epl == 0 && k.stride(1) % epl == 0 && al(q, 2 * epl) &&
      al(k, 2 * epl) && al(k_cache, 2 * epl) && al(cos_sin, 16) &&
      (qw == nullptr || reinterpret_cast<uintptr_t>(qw) % 16 == 0) &&
      (kw == nullptr || reinterpret_cast<uintptr_t>(kw) % 16 == 0)) {
#define LAUNCH_VEC(EPL_)                                                      \
  hipLaunchKernelGGL(                                                         \
      rotary_norm_append_vec_kernel<EPL_>, grid, dim3(64 * RN_WAVES), 0,      \
      stream, (short*)q.data_ptr(), (long)q.stride(0), (long)q.stride(1),     \
      (const short*)k.data_ptr(), (long)k.stride(0), (long)k.stride(1),       \
      (const short*)v.data_ptr(), (long)v.stride(0), (long)v.stride(1),       \
      (short*)k_cache.data_ptr(), (short*)v_cache.data_ptr(),                 \
      cos_sin.data_ptr<float>(), half, slot_mapping.data_ptr<long>(),         \
      (float)eps, qw, kw, norm_first ? 1 : 0, T_, H, G, Dv,                   \
      (int)k_cache.size(2))
    if (epl == 1) {
      LAUNCH_VEC(1);
    } else if (epl == 2) {
      LAUNCH_VEC(2);
    } else {
      LAUNCH_VEC(4);
    }
#undef LAUNCH_VEC
    return;
  }
  LATENT_DISPATCH_T(q, {
    hipLaunchKernelGGL(
        rotary_norm_append_kernel<T>,
        grid, dim3(64 * RN_WAVES), 0, stream, (T*)q.data_ptr(),
        (long)q.stride(0),
        (long)q.stride(1), (const T*)k.data_ptr(), (long)k.stride(0),
        (long)k.stride(1), (const T*)v.data_ptr(), (long)v.stride(0),
        (long)v.stride(1), (T*)k_cache.data_ptr(), (T*)v_cache.data_ptr(),
        cos_sin.data_ptr<float>(), half, slot_mapping.data_ptr<long>(),
        (float)eps, qw, kw, norm_first ? 1 : 0, T_, H, G, D, Dv,
        (int)k_cache.size(2));
  });
}
