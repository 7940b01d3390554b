// Latent window attention over a paged latent pool (gfx950).
//
// The pool caches ONE normalized latent row c[j] (Rp numbers, zero-padded
// to a multiple of 32) per token: pool[page][slot][Rp]. Queries arrive
// already mapped into the latent basis (q_lat[h][t][Rp]), so every head
// scores the SAME cached rows and the output is the softmax-weighted sum
// of those rows again — multi-query attention with K = V = c:
//
//   s[h,t,j]   = scale * <q_lat[h,t], c[j]>      for  pos(t)-window < j <= pos(t)
//   o_lat[h,t] = sum_j softmax_j(s[h,t,:]) c[j]
//
// Scores, softmax and the accumulation are fp32.
//
// Kernels:
//   latent_norm_append    RMS-norm the query latent and the kv latent held in
//                         two column ranges of the fused input GEMM's output;
//                         the kv latent goes straight into its pool slot.
//   latent_attn_mfma      bf16 MFMA tile kernel, prefill portions AND decode.
//                         Its row dimension is the FLATTENED (token, head)
//                         pair: a workgroup (4 waves x 16 rows) covers 64
//                         consecutive pairs of one sequence, stages each
//                         32-token tile of latents in LDS once — row-major
//                         for QK^T, transposed for PV — and all its rows
//                         share it. A decode step (1 token) therefore still
//                         fills MFMA rows with that token's heads, and each
//                         cached row is read once for all of them.
//   latent_attn_rowwave   one wave per (token, head), any element type —
//                         the fp32 path, and the fallback for ranks the
//                         tile kernel is not instantiated for.
//   sigmoid_gate_mul      heads * sigmoid(gate), also re-lays [H,T,E] to
//                         [T, H*E] for the output projection.
//
// MFMA fragment maps (v_mfma_f32_16x16x32_bf16): A lane l holds
// A[l%16][(l/16)*8 + j]; B lane l holds B[(l/16)*8 + j][l%16]; C/D lane l
// holds rows (l/16)*4 + r, column l%16.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <cfloat>
#include "latent_common.h"

namespace {

typedef __bf16 bf16v8 __attribute__((ext_vector_type(8)));

// ------------------------------------------------------------------
// latent_norm_append
// ------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_norm_append_kernel(
    const T* __restrict__ proj, long proj_rs, int q_off, int q_rank,
    int kv_off, int kv_rank, const float* __restrict__ wq,
    const float* __restrict__ wkv, float eps, T* __restrict__ cq_out,
    T* __restrict__ cache, int Rp, const long* __restrict__ slots) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const T* row = proj + t * proj_rs;
  // query latent
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += 256) {
    const float v = ldf(row, q_off + i);
    ss = fmaf(v, v, ss);
  }
  float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += 256)
    stf(cq_out, t * q_rank + i, ldf(row, q_off + i) * r * wq[i]);
  // key/value latent -> pool slot
  const long slot = slots[t];
  if (slot < 0) return;  // uniform per block
  ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += 256) {
    const float v = ldf(row, kv_off + i);
    ss = fmaf(v, v, ss);
  }
  r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)kv_rank + eps);
  T* dst = cache + slot * Rp;
  for (int i = threadIdx.x; i < Rp; i += 256)
    stf(dst, i, i < kv_rank ? ldf(row, kv_off + i) * r * wkv[i] : 0.f);
}

// ------------------------------------------------------------------
// latent_attn_rowwave: one wave per (query token, head)
// ------------------------------------------------------------------
constexpr int RW_MAX_ACC = 16;  // Rp <= 64 * 16

template <typename T>
__global__ __launch_bounds__(64) void latent_attn_rowwave_kernel(
    T* __restrict__ out, const T* __restrict__ q_lat, long q_hs, long q_ts,
    long o_hs, long o_ts, const T* __restrict__ cache,
    const int* __restrict__ page_table, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens,
    float scale, int window, int Rp, int PS, int max_pages) {
  extern __shared__ float smem[];
  float* q_s = smem;        // [Rp]
  float* p_s = smem + Rp;   // [64]
  const int qi = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
  const int lane = threadIdx.x;
  const int qlen = q_lens ? q_lens[b] : 1;
  if (qi >= qlen) return;
  const int total = seq_lens[b];
  const long rowi = (q_starts ? q_starts[b] : b) + qi;
  T* op = out + h * o_hs + rowi * o_ts;
  if (total <= 0) {  // pad row of a captured decode batch
    for (int i = lane; i < Rp; i += WAVE) stf(op, i, 0.f);
    return;
  }
  const int qpos = total - qlen + qi;
  const int lo = max(0, qpos - window + 1);
  const T* qp = q_lat + h * q_hs + rowi * q_ts;
  for (int i = lane; i < Rp; i += WAVE) q_s[i] = ldf(qp, i);
  __syncthreads();
  const int* pt = page_table + (long)b * max_pages;

  float m = -FLT_MAX, l = 0.f;
  float acc[RW_MAX_ACC];
#pragma unroll
  for (int k = 0; k < RW_MAX_ACC; ++k) acc[k] = 0.f;

  for (int j0 = lo; j0 <= qpos; j0 += WAVE) {
    const int j = j0 + lane;
    const bool valid = j <= qpos;
    float s = -FLT_MAX;
    if (valid) {
      const T* cr = cache + ((long)pt[j / PS] * PS + j % PS) * Rp;
      float d = 0.f;
      for (int i = 0; i < Rp; i += 4) {
        float c4[4];
        ld4(cr, i, c4);
        d = fmaf(q_s[i], c4[0], d);
        d = fmaf(q_s[i + 1], c4[1], d);
        d = fmaf(q_s[i + 2], c4[2], d);
        d = fmaf(q_s[i + 3], c4[3], d);
      }
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float alpha = (m == -FLT_MAX) ? 0.f : expf(m - mn);
    const float p = valid ? expf(s - mn) : 0.f;
    l = l * alpha + wave_sum(p);
    m = mn;
    p_s[lane] = p;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < RW_MAX_ACC; ++k) acc[k] *= alpha;
    const int n = min(WAVE, qpos - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const int jg = j0 + jj;
      const T* cr = cache + ((long)pt[jg / PS] * PS + jg % PS) * Rp;
      const float pj = p_s[jj];
#pragma unroll
      for (int k = 0; k < RW_MAX_ACC; ++k)
        if (k * WAVE < Rp) {
          const int d = k * WAVE + lane;
          if (d < Rp) acc[k] = fmaf(pj, ldf(cr, d), acc[k]);
        }
    }
    __syncthreads();
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int k = 0; k < RW_MAX_ACC; ++k) {
    const int d = k * WAVE + lane;
    if (d < Rp) stf(op, d, acc[k] * inv);
  }
}

// ------------------------------------------------------------------
// latent_attn_mfma: bf16 tile kernel over flattened (token, head) rows
// ------------------------------------------------------------------
constexpr int KVT = 32;            // tokens per staged tile
constexpr int ROWS_PER_WAVE = 16;
constexpr int ROWS_PER_BLOCK = 64;
constexpr int VT_STRIDE = KVT + 8;  // shorts; transposed tile row
constexpr int P_STRIDE = KVT + 8;

// MAXNC bounds the rank in 32-wide chunks (registers are sized by it);
// the actual chunk count nc <= MAXNC is a runtime argument.
template <int MAXNC>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(
    short* __restrict__ out, const short* __restrict__ q_lat, long q_hs,
    long q_ts, long o_hs, long o_ts, const short* __restrict__ cache,
    const int* __restrict__ page_table, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens,
    float scale, int window, int H, int nc, int PS, int max_pages,
    float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits) {
  extern __shared__ __attribute__((aligned(16))) short lds[];
  const int Rp = nc * 32;
  const int KS = Rp + 8;                       // padded row-major stride
  short* k_lds = lds;                          // [KVT][KS]
  short* vt_lds = k_lds + KVT * KS;            // [Rp][VT_STRIDE]
  short* p_lds = vt_lds + Rp * VT_STRIDE;      // [4][16][P_STRIDE]

  const int b = blockIdx.y;
  const int qlen = q_lens ? q_lens[b] : 1;
  const int nrows = qlen * H;
  const int r0 = blockIdx.x * ROWS_PER_BLOCK;
  if (r0 >= nrows) return;
  const int total = seq_lens[b];
  const long row_base = q_starts ? q_starts[b] : b;
  const int lane = threadIdx.x % WAVE;
  const int wid = threadIdx.x / WAVE;
  const int l16 = lane % 16, lg = lane / 16;

  if (total <= 0) {  // pad row of a captured decode batch: zeros
    if (n_splits > 0) return;  // the combine kernel writes them
    for (int i = threadIdx.x; i < nrows * Rp; i += 256) {
      const int r = i / Rp, d = i % Rp;
      out[(r % H) * o_hs + (row_base + r / H) * o_ts + d] = 0;
    }
    return;
  }
  const int ctx = total - qlen;
  const int* pt = page_table + (long)b * max_pages;

  // block's key span: first row's window start .. last row's position
  const int r_last = min(r0 + ROWS_PER_BLOCK, nrows) - 1;
  int kv_lo = max(0, ctx + r0 / H - window + 1);
  int kv_hi = ctx + r_last / H;  // inclusive
  if (n_splits > 0) {
    // split-KV (decode): this block owns one 32-aligned slice of the span;
    // an empty slice still writes its (m = -max, l = 0) partial below
    const int n_keys = kv_hi - kv_lo + 1;
    const int span = ((n_keys + n_splits - 1) / n_splits + KVT - 1) / KVT * KVT;
    kv_lo += blockIdx.z * span;
    kv_hi = min(kv_hi, kv_lo + span - 1);
  }

  // ---- this wave's Q fragments: lane -> row l16, cols dc*32 + lg*8..+8
  const int rw0 = r0 + wid * ROWS_PER_WAVE;
  bf16v8 qf[MAXNC];
  {
    const int r = rw0 + l16;
    const bool ok = r < nrows;
    const short* qp =
        ok ? q_lat + (r % H) * q_hs + (row_base + r / H) * q_ts : q_lat;
#pragma unroll
    for (int dc = 0; dc < MAXNC; ++dc) {
      if (dc < nc && ok)
        qf[dc] = *reinterpret_cast<const bf16v8*>(qp + dc * 32 + lg * 8);
      else
        qf[dc] = bf16v8{};
    }
  }
  // positions of the 4 rows this lane holds in C layout
  int qpos[4];
  bool rok[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int rr = rw0 + lg * 4 + r;
    rok[r] = rr < nrows;
    qpos[r] = ctx + rr / H;
  }
  // keys this WAVE can see at all (skips tiles outside its rows' windows)
  const int w_first = min(rw0, nrows - 1), w_last = min(rw0 + 15, nrows - 1);
  const int w_lo = max(0, ctx + w_first / H - window + 1);
  const int w_hi = ctx + w_last / H;
  const bool wave_live = rw0 < nrows;

  f32x4 o[2 * MAXNC];
#pragma unroll
  for (int dt = 0; dt < 2 * MAXNC; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { m_run[r] = -FLT_MAX; l_run[r] = 0.f; }

  const int n_chunks = KVT * (Rp / 8);
  // Staging is split in two so that a whole tile's global loads are in
  // flight at once and overlap the previous tile's MFMAs: stage_load
  // issues every 16-B load of the NEXT tile into registers, stage_write
  // (after the barrier that retires the current tile's readers) stores
  // them row-major (K role) and transposed (V role).
  // chunk -> (token fast, 16-B column slow): the transposed 2-byte writes
  // of one wave land on consecutive LDS addresses (a column-fast mapping
  // puts all 64 lanes on two banks), and the block's 4 waves together
  // consume whole 128-B lines of each row.
  constexpr int MAXIT = (MAXNC + 1) / 2;  // ceil(n_chunks / 256)
  bf16x8 st[MAXIT];
  auto stage_load = [&](int kv0) {
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      const int c = threadIdx.x + 256 * k;
      st[k] = bf16x8{};
      if (c < n_chunks) {
        const int tok = c % KVT, d8 = c / KVT;
        const int gt = kv0 + tok;
        if (gt <= kv_hi)
          st[k] = *reinterpret_cast<const bf16x8*>(
              cache + ((long)pt[gt / PS] * PS + gt % PS) * Rp + d8 * 8);
      }
    }
  };
  auto stage_write = [&]() {
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      const int c = threadIdx.x + 256 * k;
      if (c < n_chunks) {
        const int tok = c % KVT, d8 = c / KVT;
        *reinterpret_cast<bf16x8*>(k_lds + tok * KS + d8 * 8) = st[k];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          vt_lds[(d8 * 8 + j) * VT_STRIDE + tok] = st[k][j];
      }
    }
  };

  if (kv_lo <= kv_hi) stage_load(kv_lo);
  for (int kv0 = kv_lo; kv0 <= kv_hi; kv0 += KVT) {
    stage_write();
    __syncthreads();
    if (kv0 + KVT <= kv_hi) stage_load(kv0 + KVT);

    if (wave_live && kv0 <= w_hi && kv0 + KVT > w_lo) {
      // ---- S = Q K^T, two 16-key sub-tiles
      f32x4 s[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        s[ks] = f32x4{0.f, 0.f, 0.f, 0.f};
        const short* kr = k_lds + (ks * 16 + l16) * KS + lg * 8;
#pragma unroll
        for (int dc = 0; dc < MAXNC; ++dc)
          if (dc < nc) {
            const bf16v8 kf = *reinterpret_cast<const bf16v8*>(kr + dc * 32);
            s[ks] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[dc], kf, s[ks],
                                                            0, 0, 0);
          }
      }
      // ---- window mask + online softmax (fp32)
      float alpha[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const int kpos = kv0 + ks * 16 + l16;
          const bool seen = rok[r] && kpos <= qpos[r] && kpos <= kv_hi &&
                            qpos[r] - kpos < window;
          s[ks][r] = seen ? s[ks][r] * scale : -FLT_MAX;
        }
        float mx = fmaxf(s[0][r], s[1][r]);
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
          mx = fmaxf(mx, __shfl_xor(mx, off, WAVE));
        const float mn = fmaxf(m_run[r], mx);
        alpha[r] = (m_run[r] == -FLT_MAX) ? 0.f : __expf(m_run[r] - mn);
        m_run[r] = mn;
        float rowsum = 0.f;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const float p = (s[ks][r] == -FLT_MAX) ? 0.f : __expf(s[ks][r] - mn);
          s[ks][r] = p;
          rowsum += p;
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1)
          rowsum += __shfl_xor(rowsum, off, WAVE);
        l_run[r] = l_run[r] * alpha[r] + rowsum;
      }
      // ---- P (bf16) through this wave's LDS patch into A-fragment order
      short* pw = p_lds + wid * 16 * P_STRIDE;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          pw[(lg * 4 + r) * P_STRIDE + ks * 16 + l16] = f2bits(s[ks][r]);
      // own-wave LDS ordering: wait for LDS traffic only (lgkmcnt = 0),
      // the next tile's global loads stay in flight
      __builtin_amdgcn_s_waitcnt(0xc07f);
      const bf16v8 pf =
          *reinterpret_cast<const bf16v8*>(pw + l16 * P_STRIDE + lg * 8);
      // ---- O = alpha O + P V
#pragma unroll
      for (int dt = 0; dt < 2 * MAXNC; ++dt)
        if (dt < 2 * nc) {
#pragma unroll
          for (int r = 0; r < 4; ++r) o[dt][r] *= alpha[r];
          const bf16v8 vf = *reinterpret_cast<const bf16v8*>(
              vt_lds + (dt * 16 + l16) * VT_STRIDE + lg * 8);
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[dt], 0, 0,
                                                          0);
        }
    }
    __syncthreads();
  }

  // ---- epilogue
  if (n_splits > 0) {  // unnormalized partials (rows are heads: qlen == 1)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int rr = rw0 + lg * 4 + r;
      if (rr >= nrows) continue;
      const long pr = ((long)b * n_splits + blockIdx.z) * H + rr;
      if (l16 == 0) {
        part_ml[pr * 2] = m_run[r];
        part_ml[pr * 2 + 1] = l_run[r];
      }
#pragma unroll
      for (int dt = 0; dt < 2 * MAXNC; ++dt)
        if (dt < 2 * nc) part_o[pr * Rp + dt * 16 + l16] = o[dt][r];
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int rr = rw0 + lg * 4 + r;
    if (rr >= nrows) continue;
    const float inv = l_run[r] > 0.f ? 1.0f / l_run[r] : 0.f;
    short* op = out + (rr % H) * o_hs + (row_base + rr / H) * o_ts;
#pragma unroll
    for (int dt = 0; dt < 2 * MAXNC; ++dt)
      if (dt < 2 * nc) op[dt * 16 + l16] = f2bits(o[dt][r] * inv);
  }
}

// ------------------------------------------------------------------
// latent_decode_mfma: decode (one new token per sequence), bf16.
//
// The tile kernel above keeps a whole [16 x Rp] fp32 accumulator per wave,
// which at large ranks leaves one barrier-bound workgroup per CU. Here the
// RANK is split over the 4 waves of a workgroup instead: wave w owns
// columns [w*Rp/4, (w+1)*Rp/4) of every key row — for the QK^T contraction
// (partial scores, summed across the waves through LDS) and as its slice of
// the output. Each wave loads its quarter of 32 key rows straight from
// global memory into MFMA B-fragments, transposes the same registers
// through a private LDS patch for the PV product, and keeps only
// [16 x Rp/4] accumulators, so several workgroups share a CU and hide one
// another's load latency. One barrier per 32-key tile (score exchange is
// double-buffered). grid = (sequence, key slice, 16-head row tile);
// results are unnormalized partials for latent_attn_combine.
// ------------------------------------------------------------------
template <int NCW>  // 32-wide rank chunks per wave: Rp = 128 * NCW
__global__ __launch_bounds__(256) void latent_decode_mfma_kernel(
    float* __restrict__ part_o, float* __restrict__ part_ml,
    const short* __restrict__ q_lat, long q_hs, long q_ts,
    const short* __restrict__ cache, const int* __restrict__ page_table,
    const int* __restrict__ seq_lens, float scale, int window, int H, int PS,
    int max_pages, int n_splits) {
  constexpr int CW = NCW * 32;   // columns per wave
  constexpr int Rp = CW * 4;
  constexpr int NDT = CW / 16;   // 16-wide output tiles per wave
  constexpr int S_STRIDE = KVT + 1;
  __shared__ __attribute__((aligned(16))) short vt_lds[4][CW * VT_STRIDE];
  __shared__ __attribute__((aligned(16))) short p_lds[4][16 * P_STRIDE];
  __shared__ float s_lds[2][4][16 * S_STRIDE];

  const int b = blockIdx.x, split = blockIdx.y, rt = blockIdx.z;
  const int total = seq_lens[b];
  if (total <= 0) return;  // pad row: the combine kernel writes zeros
  const int lane = threadIdx.x % WAVE, wid = threadIdx.x / WAVE;
  const int l16 = lane % 16, lg = lane / 16;
  const int col0 = wid * CW;
  const int* pt = page_table + (long)b * max_pages;

  const int qpos = total - 1;
  int kv_lo = max(0, qpos - window + 1);
  int kv_hi = qpos;
  {
    const int n_keys = kv_hi - kv_lo + 1;
    const int span = ((n_keys + n_splits - 1) / n_splits + KVT - 1) / KVT * KVT;
    kv_lo += split * span;
    kv_hi = min(kv_hi, kv_lo + span - 1);
  }

  // Q fragments (A operand): row = head rt*16 + l16, this wave's columns
  bf16v8 qf[NCW];
  {
    const int h = rt * 16 + l16;
    const short* qp = q_lat + (long)min(h, H - 1) * q_hs + (long)b * q_ts + col0;
#pragma unroll
    for (int dc = 0; dc < NCW; ++dc)
      qf[dc] = h < H ? *reinterpret_cast<const bf16v8*>(qp + dc * 32 + lg * 8)
                     : bf16v8{};
  }
  f32x4 o[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { m_run[r] = -FLT_MAX; l_run[r] = 0.f; }

  // page ids are looked up TWO tiles ahead and rows ONE tile ahead, so the
  // dependent (page table -> row) load chain never sits on the critical path
  auto pages_of = [&](int kv0, int (&pg)[2]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int key = kv0 + ks * 16 + l16;
      pg[ks] = key <= kv_hi ? pt[key / PS] : -1;
    }
  };
  auto load_tile = [&](int kv0, const int (&pg)[2], bf16x8 (&kf)[2][NCW]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int key = kv0 + ks * 16 + l16;
      const bool ok = pg[ks] >= 0;
      const short* cr =
          ok ? cache + ((long)pg[ks] * PS + key % PS) * Rp + col0 + lg * 8
             : cache;
#pragma unroll
      for (int dc = 0; dc < NCW; ++dc)
        kf[ks][dc] = ok ? *reinterpret_cast<const bf16x8*>(cr + dc * 32)
                        : bf16x8{};
    }
  };

  bf16x8 kf[2][NCW];
  int pg_a[2], pg_b[2];
  pages_of(kv_lo, pg_a);
  pages_of(kv_lo + KVT, pg_b);
  load_tile(kv_lo, pg_a, kf);
  int buf = 0;
  short* vt = vt_lds[wid];
  short* pw = p_lds[wid];
  for (int kv0 = kv_lo; kv0 <= kv_hi; kv0 += KVT) {
    const bool more = kv0 + KVT <= kv_hi;
    pages_of(kv0 + 2 * KVT, pg_a);  // pages of the tile after next
    // ---- partial scores over this wave's columns
    f32x4 s[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      s[ks] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dc = 0; dc < NCW; ++dc) {
        bf16v8 kb;
        __builtin_memcpy(&kb, &kf[ks][dc], 16);
        s[ks] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[dc], kb, s[ks], 0,
                                                        0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        s_lds[buf][wid][(lg * 4 + r) * S_STRIDE + ks * 16 + l16] = s[ks][r];
    }
    // ---- the same registers, transposed, are this wave's V^T tile
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int dc = 0; dc < NCW; ++dc)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          vt[(dc * 32 + lg * 8 + j) * VT_STRIDE + ks * 16 + l16] =
              kf[ks][dc][j];
    // the fragments' last reader is done: the next tile's rows stream into
    // the same registers while this tile's softmax and PV run
    if (more) load_tile(kv0 + KVT, pg_b, kf);
    __syncthreads();
    // ---- full scores, mask, online softmax (identical in all 4 waves)
    float alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool rok = rt * 16 + lg * 4 + r < H;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const int idx = (lg * 4 + r) * S_STRIDE + ks * 16 + l16;
        const float v = s_lds[buf][0][idx] + s_lds[buf][1][idx] +
                        s_lds[buf][2][idx] + s_lds[buf][3][idx];
        const int kpos = kv0 + ks * 16 + l16;
        s[ks][r] = (rok && kpos <= kv_hi) ? v * scale : -FLT_MAX;
      }
      float mx = fmaxf(s[0][r], s[1][r]);
#pragma unroll
      for (int off = 1; off < 16; off <<= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, WAVE));
      const float mn = fmaxf(m_run[r], mx);
      alpha[r] = (m_run[r] == -FLT_MAX) ? 0.f : __expf(m_run[r] - mn);
      m_run[r] = mn;
      float rowsum = 0.f;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const float p = (s[ks][r] == -FLT_MAX) ? 0.f : __expf(s[ks][r] - mn);
        s[ks][r] = p;
        rowsum += p;
      }
#pragma unroll
      for (int off = 1; off < 16; off <<= 1)
        rowsum += __shfl_xor(rowsum, off, WAVE);
      l_run[r] = l_run[r] * alpha[r] + rowsum;
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        pw[(lg * 4 + r) * P_STRIDE + ks * 16 + l16] = f2bits(s[ks][r]);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // LDS only; global loads stay out
    const bf16v8 pf =
        *reinterpret_cast<const bf16v8*>(pw + l16 * P_STRIDE + lg * 8);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] *= alpha[r];
      const bf16v8 vf = *reinterpret_cast<const bf16v8*>(
          vt + (dt * 16 + l16) * VT_STRIDE + lg * 8);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[dt], 0, 0, 0);
    }
    // own-wave WAR on vt / pw: reads above retire before the next writes
    __builtin_amdgcn_s_waitcnt(0xc07f);
    pg_b[0] = pg_a[0];
    pg_b[1] = pg_a[1];
    buf ^= 1;
  }
  // ---- unnormalized partials for this slice
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int rr = rt * 16 + lg * 4 + r;
    if (rr >= H) continue;
    const long pr = ((long)b * n_splits + split) * H + rr;
    if (wid == 0 && l16 == 0) {
      part_ml[pr * 2] = m_run[r];
      part_ml[pr * 2 + 1] = l_run[r];
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
      part_o[pr * Rp + col0 + dt * 16 + l16] = o[dt][r];
  }
}

// merge the split-KV partials of one (sequence, head): log-sum-exp rescale
__global__ __launch_bounds__(128) void latent_attn_combine_kernel(
    short* __restrict__ out, long o_hs, long o_ts,
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int* __restrict__ seq_lens, int H, int Rp, int n_splits) {
  const int h = blockIdx.x, b = blockIdx.y;
  short* op = out + h * o_hs + (long)b * o_ts;
  if (seq_lens[b] <= 0) {
    for (int d = threadIdx.x; d < Rp; d += 128) op[d] = 0;
    return;
  }
  float M = -FLT_MAX;
  for (int s = 0; s < n_splits; ++s)
    M = fmaxf(M, part_ml[(((long)b * n_splits + s) * H + h) * 2]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const long pr = ((long)b * n_splits + s) * H + h;
    const float m = part_ml[pr * 2];
    if (m != -FLT_MAX) L += part_ml[pr * 2 + 1] * __expf(m - M);
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  // Rp is a multiple of 32: 4 consecutive columns per thread
  for (int d = threadIdx.x * 4; d < Rp; d += 128 * 4) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < n_splits; ++s) {
      const long pr = ((long)b * n_splits + s) * H + h;
      const float m = part_ml[pr * 2];
      if (m == -FLT_MAX) continue;
      const float w = __expf(m - M);
      const float4 v = *reinterpret_cast<const float4*>(part_o + pr * Rp + d);
      acc[0] = fmaf(v.x, w, acc[0]);
      acc[1] = fmaf(v.y, w, acc[1]);
      acc[2] = fmaf(v.z, w, acc[2]);
      acc[3] = fmaf(v.w, w, acc[3]);
    }
    bf16x4 o4;
#pragma unroll
    for (int j = 0; j < 4; ++j) o4[j] = f2bits(acc[j] * inv);
    *reinterpret_cast<bf16x4*>(op + d) = o4;
  }
}

template <typename T, int VEC>
__global__ void sigmoid_gate_mul_kernel(T* __restrict__ out,
                                        const T* __restrict__ a, long a_hs,
                                        long a_ts, const T* __restrict__ g,
                                        long g_rs, long n, int H, int E) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long t = i / ((long)H * E);
  const int c = (int)(i % ((long)H * E));
  const int h = c / E, e = c % E;
  float gv[VEC], av[VEC], o[VEC];
  if constexpr (VEC == 4) {
    ld4(g, t * g_rs + c, gv);
    ld4(a, h * a_hs + t * a_ts + e, av);
  } else {
    gv[0] = ldf(g, t * g_rs + c);
    av[0] = ldf(a, h * a_hs + t * a_ts + e);
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) o[j] = av[j] / (1.0f + expf(-gv[j]));
  if constexpr (VEC == 4) {
    st4(out, i, o);
  } else {
    stf(out, i, o[0]);
  }
}

size_t mfma_lds_bytes(int Rp) {
  return sizeof(short) * ((size_t)KVT * (Rp + 8) + (size_t)Rp * VT_STRIDE +
                          4 * 16 * P_STRIDE);
}

}  // namespace

void latent_norm_append(torch::Tensor proj, long q_off, long q_rank,
                        long kv_off, long kv_rank, torch::Tensor wq,
                        torch::Tensor wkv, double eps, torch::Tensor cq_out,
                        torch::Tensor cache, torch::Tensor slot_mapping) {
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const int T_ = proj.size(0);
  TORCH_CHECK(q_off >= 0 && q_off + q_rank <= proj.size(1));
  TORCH_CHECK(kv_off >= 0 && kv_off + kv_rank <= proj.size(1));
  TORCH_CHECK(wq.scalar_type() == at::kFloat && wq.numel() == q_rank &&
              wq.is_contiguous());
  TORCH_CHECK(wkv.scalar_type() == at::kFloat && wkv.numel() == kv_rank &&
              wkv.is_contiguous());
  TORCH_CHECK(cq_out.is_contiguous() && cq_out.size(0) == T_ &&
              cq_out.size(1) == q_rank &&
              cq_out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() &&
              cache.scalar_type() == proj.scalar_type());
  const int Rp = cache.size(2);
  TORCH_CHECK(Rp >= kv_rank, "pool rows narrower than the latent");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong &&
              slot_mapping.numel() == T_ && slot_mapping.is_contiguous());
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(proj, {
    hipLaunchKernelGGL(latent_norm_append_kernel<T>, dim3(T_), dim3(256), 0,
                       stream, (const T*)proj.data_ptr(), (long)proj.stride(0),
                       (int)q_off, (int)q_rank, (int)kv_off, (int)kv_rank,
                       wq.data_ptr<float>(), wkv.data_ptr<float>(), (float)eps,
                       (T*)cq_out.data_ptr(), (T*)cache.data_ptr(), Rp,
                       slot_mapping.data_ptr<long>());
  });
}

void latent_window_attention(torch::Tensor out, torch::Tensor q_lat,
                             torch::Tensor cache, torch::Tensor page_table,
                             torch::Tensor seq_lens,
                             c10::optional<torch::Tensor> query_starts,
                             c10::optional<torch::Tensor> query_lens,
                             double scale, long window, long max_qlen,
                             bool force_simple, long splits) {
  // splits < 0: run decode on the tile kernel with -splits slices (A/B)
  const bool force_tile_decode = splits < 0;
  if (splits < 0) splits = -splits;
  TORCH_CHECK(q_lat.dim() == 3 && out.dim() == 3 && q_lat.stride(2) == 1 &&
              out.stride(2) == 1);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous());
  TORCH_CHECK(q_lat.scalar_type() == cache.scalar_type() &&
              out.scalar_type() == cache.scalar_type());
  const int H = q_lat.size(0), Tq = q_lat.size(1), Rp = q_lat.size(2);
  const int PS = cache.size(1);
  TORCH_CHECK(cache.size(2) == Rp, "query rank != pool row width");
  TORCH_CHECK(out.size(0) == H && out.size(1) == Tq && out.size(2) == Rp);
  TORCH_CHECK(Rp % 4 == 0, "latent rank must be a multiple of 4");
  TORCH_CHECK(page_table.scalar_type() == at::kInt && page_table.dim() == 2 &&
              page_table.is_contiguous());
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(page_table.size(0) == B);
  TORCH_CHECK(query_starts.has_value() == query_lens.has_value());
  const int* qs = nullptr;
  const int* ql = nullptr;
  if (query_starts.has_value()) {
    TORCH_CHECK(query_starts->scalar_type() == at::kInt &&
                query_lens->scalar_type() == at::kInt &&
                query_starts->numel() == B && query_lens->numel() == B);
    qs = query_starts->data_ptr<int>();
    ql = query_lens->data_ptr<int>();
  } else {
    TORCH_CHECK(Tq >= B, "decode: one query row per sequence");
    max_qlen = 1;
  }
  TORCH_CHECK(window >= 1 && max_qlen >= 1);
  if (B == 0 || Tq == 0) return;
  const int max_pages = page_table.size(1);
  auto stream = at::hip::getCurrentHIPStream();

  const bool bf16 = cache.scalar_type() == at::kBFloat16;
  const bool aligned = (q_lat.stride(0) % 8 == 0) && (q_lat.stride(1) % 8 == 0) &&
                       (q_lat.storage_offset() % 8 == 0) &&
                       (out.stride(0) % 8 == 0) && (out.stride(1) % 8 == 0) &&
                       (out.storage_offset() % 8 == 0);
  if (bf16 && !force_simple && Rp % 32 == 0 && Rp <= 512 && aligned) {
    const int nc = Rp / 32;
    const size_t lds = mfma_lds_bytes(Rp);
    if (!query_starts.has_value() && !force_tile_decode &&
        (Rp == 128 || Rp == 256 || Rp == 512)) {
      // decode: rank-split kernel, several workgroups per CU
      const int row_tiles = (H + 15) / 16;
      const long n_max = std::min<long>(window, (long)max_pages * PS);
      const long want =
          (512 + (long)B * row_tiles - 1) / ((long)B * row_tiles);
      long ns = splits > 0 ? splits : std::min<long>(want, n_max / 64);
      if (ns < 1) ns = 1;
      auto fo = torch::TensorOptions().dtype(torch::kFloat).device(out.device());
      auto part_o = torch::empty({(long)B * ns * H * Rp}, fo);
      auto part_ml = torch::empty({(long)B * ns * H * 2}, fo);
      dim3 grid(B, ns, row_tiles);
#define LD_LAUNCH(NCW)                                                         \
  hipLaunchKernelGGL(latent_decode_mfma_kernel<NCW>, grid, dim3(256), 0,       \
                     stream, part_o.data_ptr<float>(),                         \
                     part_ml.data_ptr<float>(), (const short*)q_lat.data_ptr(),\
                     (long)q_lat.stride(0), (long)q_lat.stride(1),             \
                     (const short*)cache.data_ptr(),                           \
                     page_table.data_ptr<int>(), seq_lens.data_ptr<int>(),     \
                     (float)scale, (int)window, H, PS, max_pages, (int)ns)
      if (Rp == 128) LD_LAUNCH(1);
      else if (Rp == 256) LD_LAUNCH(2);
      else LD_LAUNCH(4);
#undef LD_LAUNCH
      hipLaunchKernelGGL(latent_attn_combine_kernel, dim3(H, B), dim3(128), 0,
                         stream, (short*)out.data_ptr(), (long)out.stride(0),
                         (long)out.stride(1), part_o.data_ptr<float>(),
                         part_ml.data_ptr<float>(), seq_lens.data_ptr<int>(),
                         H, Rp, (int)ns);
      return;
    }
    const long rows = max_qlen * H;
    const int row_blocks = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    // decode: too few (sequence, row-block) pairs to fill 256 CUs — cut
    // every sequence's key span into slices (>= 64 keys each) and merge
    int n_splits = 0;
    torch::Tensor part_o, part_ml;
    if (!query_starts.has_value()) {
      const long n_max = std::min<long>(window, (long)max_pages * PS);
      // one resident workgroup per CU at large ranks: aim at one wave of
      // 256 workgroups — more slices only add partial-merge traffic
      const long want = (256 + (long)B * row_blocks - 1) / ((long)B * row_blocks);
      const long s = splits > 0 ? splits : std::min<long>(want, n_max / 64);
      if (s >= 2) {
        n_splits = (int)s;
        auto fo = torch::TensorOptions().dtype(torch::kFloat).device(out.device());
        part_o = torch::empty({(long)B * n_splits * H * Rp}, fo);
        part_ml = torch::empty({(long)B * n_splits * H * 2}, fo);
      }
    }
    dim3 grid(row_blocks, B, n_splits > 0 ? n_splits : 1);
    bool launched = true;
#define LA_LAUNCH(MAXNC)                                                       \
  do {                                                                         \
    auto kern = latent_attn_mfma_kernel<MAXNC>;                                \
    if (lds > 48 * 1024) {                                                     \
      if (hipFuncSetAttribute((const void*)kern,                               \
                              hipFuncAttributeMaxDynamicSharedMemorySize,      \
                              (int)lds) != hipSuccess) {                       \
        (void)hipGetLastError();                                               \
        launched = false;                                                      \
        break;                                                                 \
      }                                                                        \
    }                                                                          \
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream,                     \
                       (short*)out.data_ptr(), (const short*)q_lat.data_ptr(), \
                       (long)q_lat.stride(0), (long)q_lat.stride(1),           \
                       (long)out.stride(0), (long)out.stride(1),               \
                       (const short*)cache.data_ptr(),                         \
                       page_table.data_ptr<int>(), seq_lens.data_ptr<int>(),   \
                       qs, ql, (float)scale, (int)window, H, nc, PS,           \
                       max_pages,                                              \
                       n_splits > 0 ? part_o.data_ptr<float>() : nullptr,      \
                       n_splits > 0 ? part_ml.data_ptr<float>() : nullptr,     \
                       n_splits);                                              \
  } while (0)
    if (nc <= 2) LA_LAUNCH(2);
    else if (nc <= 4) LA_LAUNCH(4);
    else if (nc <= 8) LA_LAUNCH(8);
    else LA_LAUNCH(16);
#undef LA_LAUNCH
    if (launched && n_splits > 0)
      hipLaunchKernelGGL(latent_attn_combine_kernel, dim3(H, B), dim3(128), 0,
                         stream, (short*)out.data_ptr(), (long)out.stride(0),
                         (long)out.stride(1), part_o.data_ptr<float>(),
                         part_ml.data_ptr<float>(), seq_lens.data_ptr<int>(),
                         H, Rp, n_splits);
    if (launched) return;
  }
  TORCH_CHECK(Rp <= WAVE * RW_MAX_ACC, "latent rank too large");
  dim3 grid(max_qlen, B, H);
  const size_t smem = sizeof(float) * (Rp + WAVE);
  LATENT_DISPATCH_T(cache, {
    hipLaunchKernelGGL(latent_attn_rowwave_kernel<T>, grid, dim3(64), smem,
                       stream, (T*)out.data_ptr(), (const T*)q_lat.data_ptr(),
                       (long)q_lat.stride(0), (long)q_lat.stride(1),
                       (long)out.stride(0), (long)out.stride(1),
                       (const T*)cache.data_ptr(), page_table.data_ptr<int>(),
                       seq_lens.data_ptr<int>(), qs, ql, (float)scale,
                       (int)window, Rp, PS, max_pages);
  });
}

void sigmoid_gate_mul(torch::Tensor out, torch::Tensor a, torch::Tensor g) {
  TORCH_CHECK(a.dim() == 3 && a.stride(2) == 1 && g.dim() == 2 &&
              g.stride(1) == 1 && out.is_contiguous() && out.dim() == 2);
  TORCH_CHECK(a.scalar_type() == out.scalar_type() &&
              g.scalar_type() == out.scalar_type());
  const int H = a.size(0), T_ = a.size(1), E = a.size(2);
  TORCH_CHECK(out.size(0) == T_ && out.size(1) == (long)H * E);
  TORCH_CHECK(g.size(0) == T_ && g.size(1) == (long)H * E);
  const long n = (long)T_ * H * E;
  if (n == 0) return;
  const bool vec = E % 4 == 0 && a.stride(0) % 4 == 0 && a.stride(1) % 4 == 0 &&
                   a.storage_offset() % 4 == 0 && g.stride(0) % 4 == 0 &&
                   g.storage_offset() % 4 == 0;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((sigmoid_gate_mul_kernel<T, 4>),
                         dim3((n / 4 + 255) / 256), dim3(256), 0, stream,
                         (T*)out.data_ptr(), (const T*)a.data_ptr(),
                         (long)a.stride(0), (long)a.stride(1),
                         (const T*)g.data_ptr(), (long)g.stride(0), n, H, E);
    } else {
      hipLaunchKernelGGL((sigmoid_gate_mul_kernel<T, 1>),
                         dim3((n + 255) / 256), dim3(256), 0, stream,
                         (T*)out.data_ptr(), (const T*)a.data_ptr(),
                         (long)a.stride(0), (long)a.stride(1),
                         (const T*)g.data_ptr(), (long)g.stride(0), n, H, E);
    }
  });
}
