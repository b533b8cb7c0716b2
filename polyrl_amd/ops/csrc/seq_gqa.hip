// Grouped-query window attention over paged K/V rows: the cache writer and
// the any-dtype attention kernel.
//
// Cache row of a token (one per layer run): [G heads of D key numbers |
// G heads of Dv value numbers], activation type T (bf16 or fp32).
//
// gqa_prepare_kernel: one block per token.  Optional RMS norm over the WHOLE
// query projection (H*D numbers) and the whole key projection (G*D), each
// with its own weight vector; rotate-half rotary positions on the first
// 2*half entries of every head, angle = fp32(position) * inv_freq[i], cos
// and sin scaled by ``amp``; keys go to the cache row, queries to q_out;
// values are a separate projection or the key projection as it came in.
//
// gqa_attn_kernel: one wave per (token, head): decode steps in either type,
// and the exactness path (fp32 activations, odd head sizes).  A row at
// position p sees key j <= p when p - j < window or j < keep; the two key
// ranges [0, min(keep, lo)) and [lo, p] are walked as one list.  Scores, the
// optional distance-bucket bias rel[bucket[p-j], head], the online softmax
// and the per-head sigmoid gate are fp32.  Two further options: a sink, one
// learned logit per head that is one more term of the softmax denominator
// and adds nothing to the weighted sum (the running maximum starts at the
// sink, the running sum at one), and a query temperature that multiplies
// the score scale of the row at position p by
// 1 + coef * ln(floor((p + 1) / every) + 1).
//
// Further options of the writer (gqa_prepare_heads_kernel, one wave per
// head): every query and key head is divided by its own root mean square
// AFTER the rotation (no weight), and every value head is rotated over all
// its entries by its position (pairs (m, m + Dv/2)) before it is cached.
// Further options of the attention kernels: scores capped as
// cap * tanh(score / cap), a number per head added to the capped score, and
// weights sigmoid(score) per visible key with no normalisation over the
// keys (the running maximum and sum are then unused).  The head sums can be
// written as fp32 to a separate buffer for a pass that turns them back by
// the row's position.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

template <typename T>
__global__ __launch_bounds__(256) void gqa_prepare_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long ldq,
    const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
    const float* __restrict__ qn, const float* __restrict__ kn, float eps,
    const float* __restrict__ inv_freq, int half, float amp,
    const int* __restrict__ positions, T* __restrict__ cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int Dv) {
  __shared__ float red[8], red2[8];
  const long n = blockIdx.x;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  const T* qr = q + n * ldq;
  const T* kr = k + n * ldk;
  float inv_q = 1.f, inv_k = 1.f;
  if (qn) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) {
      const float f = ldf(qr + i);
      sq += f * f;
    }
    for (int i = threadIdx.x; i < nk; i += 256) {
      const float f = ldf(kr + i);
      sk += f * f;
    }
    sq = block_reduce_sum<4>(sq, red);
    sk = block_reduce_sum<4>(sk, red2);
    inv_q = rsqrtf(sq / nq + eps);
    inv_k = rsqrtf(sk / nk + eps);
  }
  const float pos = (float)positions[n];
  T* crow = cache + (long)slot_mapping[n] * (nk + nv);
  T* qo = q_out + n * nq;
  // queries, then keys: same treatment, different source / weight / target
  for (int part = 0; part < 2; ++part) {
    const T* src = part ? kr : qr;
    const float* wn = part ? kn : qn;
    const float inv = part ? inv_k : inv_q;
    T* dst = part ? crow : qo;
    const int cnt = part ? nk : nq;
    for (int i = threadIdx.x; i < cnt; i += 256) {
      const int d = i % D;
      if (d < half) {
        const int j = i + half;
        const float a = ldf(src + i) * inv * (wn ? wn[i] : 1.f);
        const float b = ldf(src + j) * inv * (wn ? wn[j] : 1.f);
        const float ang = pos * inv_freq[d];
        const float c = cosf(ang) * amp, s = sinf(ang) * amp;
        stf(dst + i, a * c - b * s);
        stf(dst + j, b * c + a * s);
      } else if (d >= 2 * half) {
        stf(dst + i, ldf(src + i) * inv * (wn ? wn[i] : 1.f));
      }
    }
  }
  const T* vr = v ? v + n * ldv : kr;
  for (int i = threadIdx.x; i < nv; i += 256) crow[nk + i] = vr[i];
}

// One wave per head of a token (H query heads, G key heads, G value heads;
// four heads a block, grid (tokens, heads / 4)).  Query / key heads: rotate the
// first 2*half entries, then (unit) divide the head by its root mean square;
// the statistics are taken of the rotated numbers, which are computed again
// for the store (nothing is rounded in between).  Value heads: rotate all Dv
// entries in halves with their own frequencies, or copy.
template <typename T>
__global__ __launch_bounds__(256) void gqa_prepare_heads_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long ldq,
    const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
    float eps, const float* __restrict__ inv_freq, int half, float amp,
    const float* __restrict__ v_freq, const int* __restrict__ positions,
    T* __restrict__ cache, const int* __restrict__ slot_mapping, int H, int G,
    int D, int Dv, bool unit) {
  const long n = blockIdx.x;
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float pos = (float)positions[n];
  T* crow = cache + (long)slot_mapping[n] * (G * (D + Dv));
  {
    const int hu = blockIdx.y * 4 + wid;
    if (hu >= H + 2 * G) return;          // whole wave; no barrier follows
    const T* src;
    T* dst;
    int dim, hf;
    const float* fr;
    float am;
    bool un;
    if (hu < H) {
      src = q + n * ldq + (long)hu * D;
      dst = q_out + (n * H + hu) * D;
      dim = D; hf = half; fr = inv_freq; am = amp; un = unit;
    } else if (hu < H + G) {
      src = k + n * ldk + (long)(hu - H) * D;
      dst = crow + (hu - H) * D;
      dim = D; hf = half; fr = inv_freq; am = amp; un = unit;
    } else {
      src = v + n * ldv + (long)(hu - H - G) * Dv;
      dst = crow + G * D + (hu - H - G) * Dv;
      dim = Dv; hf = v_freq ? Dv / 2 : 0; fr = v_freq; am = 1.f; un = false;
    }
    float inv = 1.f;
    if (un) {
      float ss = 0.f;
      for (int i = lane; i < hf; i += 64) {
        const float ang = pos * fr[i];
        const float c = cosf(ang) * am, s = sinf(ang) * am;
        const float a = ldf(src + i), b = ldf(src + i + hf);
        const float x = a * c - b * s, y = b * c + a * s;
        ss += x * x + y * y;
      }
      for (int i = 2 * hf + lane; i < dim; i += 64) {
        const float a = ldf(src + i);
        ss += a * a;
      }
      inv = rsqrtf(wave_reduce_sum(ss) / dim + eps);
    }
    for (int i = lane; i < hf; i += 64) {
      const float ang = pos * fr[i];
      const float c = cosf(ang) * am, s = sinf(ang) * am;
      const float a = ldf(src + i), b = ldf(src + i + hf);
      stf(dst + i, (a * c - b * s) * inv);
      stf(dst + i + hf, (b * c + a * s) * inv);
    }
    for (int i = 2 * hf + lane; i < dim; i += 64)
      stf(dst + i, ldf(src + i) * inv);
  }
}

void seq_gqa_prepare_store(torch::Tensor q_out, torch::Tensor q,
                           torch::Tensor k, torch::Tensor v,
                           torch::Tensor q_norm, torch::Tensor k_norm,
                           double eps, torch::Tensor inv_freq, double amp,
                           torch::Tensor positions, torch::Tensor cache,
                           torch::Tensor slot_mapping, int64_t H, int64_t G,
                           int64_t D, int64_t Dv, bool head_unit,
                           torch::Tensor v_inv_freq) {
  CHECK_ROWS(q);
  CHECK_ROWS(k);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  const long N = q.size(0);
  const bool has_v = v.defined() && v.numel() > 0;
  const bool has_norm = q_norm.defined() && q_norm.numel() > 0;
  const int half = inv_freq.defined() ? (int)inv_freq.numel() : 0;
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0);
  TORCH_CHECK(q.size(1) == H * D && k.size(0) == N && k.size(1) == G * D);
  TORCH_CHECK(2 * half <= D, "rotated entries exceed the head size");
  TORCH_CHECK(has_v || Dv == D, "keys serve as values only when Dv == D");
  auto ty = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == ty && cache.scalar_type() == ty &&
              q_out.scalar_type() == ty);
  if (has_v) {
    CHECK_ROWS(v);
    TORCH_CHECK(v.size(0) == N && v.size(1) == G * Dv && v.scalar_type() == ty);
  }
  if (has_norm) {
    CHECK_F32(q_norm);
    CHECK_F32(k_norm);
    TORCH_CHECK(q_norm.numel() == H * D && k_norm.numel() == G * D);
  }
  if (half) CHECK_F32(inv_freq);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == G * (D + Dv), "cache row must be G*(D+Dv)");
  TORCH_CHECK(q_out.is_cuda() && q_out.is_contiguous() &&
              q_out.numel() == N * H * D);
  TORCH_CHECK(positions.numel() == N && slot_mapping.numel() == N);
  if (N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const bool v_rot = v_inv_freq.defined() && v_inv_freq.numel() > 0;
  if (head_unit || v_rot) {
    TORCH_CHECK(!has_norm, "whole-row and per-head norms do not combine");
    TORCH_CHECK(has_v, "the per-head writer needs a value projection");
    if (v_rot) {
      CHECK_F32(v_inv_freq);
      TORCH_CHECK(Dv % 2 == 0 && v_inv_freq.numel() == Dv / 2,
                  "one frequency per value pair");
    }
    SEQ_DISPATCH_T(ty, { hipLaunchKernelGGL((gqa_prepare_heads_kernel<T>), dim3(N, (H + 2 * G + 3) / 4), dim3(256), 0, stream,
        (T*)q_out.data_ptr(), (const T*)q.data_ptr(), q.stride(0),
        (const T*)k.data_ptr(), k.stride(0), (const T*)v.data_ptr(),
        v.stride(0), (float)eps,
        half ? inv_freq.data_ptr<float>() : nullptr, half, (float)amp,
        v_rot ? v_inv_freq.data_ptr<float>() : nullptr,
        positions.data_ptr<int>(), (T*)cache.data_ptr(),
        slot_mapping.data_ptr<int>(), (int)H, (int)G, (int)D, (int)Dv,
        head_unit); });
    HIP_CHECK_KERNEL();
    return;
  }
  SEQ_DISPATCH_T(ty, { hipLaunchKernelGGL((gqa_prepare_kernel<T>), dim3(N), dim3(256), 0, stream,
      (T*)q_out.data_ptr(), (const T*)q.data_ptr(), q.stride(0),
      (const T*)k.data_ptr(), k.stride(0),
      has_v ? (const T*)v.data_ptr() : nullptr, has_v ? v.stride(0) : 0,
      has_norm ? q_norm.data_ptr<float>() : nullptr,
      has_norm ? k_norm.data_ptr<float>() : nullptr, (float)eps,
      half ? inv_freq.data_ptr<float>() : nullptr, half, (float)amp,
      positions.data_ptr<int>(), (T*)cache.data_ptr(),
      slot_mapping.data_ptr<int>(), (int)H, (int)G, (int)D, (int)Dv); });
  HIP_CHECK_KERNEL();
}

// dot(q_s[0..D), row[0..D)) with 16-byte loads when the rows allow them
template <typename T>
DEV_INLINE float dot_row(const T* __restrict__ r, const float* __restrict__ qs,
                         int D, bool vec);
template <>
DEV_INLINE float dot_row<bf16_t>(const bf16_t* __restrict__ r,
                                 const float* __restrict__ qs, int D,
                                 bool vec) {
  float acc = 0.f;
  if (vec) {
#pragma unroll 4
    for (int d = 0; d < D; d += 8) {
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(r + d);
#pragma unroll
      for (int k = 0; k < 8; ++k) acc += bf2f(v.v[k]) * qs[d + k];
    }
  } else {
    for (int d = 0; d < D; ++d) acc += bf2f(r[d]) * qs[d];
  }
  return acc;
}
template <>
DEV_INLINE float dot_row<float>(const float* __restrict__ r,
                                const float* __restrict__ qs, int D,
                                bool vec) {
  float acc = 0.f;
  if (vec) {
#pragma unroll 4
    for (int d = 0; d < D; d += 4) {
      const f32x4v v = *reinterpret_cast<const f32x4v*>(r + d);
#pragma unroll
      for (int k = 0; k < 4; ++k) acc += v.v[k] * qs[d + k];
    }
  } else {
    for (int d = 0; d < D; ++d) acc += r[d] * qs[d];
  }
  return acc;
}

// 16 bytes of a value row as floats
template <typename T>
struct Vec16;
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  static DEV_INLINE void load(const bf16_t* p, float* o) {
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = bf2f(v.v[k]);
  }
};
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  static DEV_INLINE void load(const float* p, float* o) {
    const f32x4v v = *reinterpret_cast<const f32x4v*>(p);
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = v.v[k];
  }
};

// One wave per (token, head), four heads of a token per block (they share
// their key/value group's rows in cache when H/G >= 4).  Keys are walked 64
// at a time in two phases: lane = key for the scores (each lane reads its
// key row against the query in LDS), then lane = value entry for the
// weighted sum (weights and row numbers from LDS).  When a value row is
// ``lpr`` 16-byte pieces with lpr a power of two, lpr lanes read one row and
// the wave reads 64/lpr rows per load; the lane groups' partial sums meet in
// a shuffle reduction at the end.  Otherwise (lpr = 0) the wave reads one
// value row per key.  The waves never meet at a block barrier.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void gqa_attn_kernel(
    T* __restrict__ out,                // (N, H*Dv)
    const T* __restrict__ q,            // (N, H*D) contiguous
    const T* __restrict__ cache,        // (pages*page_size, G*(D+Dv))
    const int* __restrict__ page_table, int max_pages,
    const int* __restrict__ seq_of_tok, const int* __restrict__ positions,
    const float* __restrict__ rel,      // (rows, H) or null
    const int* __restrict__ dist_bucket,   // (window,) or null
    const T* __restrict__ gate, long ldg,  // (N, H) view or null
    int H, int G, int D, int Dv, int page_size, int window, int keep,
    float scale, bool vec, int lpr, const float* __restrict__ sink,
    float qt_coef, int qt_every, float cap, const float* __restrict__ hbias,
    bool sigm, float* __restrict__ out32) {
  constexpr int EPL = Vec16<T>::N;
  __shared__ float q_sh[4][NCH * 64];
  __shared__ float p_sh[4][64];
  __shared__ int slot_sh[4][64];
  const long n = blockIdx.x;
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wid;
  if (h >= H) return;                   // whole wave
  const int g = h / (H / G);
  const int row = G * (D + Dv);
  const int koff = g * D, voff = G * D + g * Dv;
  const int pos = positions[n];
  const int b = seq_of_tok[n];
  const int* ptab = page_table + (long)b * max_pages;
  if (qt_coef != 0.f)
    scale *= 1.f + qt_coef * logf((float)((pos + 1) / qt_every + 1));
  const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;
  const int nkeep = keep < lo ? keep : lo;
  const int total = nkeep + (pos - lo + 1);
  float* qs = q_sh[wid];
  float* ps = p_sh[wid];
  int* ss = slot_sh[wid];
  for (int d = lane; d < D; d += 64) qs[d] = ldf(q + (n * H + h) * D + d);

  float o[NCH], ov[EPL];
#pragma unroll
  for (int c = 0; c < NCH; ++c) o[c] = 0.f;
#pragma unroll
  for (int k = 0; k < EPL; ++k) ov[k] = 0.f;
  float m = sink ? sink[h] : -INFINITY, l = sink ? 1.f : 0.f;
  const float hb = hbias ? hbias[h] : 0.f;
  const int kgrp = lpr ? lane / lpr : 0;          // key of an iteration
  const int dcol = lpr ? (lane % lpr) * EPL : 0;  // first value entry
  const int kper = lpr ? 64 / lpr : 1;            // keys per iteration

  for (int base = 0; base < total; base += 64) {
    const int i = base + lane;
    const bool valid = i < total;
    const int ii = valid ? i : total - 1;
    const int j = ii < nkeep ? ii : lo + (ii - nkeep);
    const int slot = ptab[j / page_size] * page_size + j % page_size;
    float s = dot_row<T>(cache + (long)slot * row + koff, qs, D, vec) * scale;
    if (rel) s += rel[(long)dist_bucket[pos - j] * H + h];
    if (cap > 0.f) s = cap * tanhf(s / cap);
    s += hb;
    if (!valid) s = -INFINITY;
    float p, corr;
    if (sigm) {
      p = valid ? sigmoidf_acc(s) : 0.f;
      corr = 1.f;
    } else {
      const float mn = fmaxf(m, wave_reduce_max(s));
      p = valid ? expf(s - mn) : 0.f;
      corr = expf(m - mn);
      l = l * corr + wave_reduce_sum(p);
      m = mn;
    }
    ps[lane] = p;
    ss[lane] = slot;
    const int cntk = total - base < 64 ? total - base : 64;
    if (lpr) {
#pragma unroll
      for (int k = 0; k < EPL; ++k) ov[k] *= corr;
#pragma unroll 4
      for (int jj0 = 0; jj0 < cntk; jj0 += kper) {
        const int jj = jj0 + kgrp;
        if (jj < cntk) {
          const float pj = ps[jj];
          float vv[EPL];
          Vec16<T>::load(cache + (long)ss[jj] * row + voff + dcol, vv);
#pragma unroll
          for (int k = 0; k < EPL; ++k) ov[k] += pj * vv[k];
        }
      }
      continue;
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) o[c] *= corr;
#pragma unroll 4
    for (int jj = 0; jj < cntk; ++jj) {
      const float pj = ps[jj];
      const T* vr = cache + (long)ss[jj] * row + voff;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = lane + 64 * c;
        if (d < Dv) o[c] += pj * ldf(vr + d);
      }
    }
  }
  float inv = sigm ? 1.f : 1.f / l;
  if (gate && !out32) inv *= sigmoidf_acc(ldf(gate + n * ldg + h));
  if (lpr) {
#pragma unroll
    for (int k = 0; k < EPL; ++k)
      for (int off = lpr; off < 64; off <<= 1)
        ov[k] += __shfl_xor(ov[k], off, WAVE_SIZE);
    if (lane < lpr) {
#pragma unroll
      for (int k = 0; k < EPL; ++k) {
        if (out32) out32[(n * H + h) * Dv + dcol + k] = ov[k] * inv;
        else stf(out + (n * H + h) * Dv + dcol + k, ov[k] * inv);
      }
    }
    return;
  }
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d = lane + 64 * c;
    if (d < Dv) {
      if (out32) out32[(n * H + h) * Dv + d] = o[c] * inv;
      else stf(out + (n * H + h) * Dv + d, o[c] * inv);
    }
  }
}

void seq_rotate_back_heads(torch::Tensor out, torch::Tensor x,
                           torch::Tensor inv_freq, torch::Tensor positions,
                           torch::Tensor gate, int64_t H);

// shared argument checks of both attention entry points
void gqa_attention_check(torch::Tensor out, torch::Tensor q,
                         torch::Tensor cache, torch::Tensor page_table,
                         torch::Tensor seq_of_tok, torch::Tensor positions,
                         int64_t H, int64_t G, int64_t D, int64_t Dv,
                         int64_t window, int64_t keep_first,
                         torch::Tensor rel, torch::Tensor dist_bucket,
                         torch::Tensor gate, torch::Tensor sink,
                         int64_t q_temp_every) {
  CHECK_I32(page_table); CHECK_I32(seq_of_tok); CHECK_I32(positions);
  const long N = q.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && window >= 1 &&
              keep_first >= 0);
  TORCH_CHECK(q.is_cuda() && q.is_contiguous() && q.dim() == 2 &&
              q.size(1) == H * D);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 &&
              out.size(0) == N && out.size(1) == H * Dv);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == G * (D + Dv), "cache row must be G*(D+Dv)");
  auto ty = q.scalar_type();
  TORCH_CHECK(cache.scalar_type() == ty && out.scalar_type() == ty);
  TORCH_CHECK(page_table.dim() == 2 && seq_of_tok.numel() == N &&
              positions.numel() == N);
  const bool has_rel = rel.defined() && rel.numel() > 0;
  if (has_rel) {
    CHECK_F32(rel);
    CHECK_I32(dist_bucket);
    TORCH_CHECK(rel.dim() == 2 && rel.size(1) == H);
    TORCH_CHECK(dist_bucket.numel() >= window && keep_first == 0,
                "the distance table must cover the window");
  }
  if (gate.defined() && gate.numel() > 0) {
    CHECK_ROWS(gate);
    TORCH_CHECK(gate.size(0) == N && gate.size(1) == H &&
                gate.scalar_type() == ty);
  }
  if (sink.defined() && sink.numel() > 0) {
    CHECK_F32(sink);
    TORCH_CHECK(sink.numel() == H, "one sink per query head");
  }
  TORCH_CHECK(q_temp_every >= 1, "query temperature period");
}

#define GQA_LAUNCH(NCHV)                                                      \
  hipLaunchKernelGGL((gqa_attn_kernel<T, NCHV>), dim3(N, (H + 3) / 4),       \
      dim3(256), 0, stream, (T*)out.data_ptr(), (const T*)q.data_ptr(),                     \
      (const T*)cache.data_ptr(), page_table.data_ptr<int>(),                 \
      (int)page_table.size(1), seq_of_tok.data_ptr<int>(),                    \
      positions.data_ptr<int>(), has_rel ? rel.data_ptr<float>() : nullptr,   \
      has_rel ? dist_bucket.data_ptr<int>() : nullptr,                        \
      has_gate ? (const T*)gate.data_ptr() : nullptr,                         \
      has_gate ? gate.stride(0) : 0, (int)H, (int)G, (int)D, (int)Dv,         \
      (int)cache.size(1), (int)window, (int)keep_first, (float)scale, vec,     \
      lpr, has_sink ? sink.data_ptr<float>() : nullptr, (float)q_temp_coef,   \
      (int)q_temp_every, (float)softcap,                                      \
      has_hb ? head_bias.data_ptr<float>() : nullptr, sigmoid_weights,        \
      o32)

void seq_gqa_window_attention(torch::Tensor out, torch::Tensor q,
                              torch::Tensor cache, torch::Tensor page_table,
                              torch::Tensor seq_of_tok,
                              torch::Tensor positions, int64_t H, int64_t G,
                              int64_t D, int64_t Dv, int64_t window,
                              int64_t keep_first, torch::Tensor rel,
                              torch::Tensor dist_bucket, torch::Tensor gate,
                              double scale, torch::Tensor sink,
                              double q_temp_coef, int64_t q_temp_every,
                              double softcap, torch::Tensor head_bias,
                              bool sigmoid_weights, torch::Tensor v_inv_freq) {
  gqa_attention_check(out, q, cache, page_table, seq_of_tok, positions, H, G,
                      D, Dv, window, keep_first, rel, dist_bucket, gate, sink,
                      q_temp_every);
  const int N = q.size(0);
  if (N == 0) return;
  const bool has_hb = head_bias.defined() && head_bias.numel() > 0;
  if (has_hb) {
    CHECK_F32(head_bias);
    TORCH_CHECK(head_bias.numel() == H, "one bias per query head");
  }
  TORCH_CHECK(!sigmoid_weights || !(sink.defined() && sink.numel() > 0),
              "a sink needs softmax weights");
  // rotated values: the head sums leave as fp32 and a second pass turns
  // them back by the row's position (and applies the gate)
  const bool v_rot = v_inv_freq.defined() && v_inv_freq.numel() > 0;
  torch::Tensor sums;
  float* o32 = nullptr;
  if (v_rot) {
    sums = torch::empty({q.size(0), H * Dv}, q.options().dtype(torch::kFloat32));
    o32 = sums.data_ptr<float>();
  }
  const bool has_sink = sink.defined() && sink.numel() > 0;
  const bool has_rel = rel.defined() && rel.numel() > 0;
  const bool has_gate = gate.defined() && gate.numel() > 0;
  const int nch = (int)((std::max(D, Dv) + 63) / 64);
  TORCH_CHECK(nch <= 8, "head sizes above 512 are not supported");
  // 16-byte row loads need every head's keys to start on a 16-byte border
  const int per16 = q.scalar_type() == torch::kBFloat16 ? 8 : 4;
  const bool vec = D % per16 == 0 && Dv % per16 == 0;
  // lanes per value row of 16-byte pieces, when that is a power of two <= 64
  int lpr = vec ? (int)(Dv / per16) : 0;
  if (lpr > 64 || (lpr & (lpr - 1))) lpr = 0;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(q.scalar_type(), {
    switch (nch) {
      case 1: GQA_LAUNCH(1); break;
      case 2: GQA_LAUNCH(2); break;
      case 3: case 4: GQA_LAUNCH(4); break;
      default: GQA_LAUNCH(8); break;
    }
  });
  HIP_CHECK_KERNEL();
  if (v_rot) seq_rotate_back_heads(out, sums, v_inv_freq, positions, gate, H);
}
