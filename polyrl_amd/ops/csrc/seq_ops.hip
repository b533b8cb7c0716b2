// Row-wise kernels of the hybrid decoders: fp32-residual add + RMS norms,
// the composed embedding (scaled row + hashed pair row + sinusoid), stateful
// depthwise causal convolution, grouped RMS norm with an optional sigmoid or
// SiLU gate, partial rotary embedding, the latent-cache writer, gated
// activations, and the expert-output combine.
//
// Activations are T (bf16 or fp32); the residual stream, norm statistics,
// convolution histories and all transcendental math are fp32.  These ops are
// HBM-bound: one block per row (or a flat grid-stride loop), no LDS staging
// beyond the block reductions.  Reference semantics: ops/seq_ref.py.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

// ------------------------------------------------- residual add + RMS norm
// g[i] = off + w[i] (w holds 1 or D numbers; off = 0 for plain weights, 1 for
// weights stored around zero)
// mode 0: res += ys*y [+ ex] [+ exv]; out = res * rsqrt(mean(res^2)+eps) * g
// mode 1: res += ys*y; out = res (cast)                          (no norm)
// mode 2: res += ys * y * rsqrt(mean(y^2)+eps) * g               (out unused)
// mode 3: mode 2 [+ ex] [+ exv], then out = res * rsqrt(mean(res^2)+eps)
//         * (off + w2)  (the joint between two normed sublayers in one pass)
// ys scales the branch that joins the stream; ex (rows, D) fp32 and exv (D)
// fp32 are what a pass of a looped span adds at its start.
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ y,
    long ldy, const float* __restrict__ w, int wn, int D, float eps,
    int mode, bool out_is_res, float off, const float* __restrict__ w2,
    int w2n, float ys, const float* __restrict__ ex,
    const float* __restrict__ exv) {
  __shared__ float red[8], red2[8];
  const long row = blockIdx.x;
  float* rr = res + row * D;
  const T* yr = y ? y + row * ldy : nullptr;
  float ss = 0.f;
  if (mode >= 2) {
    for (int i = threadIdx.x; i < D; i += 256) {
      const float f = ldf(yr + i);
      ss += f * f;
    }
  } else {
    const float* er = ex ? ex + row * D : nullptr;
    for (int i = threadIdx.x; i < D; i += 256) {
      float f = rr[i];
      if (yr) f += ys * ldf(yr + i);
      if (er) f += er[i];
      if (exv) f += exv[i];
      if (yr || er || exv) rr[i] = f;
      ss += f * f;
    }
  }
  if (mode == 1) {
    if (!out_is_res)
      for (int i = threadIdx.x; i < D; i += 256)
        stf(out + row * D + i, rr[i]);   // own writes: same thread, same i
    return;
  }
  ss = block_reduce_sum<4>(ss, red);
  const float inv = rsqrtf(ss / D + eps);
  if (mode == 0) {
    for (int i = threadIdx.x; i < D; i += 256)
      stf(out + row * D + i, rr[i] * inv * (w[wn == 1 ? 0 : i] + off));
    return;
  }
  float ss2 = 0.f;
  const float* er3 = ex ? ex + row * D : nullptr;
  for (int i = threadIdx.x; i < D; i += 256) {
    float f = rr[i] + ys * (ldf(yr + i) * inv * (w[wn == 1 ? 0 : i] + off));
    if (er3) f += er3[i];
    if (exv) f += exv[i];
    rr[i] = f;
    ss2 += f * f;
  }
  if (mode == 2) return;
  ss2 = block_reduce_sum<4>(ss2, red2);
  const float inv2 = rsqrtf(ss2 / D + eps);
  for (int i = threadIdx.x; i < D; i += 256)   // own writes again
    stf(out + row * D + i, rr[i] * inv2 * (w2[w2n == 1 ? 0 : i] + off));
}

void seq_add_rmsnorm(torch::Tensor out, torch::Tensor res, torch::Tensor y,
                     torch::Tensor weight, double eps, int64_t mode,
                     double offset, torch::Tensor weight2, double y_scale,
                     torch::Tensor extra, torch::Tensor extra_vec) {
  CHECK_F32(res);
  TORCH_CHECK(res.dim() == 2);
  const int D = res.size(1);
  const long rows = res.size(0);
  if (rows == 0) return;
  const bool has_y = y.defined() && y.numel() > 0;
  if (has_y) {
    CHECK_ROWS(y);
    TORCH_CHECK(y.size(0) == rows && y.size(1) == D, "y shape");
  }
  TORCH_CHECK(mode >= 0 && mode <= 3);
  TORCH_CHECK(mode < 2 || has_y);
  const float* w = nullptr;
  const float* w2 = nullptr;
  int wn = 0, w2n = 0;
  if (mode != 1) {
    CHECK_F32(weight);
    wn = weight.numel();
    TORCH_CHECK(wn == 1 || wn == D, "norm weight must hold 1 or D numbers");
    w = weight.data_ptr<float>();
  }
  if (mode == 3) {
    CHECK_F32(weight2);
    w2n = weight2.numel();
    TORCH_CHECK(w2n == 1 || w2n == D, "norm weight must hold 1 or D numbers");
    w2 = weight2.data_ptr<float>();
  }
  const float* ex = nullptr;
  const float* exv = nullptr;
  if (extra.defined() && extra.numel() > 0) {
    CHECK_F32(extra);
    TORCH_CHECK((mode == 0 || mode == 3) && extra.numel() == res.numel(),
                "extra shape");
    ex = extra.data_ptr<float>();
  }
  if (extra_vec.defined() && extra_vec.numel() > 0) {
    CHECK_F32(extra_vec);
    TORCH_CHECK((mode == 0 || mode == 3) && extra_vec.numel() == D,
                "extra_vec shape");
    exv = extra_vec.data_ptr<float>();
  }
  const bool out_is_res = out.data_ptr() == res.data_ptr();
  TORCH_CHECK(mode != 3 || !out_is_res);
  if (mode != 2) {
    TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
                out.numel() == res.numel());
  }
  auto dt = mode == 2 ? y.scalar_type()
                      : (out_is_res ? (has_y ? y.scalar_type()
                                             : torch::kFloat32)
                                    : out.scalar_type());
  if (has_y) TORCH_CHECK(y.scalar_type() == dt, "y / out dtype mismatch");
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(dt, { hipLaunchKernelGGL((add_rmsnorm_kernel<T>), dim3(rows), dim3(256), 0, stream, 
      mode == 2 || out_is_res ? nullptr : (T*)out.data_ptr(),
      res.data_ptr<float>(), has_y ? (const T*)y.data_ptr() : nullptr,
      has_y ? y.stride(0) : 0, w, wn, D, (float)eps, (int)mode, out_is_res,
      (float)offset, w2, w2n, (float)y_scale, ex, exv); });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------ composed embedding
// out[n] = table[tok] * scale [+ pair[row]] [+ sinusoid(pos)], fp32.
// row = (prev * mul_prev + tok * mul_cur) mod buckets, or ``buckets`` (the
// table's last row) where prev < 0.  Sinusoid: sin(a_i) at the even entry
// 2i and cos(a_i) at the odd one, a_i = fp32(pos) * inv_freq[i].
template <typename T>
__global__ __launch_bounds__(256) void embed_compose_kernel(
    float* __restrict__ out, const T* __restrict__ table,
    const long* __restrict__ tokens, float scale, const T* __restrict__ pair,
    const long* __restrict__ prev, long mul_prev, long mul_cur, long buckets,
    const int* __restrict__ pos, const float* __restrict__ inv_freq, int D) {
  const long n = blockIdx.x;
  const long tok = tokens[n];
  const T* er = table + tok * D;
  const T* pr = nullptr;
  if (pair) {
    const long pv = prev[n];
    const long row = pv < 0 ? buckets : (pv * mul_prev + tok * mul_cur) % buckets;
    pr = pair + row * D;
  }
  const float p = inv_freq ? (float)pos[n] : 0.f;
  for (int i = threadIdx.x; i < D; i += 256) {
    float f = ldf(er + i) * scale;
    if (pr) f += ldf(pr + i);
    if (inv_freq) {
      const float ang = p * inv_freq[i >> 1];
      f += (i & 1) ? cosf(ang) : sinf(ang);
    }
    out[n * D + i] = f;
  }
}

void seq_embed_compose(torch::Tensor out, torch::Tensor table,
                       torch::Tensor tokens, double scale,
                       torch::Tensor pair_table, torch::Tensor prev_tokens,
                       int64_t mul_prev, int64_t mul_cur, int64_t buckets,
                       torch::Tensor positions, torch::Tensor inv_freq) {
  CHECK_F32(out);
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2);
  TORCH_CHECK(tokens.is_cuda() && tokens.dtype() == torch::kInt64 &&
              tokens.is_contiguous());
  const long N = tokens.numel();
  const int D = table.size(1);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == N && out.size(1) == D);
  const bool has_pair = pair_table.defined() && pair_table.numel() > 0;
  if (has_pair) {
    TORCH_CHECK(pair_table.is_cuda() && pair_table.is_contiguous() &&
                pair_table.dim() == 2 && pair_table.size(1) == D &&
                pair_table.scalar_type() == table.scalar_type());
    TORCH_CHECK(buckets > 0 && pair_table.size(0) == buckets + 1,
                "the pair table holds buckets + 1 rows");
    TORCH_CHECK(mul_prev >= 0 && mul_cur >= 0);
    TORCH_CHECK(prev_tokens.is_cuda() && prev_tokens.dtype() == torch::kInt64 &&
                prev_tokens.is_contiguous() && prev_tokens.numel() == N);
  }
  const bool has_pos = inv_freq.defined() && inv_freq.numel() > 0;
  if (has_pos) {
    CHECK_F32(inv_freq);
    CHECK_I32(positions);
    TORCH_CHECK(inv_freq.numel() == (D + 1) / 2 && positions.numel() == N);
  }
  if (N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(table.scalar_type(), {
    hipLaunchKernelGGL((embed_compose_kernel<T>), dim3(N), dim3(256), 0,
        stream, out.data_ptr<float>(), (const T*)table.data_ptr(),
        (const long*)tokens.data_ptr<int64_t>(), (float)scale,
        has_pair ? (const T*)pair_table.data_ptr() : nullptr,
        has_pair ? (const long*)prev_tokens.data_ptr<int64_t>() : nullptr,
        (long)mul_prev, (long)mul_cur, (long)buckets,
        has_pos ? positions.data_ptr<int>() : nullptr,
        has_pos ? inv_freq.data_ptr<float>() : nullptr, D); });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------- stateful causal convolution
// y_t = sum_j w[c, j] * x_(t - taps + 1 + j) (+ bias) (+ x_t) (silu)
// history before the portion's first row comes from state[slot] (taps-1, C)
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    T* __restrict__ out, const T* __restrict__ x, long ldx,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slot, const int* __restrict__ seq_of_tok,
    int C, int taps, bool add_input, bool act_silu) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = seq_of_tok[n];
  const int q0 = cu_q[b];
  const int t = n - q0;
  const float* st = state + (long)state_slot[b] * (taps - 1) * C;
  float acc = bias ? bias[c] : 0.f;
  float cur = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = t - (taps - 1) + j;
    const float v = src >= 0 ? ldf(x + (long)(q0 + src) * ldx + c)
                             : st[(long)(taps - 1 + src) * C + c];
    acc += w[(long)c * taps + j] * v;
    cur = v;
  }
  if (add_input) acc += cur;
  if (act_silu) acc = siluf_acc(acc);
  stf(out + (long)n * C + c, acc);
}

// new history = last taps-1 rows of [old history ; portion].  Ascending
// order is safe in place: row i reads old row i+L (L >= 1), never a row
// already overwritten; each thread owns one channel column.
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(
    float* __restrict__ state, const T* __restrict__ x, long ldx,
    const int* __restrict__ cu_q, const int* __restrict__ state_slot, int C,
    int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int q0 = cu_q[b];
  const int L = cu_q[b + 1] - q0;
  if (L <= 0) return;
  float* st = state + (long)state_slot[b] * (taps - 1) * C;
  for (int i = 0; i < taps - 1; ++i) {
    const int h = L + i;                      // index into [old ; portion]
    st[(long)i * C + c] = h < taps - 1
                              ? st[(long)h * C + c]
                              : ldf(x + (long)(q0 + h - (taps - 1)) * ldx + c);
  }
}

void seq_causal_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                     torch::Tensor bias, torch::Tensor state,
                     torch::Tensor cu_q, torch::Tensor state_slot,
                     torch::Tensor seq_of_tok, bool add_input, bool act_silu) {
  CHECK_ROWS(x);
  CHECK_F32(w);
  CHECK_F32(state);
  CHECK_I32(cu_q);
  CHECK_I32(state_slot);
  CHECK_I32(seq_of_tok);
  const int N = x.size(0), C = w.size(0), taps = w.size(1);
  TORCH_CHECK(x.size(1) == C && out.is_contiguous() && out.size(0) == N &&
              out.size(1) == C && out.scalar_type() == x.scalar_type());
  TORCH_CHECK(taps >= 1 && state.dim() == 3 && state.size(1) == taps - 1 &&
              state.size(2) == C, "state must be (slots, taps-1, C)");
  TORCH_CHECK(seq_of_tok.numel() == N && cu_q.numel() == state_slot.numel() + 1);
  const float* bp = nullptr;
  if (bias.defined() && bias.numel() > 0) {
    CHECK_F32(bias);
    TORCH_CHECK(bias.numel() == C);
    bp = bias.data_ptr<float>();
  }
  const int B = state_slot.numel();
  auto stream = at::hip::getCurrentHIPStream();
  const int cb = (C + 255) / 256;
  SEQ_DISPATCH_T(x.scalar_type(), {
    hipLaunchKernelGGL((causal_conv_kernel<T>), dim3(N, cb), dim3(256), 0, stream, 
        (T*)out.data_ptr(), (const T*)x.data_ptr(), x.stride(0),
        w.data_ptr<float>(), bp, state.data_ptr<float>(),
        cu_q.data_ptr<int>(), state_slot.data_ptr<int>(),
        seq_of_tok.data_ptr<int>(), C, taps, add_input, act_silu);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_kernel<T>), dim3(B, cb), dim3(256), 0, stream, 
          state.data_ptr<float>(), (const T*)x.data_ptr(), x.stride(0),
          cu_q.data_ptr<int>(), state_slot.data_ptr<int>(), C, taps);
  });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------ grouped RMS norm (+gate)
// out = y / rms_group(y) * w * (gate ? sigmoid(gate) or silu(gate) : 1); w
// holds D numbers or one group's worth shared by all groups.  Small groups
// (heads): one wave per (row, group), grid.y covers the groups four at a
// time.  Large groups (BLOCK): the whole block reduces one (row, group).
template <typename T, bool BLOCK>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(
    T* __restrict__ out, const float* __restrict__ y,
    const float* __restrict__ w, const T* __restrict__ gate, long ldg, int D,
    int groups, float eps, bool w_shared, int gate_act) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int gs = D / groups;
  const int g = BLOCK ? blockIdx.y : blockIdx.y * 4 + wid;
  if (g >= groups) return;                  // wave-uniform (block-uniform)
  const int t0 = BLOCK ? threadIdx.x : lane;
  const int step = BLOCK ? 256 : 64;
  const float* yr = y + row * D + (long)g * gs;
  float ss = 0.f;
  for (int i = t0; i < gs; i += step) ss += yr[i] * yr[i];
  ss = BLOCK ? block_reduce_sum<4>(ss, red) : wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / gs + eps);
  for (int i = t0; i < gs; i += step) {
    const int c = g * gs + i;
    float v = yr[i] * inv * w[w_shared ? i : c];
    if (gate) {
      const float gv = ldf(gate + row * ldg + c);
      v *= gate_act == 2 ? siluf_acc(gv) : sigmoidf_acc(gv);
    }
    stf(out + row * D + c, v);
  }
}

void seq_group_rmsnorm(torch::Tensor out, torch::Tensor y,
                       torch::Tensor weight, int64_t groups, double eps,
                       torch::Tensor gate, int64_t gate_act) {
  CHECK_F32(y);
  CHECK_F32(weight);
  TORCH_CHECK(y.dim() == 2 && out.is_contiguous() && out.sizes() == y.sizes());
  const int D = y.size(1);
  TORCH_CHECK(groups >= 1 && D % groups == 0 &&
              (weight.numel() == D || weight.numel() == D / groups));
  TORCH_CHECK(gate_act == 1 || gate_act == 2);
  const bool w_shared = weight.numel() != D;
  const bool has_g = gate.defined() && gate.numel() > 0;
  if (has_g) {
    CHECK_ROWS(gate);
    TORCH_CHECK(gate.size(0) == y.size(0) && gate.size(1) == D &&
                gate.scalar_type() == out.scalar_type());
  }
  if (y.size(0) == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const bool big = D / groups >= 512;
  const dim3 grid(y.size(0), big ? groups : (groups + 3) / 4);
  SEQ_DISPATCH_T(out.scalar_type(), {
    if (big)
      hipLaunchKernelGGL((group_rmsnorm_kernel<T, true>), grid, dim3(256), 0,
          stream, (T*)out.data_ptr(), y.data_ptr<float>(),
          weight.data_ptr<float>(),
          has_g ? (const T*)gate.data_ptr() : nullptr,
          has_g ? gate.stride(0) : 0, D, (int)groups, (float)eps, w_shared,
          (int)gate_act);
    else
      hipLaunchKernelGGL((group_rmsnorm_kernel<T, false>), grid, dim3(256), 0,
          stream, (T*)out.data_ptr(), y.data_ptr<float>(),
          weight.data_ptr<float>(),
          has_g ? (const T*)gate.data_ptr() : nullptr,
          has_g ? gate.stride(0) : 0, D, (int)groups, (float)eps, w_shared,
          (int)gate_act);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------- partial rotary (q)
// q (N, H, Dh) with token stride ldn: rotate the pair (off+i, off+i+half),
// or (off+2i, off+2i+1) when the pairs are interleaved, by angle
// fp32(pos) * inv_freq[i]; cos and sin are multiplied by amp.
template <typename T>
__global__ void rope_partial_kernel(T* __restrict__ q, long ldn, int H, int Dh,
                                    int off, const float* __restrict__ inv_freq,
                                    int half, const int* __restrict__ pos,
                                    long total, float amp, bool inter) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int i = idx % half;
  const int h = (idx / half) % H;
  const long n = idx / ((long)half * H);
  const float ang = (float)pos[n] * inv_freq[i];
  const float c = cosf(ang) * amp, s = sinf(ang) * amp;
  T* p = q + n * ldn + (long)h * Dh + off + (inter ? 2 * i : i);
  const int step = inter ? 1 : half;
  const float a = ldf(p), b = ldf(p + step);
  stf(p, a * c - b * s);
  stf(p + step, b * c + a * s);
}

void seq_rope_partial(torch::Tensor q, int64_t offset, torch::Tensor inv_freq,
                      torch::Tensor positions, double amp, bool interleaved) {
  CHECK_F32(inv_freq);
  CHECK_I32(positions);
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.stride(2) == 1 &&
              q.stride(1) == q.size(2), "q must be (N, H, Dh), heads packed");
  const int half = inv_freq.numel();
  TORCH_CHECK(offset >= 0 && offset + 2 * half <= q.size(2));
  TORCH_CHECK(positions.numel() == q.size(0));
  const long total = (long)q.size(0) * q.size(1) * half;
  if (total == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(q.scalar_type(), { hipLaunchKernelGGL((rope_partial_kernel<T>), dim3((total + 255) / 256), dim3(256), 0, stream, 
      (T*)q.data_ptr(), q.stride(0), (int)q.size(1), (int)q.size(2),
      (int)offset, inv_freq.data_ptr<float>(), half,
      positions.data_ptr<int>(), total, (float)amp, interleaved); });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------ latent cache store
// one wave per token: RMS-norm the latent (first R columns) times norm_w,
// rotate the first 2*half columns of the key part (pairs in halves or
// interleaved, cos/sin times amp), write the cache row.
template <typename T>
__global__ __launch_bounds__(64) void latent_store_kernel(
    const T* __restrict__ dkv, long ld, int R, int rd,
    const float* __restrict__ norm_w, float eps, const int* __restrict__ pos,
    const float* __restrict__ inv_freq, int half, T* __restrict__ cache,
    const int* __restrict__ slot_mapping, float amp, bool inter) {
  const long n = blockIdx.x;
  const int lane = threadIdx.x;
  const int slot = slot_mapping[n];
  if (slot < 0) return;
  const T* src = dkv + n * ld;
  T* dst = cache + (long)slot * (R + rd);
  float ss = 0.f;
  for (int i = lane; i < R; i += 64) {
    const float f = ldf(src + i);
    ss += f * f;
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / R + eps);
  for (int i = lane; i < R; i += 64) stf(dst + i, ldf(src + i) * inv * norm_w[i]);
  const float p = (float)pos[n];
  for (int i = lane; i < half; i += 64) {
    const float ang = p * inv_freq[i];
    const float c = cosf(ang) * amp, s = sinf(ang) * amp;
    const int ia = inter ? 2 * i : i, ib = inter ? 2 * i + 1 : i + half;
    const float a = ldf(src + R + ia), b = ldf(src + R + ib);
    stf(dst + R + ia, a * c - b * s);
    stf(dst + R + ib, b * c + a * s);
  }
  for (int i = 2 * half + lane; i < rd; i += 64) stf(dst + R + i, ldf(src + R + i));
}

void seq_latent_kv_store(torch::Tensor dkv, int64_t rank, torch::Tensor norm_w,
                         double eps, torch::Tensor positions,
                         torch::Tensor inv_freq, torch::Tensor cache,
                         torch::Tensor slot_mapping, double amp,
                         bool interleaved) {
  CHECK_ROWS(dkv);
  CHECK_F32(norm_w);
  CHECK_F32(inv_freq);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  const int N = dkv.size(0), row = dkv.size(1);
  const int half = inv_freq.numel();
  TORCH_CHECK(rank > 0 && rank <= row && norm_w.numel() == rank);
  TORCH_CHECK(2 * half <= row - rank);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == row && cache.scalar_type() == dkv.scalar_type());
  TORCH_CHECK(positions.numel() == N && slot_mapping.numel() == N);
  if (N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(dkv.scalar_type(), { hipLaunchKernelGGL((latent_store_kernel<T>), dim3(N), dim3(64), 0, stream, 
      (const T*)dkv.data_ptr(), dkv.stride(0), (int)rank, (int)(row - rank),
      norm_w.data_ptr<float>(), (float)eps, positions.data_ptr<int>(),
      inv_freq.data_ptr<float>(), half, (T*)cache.data_ptr(),
      slot_mapping.data_ptr<int>(), (float)amp, interleaved); });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------- gated activations
// mode 0: silu(a) * b   mode 1: sigmoid(a) * b   mode 2: tanh(a)
// mode 3: gelu(a), the exact (erf) form
// mode 4: g * sigmoid(p1 * g) * (u + p2), g = min(a, p0), u = clamp(b, +-p0)
template <typename T>
__global__ void act_mul_kernel(T* __restrict__ out, const T* __restrict__ a,
                               long lda, const T* __restrict__ b, long ldb,
                               long rows, int cols, int mode, float p0,
                               float p1, float p2) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  const long n = rows * cols;
  for (; i < n; i += stride) {
    const long r = i / cols;
    const int c = i % cols;
    const float av = ldf(a + r * lda + c);
    float v;
    if (mode == 2) {
      v = tanhf(av);
    } else if (mode == 3) {
      v = gelu_erff_acc(av);
    } else if (mode == 4) {
      const float g = fminf(av, p0);
      const float u = fminf(fmaxf(ldf(b + r * ldb + c), -p0), p0);
      v = g * sigmoidf_acc(p1 * g) * (u + p2);
    } else {
      const float bv = ldf(b + r * ldb + c);
      v = (mode == 0 ? siluf_acc(av) : sigmoidf_acc(av)) * bv;
    }
    stf(out + i, v);
  }
}

void seq_act_mul(torch::Tensor out, torch::Tensor a, torch::Tensor b,
                 int64_t mode, double p0, double p1, double p2) {
  CHECK_ROWS(a);
  CHECK_ROWS(b);
  TORCH_CHECK(a.sizes() == b.sizes() && out.is_contiguous() &&
              out.sizes() == a.sizes() &&
              a.scalar_type() == b.scalar_type() &&
              out.scalar_type() == a.scalar_type());
  const long rows = a.size(0);
  const int cols = a.size(1);
  if (rows * cols == 0) return;
  const long nblk = std::min<long>((rows * cols + 255) / 256, MAX_RESIDENT_BLOCKS * 4);
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(a.scalar_type(), { hipLaunchKernelGGL((act_mul_kernel<T>), dim3(nblk), dim3(256), 0, stream, 
      (T*)out.data_ptr(), (const T*)a.data_ptr(), a.stride(0),
      (const T*)b.data_ptr(), b.stride(0), rows, cols, (int)mode, (float)p0,
      (float)p1, (float)p2); });
  HIP_CHECK_KERNEL();
}

// out = gelu_tanh(gate) * table[tokens[n], col0 + c]
template <typename T>
__global__ void gelu_mul_rows_kernel(T* __restrict__ out,
                                     const T* __restrict__ gate, long ldg,
                                     const T* __restrict__ table, long ldt,
                                     const long* __restrict__ tokens, int col0,
                                     long rows, int cols) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  const long r = i / cols;
  const int c = i % cols;
  const float z = ldf(gate + r * ldg + c);
  const float e = ldf(table + tokens[r] * ldt + col0 + c);
  stf(out + i, gelu_tanhf_acc(z) * e);
}

void seq_gelu_mul_rows(torch::Tensor out, torch::Tensor gate,
                       torch::Tensor table, torch::Tensor tokens,
                       int64_t col0) {
  CHECK_ROWS(gate);
  CHECK_ROWS(table);
  TORCH_CHECK(tokens.is_cuda() && tokens.dtype() == torch::kInt64 &&
              tokens.is_contiguous() && tokens.numel() == gate.size(0));
  TORCH_CHECK(out.is_contiguous() && out.sizes() == gate.sizes() &&
              table.scalar_type() == gate.scalar_type() &&
              out.scalar_type() == gate.scalar_type());
  TORCH_CHECK(col0 >= 0 && col0 + gate.size(1) <= table.size(1));
  const long n = gate.numel();
  if (n == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(gate.scalar_type(), { hipLaunchKernelGGL((gelu_mul_rows_kernel<T>), dim3((n + 255) / 256), dim3(256), 0, stream, 
      (T*)out.data_ptr(), (const T*)gate.data_ptr(), gate.stride(0),
      (const T*)table.data_ptr(), table.stride(0),
      (const long*)tokens.data_ptr<int64_t>(), (int)col0, gate.size(0),
      (int)gate.size(1)); });
  HIP_CHECK_KERNEL();
}

// res[n, d] += scale * sum_k y[inv[n, k], d]
template <typename T>
__global__ void moe_combine_kernel(float* __restrict__ res,
                                   const T* __restrict__ y,
                                   const int* __restrict__ inv, int top,
                                   float scale, long rows, int D) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * D) return;
  const long n = i / D;
  const int d = i % D;
  float acc = 0.f;
  for (int k = 0; k < top; ++k) acc += ldf(y + (long)inv[n * top + k] * D + d);
  res[i] += scale * acc;
}

void seq_moe_combine(torch::Tensor res, torch::Tensor y, torch::Tensor inv,
                     double scale) {
  CHECK_F32(res);
  CHECK_I32(inv);
  TORCH_CHECK(res.dim() == 2 && inv.dim() == 2 && inv.size(0) == res.size(0));
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.dim() == 2 &&
              y.size(1) == res.size(1) &&
              y.size(0) == inv.size(0) * inv.size(1));
  const long n = res.numel();
  if (n == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(y.scalar_type(), { hipLaunchKernelGGL((moe_combine_kernel<T>), dim3((n + 255) / 256), dim3(256), 0, stream, 
      res.data_ptr<float>(), (const T*)y.data_ptr(), inv.data_ptr<int>(),
      (int)inv.size(1), (float)scale, res.size(0), (int)res.size(1)); });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------- gated joint + shared layer norm
// One block per row.  res (fp32) += y1 * sigmoid(g1) [+ y2 * sigmoid(g2)]
// (a missing gate: plain add; a missing y1: no add), then the layer norm of
// the new row, (x - mean) * rsqrt(var + eps), is written once per weight
// vector: out1 = unit * w1, out2 = unit * w2.  Two sublayers that read the
// same stream share the statistics, so their norms cost one pass.  The
// variance is the mean of the squared deviations.  A row of up to 256*EPT
// numbers stays in registers between the passes (EPT > 0); longer rows
// (EPT = 0) are read again from the values the thread itself wrote.
template <typename T, int EPT>
__global__ __launch_bounds__(256) void gated_add_layernorm_kernel(
    T* __restrict__ out1, T* __restrict__ out2, float* __restrict__ res,
    const T* __restrict__ y1, long ld1, const T* __restrict__ g1, long ldg1,
    const T* __restrict__ y2, long ld2, const T* __restrict__ g2, long ldg2,
    const float* __restrict__ w1, const float* __restrict__ w2, int D,
    float eps) {
  __shared__ float red[8], red2[8];
  const long row = blockIdx.x;
  float* rr = res + row * D;
  auto joined = [&](int i) {
    float f = rr[i];
    if (y1) {
      float a = ldf(y1 + row * ld1 + i);
      if (g1) a *= sigmoidf_acc(ldf(g1 + row * ldg1 + i));
      if (y2) {
        float b = ldf(y2 + row * ld2 + i);
        if (g2) b *= sigmoidf_acc(ldf(g2 + row * ldg2 + i));
        a += b;
      }
      f += a;
      rr[i] = f;
    }
    return f;
  };
  float sum = 0.f;
  if (EPT > 0) {
    float v[EPT > 0 ? EPT : 1];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + e * 256;
      v[e] = i < D ? joined(i) : 0.f;
      sum += v[e];
    }
    if (!out1) return;
    const float mean = block_reduce_sum<4>(sum, red) / D;
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const float d = v[e] - mean;
      if (threadIdx.x + e * 256 < D) sq += d * d;
    }
    const float inv = rsqrtf(block_reduce_sum<4>(sq, red2) / D + eps);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + e * 256;
      if (i < D) {
        const float u = (v[e] - mean) * inv;
        stf(out1 + row * D + i, u * w1[i]);
        if (out2) stf(out2 + row * D + i, u * w2[i]);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < D; i += 256) sum += joined(i);
  if (!out1) return;
  const float mean = block_reduce_sum<4>(sum, red) / D;
  float sq = 0.f;
  for (int i = threadIdx.x; i < D; i += 256) {
    const float d = rr[i] - mean;          // own writes: same thread, same i
    sq += d * d;
  }
  const float inv = rsqrtf(block_reduce_sum<4>(sq, red2) / D + eps);
  for (int i = threadIdx.x; i < D; i += 256) {
    const float u = (rr[i] - mean) * inv;
    stf(out1 + row * D + i, u * w1[i]);
    if (out2) stf(out2 + row * D + i, u * w2[i]);
  }
}

#define GALN_LAUNCH(EPTV)                                                     \
  hipLaunchKernelGGL((gated_add_layernorm_kernel<T, EPTV>), dim3(rows),     \
        dim3(256), 0, stream, h1 ? (T*)out1.data_ptr() : nullptr,             \
        h2 ? (T*)out2.data_ptr() : nullptr, res.data_ptr<float>(), p(y1),     \
        ld(y1), p(g1), ld(g1), p(y2), ld(y2), p(g2), ld(g2),                  \
        h1 ? w1.data_ptr<float>() : nullptr,                                  \
        h2 ? w2.data_ptr<float>() : nullptr, D, (float)eps)

void seq_gated_add_layernorm(torch::Tensor out1, torch::Tensor out2,
                             torch::Tensor res, torch::Tensor y1,
                             torch::Tensor g1, torch::Tensor y2,
                             torch::Tensor g2, torch::Tensor w1,
                             torch::Tensor w2, double eps) {
  CHECK_F32(res);
  TORCH_CHECK(res.dim() == 2);
  const long rows = res.size(0);
  const int D = res.size(1);
  if (rows == 0) return;
  auto has = [](const torch::Tensor& t) { return t.defined() && t.numel() > 0; };
  const bool h1 = has(out1), h2 = has(out2);
  TORCH_CHECK(h1 || !h2, "a second norm needs the first");
  TORCH_CHECK(has(y1) || (!has(g1) && !has(y2) && !has(g2)));
  TORCH_CHECK(has(y2) || !has(g2));
  TORCH_CHECK(h1 || has(y1), "nothing to do");
  auto ty = h1 ? out1.scalar_type() : y1.scalar_type();
  for (const torch::Tensor* t : {&y1, &g1, &y2, &g2}) {
    if (!has(*t)) continue;
    TORCH_CHECK(t->is_cuda() && t->dim() == 2 && t->stride(1) == 1 &&
                t->size(0) == rows && t->size(1) == D &&
                t->scalar_type() == ty, "branch rows / dtype");
  }
  for (const torch::Tensor* t : {&out1, &out2}) {
    if (!has(*t)) continue;
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() &&
                t->numel() == res.numel() && t->scalar_type() == ty);
  }
  if (h1) { CHECK_F32(w1); TORCH_CHECK(w1.numel() == D); }
  if (h2) { CHECK_F32(w2); TORCH_CHECK(w2.numel() == D); }
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(ty, {
    auto p = [&](const torch::Tensor& t) {
      return has(t) ? (const T*)t.data_ptr() : (const T*)nullptr; };
    auto ld = [&](const torch::Tensor& t) { return has(t) ? t.stride(0) : 0L; };
    if (D <= 1024) GALN_LAUNCH(4);
    else if (D <= 2048) GALN_LAUNCH(8);
    else if (D <= 4096) GALN_LAUNCH(16);
    else GALN_LAUNCH(0);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------- per-head sigmoid gate
// out[n, h*Dv + d] = x[n, h*Dv + d] * sigmoid(gate[n, h])
template <typename T>
__global__ void sigmoid_mul_heads_kernel(T* __restrict__ out,
                                         const T* __restrict__ x, long ldx,
                                         const T* __restrict__ gate, long ldg,
                                         int H, int Dv, long total) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int hd = H * Dv;
  const long n = i / hd;
  const int c = i % hd;
  stf(out + i, ldf(x + n * ldx + c) *
                   sigmoidf_acc(ldf(gate + n * ldg + c / Dv)));
}

void seq_sigmoid_mul_heads(torch::Tensor out, torch::Tensor x,
                           torch::Tensor gate) {
  CHECK_ROWS(x);
  CHECK_ROWS(gate);
  const long N = x.size(0);
  const int H = gate.size(1);
  TORCH_CHECK(gate.size(0) == N && H > 0 && x.size(1) % H == 0);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
              out.sizes() == x.sizes() &&
              out.scalar_type() == x.scalar_type() &&
              gate.scalar_type() == x.scalar_type());
  const long total = N * x.size(1);
  if (total == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(x.scalar_type(), {
    hipLaunchKernelGGL((sigmoid_mul_heads_kernel<T>),
        dim3((total + 255) / 256), dim3(256), 0, stream, (T*)out.data_ptr(),
        (const T*)x.data_ptr(), x.stride(0), (const T*)gate.data_ptr(),
        gate.stride(0), H, (int)(x.size(1) / H), total);
  });
  HIP_CHECK_KERNEL();
}

// ----------------------------------- turn every head's row back (fp32 in)
// x (N, H*Dv) fp32: head sums over values that were rotated by their own
// positions.  Pair (m, m + Dv/2) of every head is rotated by
// -fp32(pos) * inv_freq[m]; then the optional per-head sigmoid gate; the
// result is rounded once, to T.
template <typename T>
__global__ void rotate_back_heads_kernel(T* __restrict__ out,
                                         const float* __restrict__ x,
                                         const float* __restrict__ inv_freq,
                                         const int* __restrict__ pos,
                                         const T* __restrict__ gate, long ldg,
                                         int H, int Dv, long total) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int half = Dv / 2;
  const int m = i % half;
  const int h = (i / half) % H;
  const long n = i / ((long)half * H);
  const float ang = (float)pos[n] * inv_freq[m];
  const float c = cosf(ang), s = sinf(ang);
  const long at = (n * H + h) * Dv + m;
  const float a = x[at], b = x[at + half];
  float g = 1.f;
  if (gate) g = sigmoidf_acc(ldf(gate + n * ldg + h));
  stf(out + at, (a * c + b * s) * g);
  stf(out + at + half, (b * c - a * s) * g);
}

void seq_rotate_back_heads(torch::Tensor out, torch::Tensor x,
                           torch::Tensor inv_freq, torch::Tensor positions,
                           torch::Tensor gate, int64_t H) {
  CHECK_F32(x);
  CHECK_F32(inv_freq);
  CHECK_I32(positions);
  TORCH_CHECK(x.dim() == 2 && H > 0 && x.size(1) % H == 0);
  const long N = x.size(0);
  const int Dv = x.size(1) / H;
  TORCH_CHECK(Dv % 2 == 0 && inv_freq.numel() == Dv / 2 &&
              positions.numel() == N);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
              out.sizes() == x.sizes());
  const bool has_gate = gate.defined() && gate.numel() > 0;
  if (has_gate) {
    CHECK_ROWS(gate);
    TORCH_CHECK(gate.size(0) == N && gate.size(1) == H &&
                gate.scalar_type() == out.scalar_type());
  }
  const long total = N * H * (Dv / 2);
  if (total == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(out.scalar_type(), {
    hipLaunchKernelGGL((rotate_back_heads_kernel<T>),
        dim3((total + 255) / 256), dim3(256), 0, stream, (T*)out.data_ptr(),
        x.data_ptr<float>(), inv_freq.data_ptr<float>(),
        positions.data_ptr<int>(),
        has_gate ? (const T*)gate.data_ptr() : nullptr,
        has_gate ? gate.stride(0) : 0, (int)H, Dv, total);
  });
  HIP_CHECK_KERNEL();
}
