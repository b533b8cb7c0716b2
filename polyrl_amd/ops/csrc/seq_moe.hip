// Table-routed expert feed-forward for decode-sized batches (bf16, MFMA).
//
// Routing is a table over token ids, so a block finds its expert's rows by
// scanning the batch's (token, choice) slots itself: no host routing, no
// sort, no gather copy, and the launch shape depends only on the batch size
// (capturable in a graph).  Grid = (64-column tile, expert); a block whose
// expert got no row exits at once.  The op is weight-read bound at these
// batch sizes (every live expert streams its matrices once per step), so a
// wave just streams 16 weight rows with 16-byte loads straight into
// v_mfma_f32_16x16x32_bf16 B fragments while the A fragments (<= 16 token
// rows per pass) come from the activations; fp32 accumulation.
//
//   ACT 1 : act[slot, j] = silu(x_t . Wg[e][j]) * (x_t . Wu[e][j])   (gated)
//   ACT 2 : act[slot, j] = gelu_erf(x_t . Wu[e][j])                  (plain)
//   ACT 0 : y[slot, n]   = act[slot] . Wd[e][n]
// slot = t * top + choice, e = table[token_t][choice], or, for experts
// chosen by a router, e = slot_expert[slot] (an index >= the number of
// expert matrices names an expert without matrices: no block serves it).
//
// The router itself (softmax, selection-only correction, group-limited
// top-k) and the weighted combine of the chosen rows are here too.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;

constexpr int MOE_MAX_SLOTS = 1024;

template <int ACT>
__global__ __launch_bounds__(256) void moe_table_gemm_kernel(
    bf16_t* __restrict__ out,           // (B*top, Nout)
    const bf16_t* __restrict__ x, long ldx,   // gated: (B, K) by token; else (B*top, K) by slot
    const long* __restrict__ tokens,    // (B,)
    const int* __restrict__ table,      // (V, top)
    const int* __restrict__ slot_expert,   // (B*top,) or null (use the table)
    const bf16_t* __restrict__ w,       // (E, Nw, K): Nw = 2*Nout if gated
    int B, int top, int K, int Nout) {
  constexpr bool GATED = ACT == 1;
  constexpr bool BYTOKEN = ACT != 0;    // x rows by token, else by slot
  __shared__ int slots[MOE_MAX_SLOTS];
  __shared__ int count;
  const int e = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int l15 = lane & 15, lhi = lane >> 4;
  if (threadIdx.x == 0) count = 0;
  __syncthreads();
  const int S = B * top;
  for (int s = threadIdx.x; s < S; s += 256) {
    const int es = slot_expert ? slot_expert[s]
                               : table[tokens[s / top] * top + s % top];
    if (es == e) slots[atomicAdd(&count, 1)] = s;
  }
  __syncthreads();
  const int cnt = count;
  if (cnt == 0) return;

  const int n = blockIdx.x * 64 + wid * 16 + l15;   // this lane's B column
  const bool nok = n < Nout;
  const long Nw = GATED ? 2L * Nout : Nout;
  const bf16_t* wrow = w + ((long)e * Nw + (nok ? n : 0)) * K + lhi * 8;
  const bf16_t* wrow2 = wrow + (long)Nout * K;       // up rows (gated)

  for (int c0 = 0; c0 < cnt; c0 += 16) {
    const int si = c0 + l15;
    const int slot = si < cnt ? slots[si] : -1;
    const bf16_t* xrow = x + (long)(slot < 0 ? 0 : (BYTOKEN ? slot / top : slot)) * ldx + lhi * 8;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    const i32x4_t zi = {0, 0, 0, 0};
    const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, zi);
#pragma unroll 4
    for (int k0 = 0; k0 < K; k0 += 32) {
      const bf16x8_t a = slot >= 0 ? *reinterpret_cast<const bf16x8_t*>(xrow + k0) : zero;
      const bf16x8_t b = nok ? *reinterpret_cast<const bf16x8_t*>(wrow + k0) : zero;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
      if (GATED) {
        const bf16x8_t b2 = nok ? *reinterpret_cast<const bf16x8_t*>(wrow2 + k0) : zero;
        acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2, acc2, 0, 0, 0);
      }
    }
    // C layout: row = lhi*4 + r (slot of the pass), col = l15
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ri = c0 + lhi * 4 + r;
      if (ri < cnt && nok) {
        const float v = ACT == 1 ? siluf_acc(acc[r]) * acc2[r]
                      : ACT == 2 ? gelu_erff_acc(acc[r]) : acc[r];
        out[(long)slots[ri] * Nout + n] = f2bf(v);
      }
    }
  }
}

// y (B*top, width) = table-routed experts on h (B, width); fills ``act``
// (B*top, ff) on the way.
void seq_moe_table_ffn(torch::Tensor y, torch::Tensor act, torch::Tensor h,
                       torch::Tensor tokens, torch::Tensor table,
                       torch::Tensor w_gu, torch::Tensor w_down) {
  CHECK_I32(table);
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 &&
              h.scalar_type() == torch::kBFloat16);
  TORCH_CHECK(tokens.is_cuda() && tokens.dtype() == torch::kInt64 &&
              tokens.is_contiguous());
  TORCH_CHECK(w_gu.is_contiguous() && w_down.is_contiguous() &&
              w_gu.dim() == 3 && w_down.dim() == 3 &&
              w_gu.scalar_type() == torch::kBFloat16 &&
              w_down.scalar_type() == torch::kBFloat16);
  const int B = h.size(0), W = h.size(1), top = table.size(1);
  const int E = w_gu.size(0), ff = w_gu.size(1) / 2;
  TORCH_CHECK(tokens.numel() == B && table.dim() == 2);
  TORCH_CHECK(w_gu.size(2) == W && w_down.size(0) == E &&
              w_down.size(1) == W && w_down.size(2) == ff);
  TORCH_CHECK(W % 32 == 0 && ff % 32 == 0 && h.stride(0) % 8 == 0,
              "expert GEMM needs widths in multiples of 32");
  TORCH_CHECK(B * top <= MOE_MAX_SLOTS, "batch too large for the decode path");
  TORCH_CHECK(act.is_contiguous() && act.scalar_type() == torch::kBFloat16 &&
              act.size(0) == (long)B * top && act.size(1) == ff);
  TORCH_CHECK(y.is_contiguous() && y.scalar_type() == torch::kBFloat16 &&
              y.size(0) == (long)B * top && y.size(1) == W);
  if (B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL((moe_table_gemm_kernel<1>), dim3((ff + 63) / 64, E),
                     dim3(256), 0, stream, (bf16_t*)act.data_ptr(),
                     (const bf16_t*)h.data_ptr(), h.stride(0),
                     (const long*)tokens.data_ptr<int64_t>(),
                     table.data_ptr<int>(), (const int*)nullptr,
                     (const bf16_t*)w_gu.data_ptr(), B, top, W, ff);
  hipLaunchKernelGGL((moe_table_gemm_kernel<0>), dim3((W + 63) / 64, E),
                     dim3(256), 0, stream, (bf16_t*)y.data_ptr(),
                     (const bf16_t*)act.data_ptr(), (long)ff,
                     (const long*)tokens.data_ptr<int64_t>(),
                     table.data_ptr<int>(), (const int*)nullptr,
                     (const bf16_t*)w_down.data_ptr(), B, top, ff, W);
  HIP_CHECK_KERNEL();
}

// y (B*top, width) = router-chosen experts on h (B, width), plain
// (gelu(W_up h), w_up (E, ff, W)) or gated (silu(W_gate h) * W_up h, w_up
// (E, 2*ff, W) with the gate rows first); fills ``act`` (B*top, ff) on the
// way.  Rows of identity experts stay unwritten.
void seq_moe_routed_ffn(torch::Tensor y, torch::Tensor act, torch::Tensor h,
                        torch::Tensor idx, torch::Tensor w_up,
                        torch::Tensor w_down, bool gated) {
  CHECK_I32(idx);
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 &&
              h.scalar_type() == torch::kBFloat16);
  TORCH_CHECK(w_up.is_contiguous() && w_down.is_contiguous() &&
              w_up.dim() == 3 && w_down.dim() == 3 &&
              w_up.scalar_type() == torch::kBFloat16 &&
              w_down.scalar_type() == torch::kBFloat16);
  const int B = h.size(0), W = h.size(1);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == B);
  const int top = idx.size(1);
  const int E = w_up.size(0), ff = w_up.size(1) / (gated ? 2 : 1);
  TORCH_CHECK(!gated || w_up.size(1) % 2 == 0);
  TORCH_CHECK(w_up.size(2) == W && w_down.size(0) == E &&
              w_down.size(1) == W && w_down.size(2) == ff);
  TORCH_CHECK(W % 32 == 0 && ff % 32 == 0 && h.stride(0) % 8 == 0,
              "expert GEMM needs widths in multiples of 32");
  TORCH_CHECK(B * top <= MOE_MAX_SLOTS, "batch too large for the decode path");
  TORCH_CHECK(act.is_contiguous() && act.scalar_type() == torch::kBFloat16 &&
              act.size(0) == (long)B * top && act.size(1) == ff);
  TORCH_CHECK(y.is_contiguous() && y.scalar_type() == torch::kBFloat16 &&
              y.size(0) == (long)B * top && y.size(1) == W);
  if (B == 0 || E == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  if (gated)
    hipLaunchKernelGGL((moe_table_gemm_kernel<1>), dim3((ff + 63) / 64, E),
                       dim3(256), 0, stream, (bf16_t*)act.data_ptr(),
                       (const bf16_t*)h.data_ptr(), h.stride(0),
                       (const long*)nullptr, (const int*)nullptr,
                       idx.data_ptr<int>(), (const bf16_t*)w_up.data_ptr(), B,
                       top, W, ff);
  else
    hipLaunchKernelGGL((moe_table_gemm_kernel<2>), dim3((ff + 63) / 64, E),
                       dim3(256), 0, stream, (bf16_t*)act.data_ptr(),
                       (const bf16_t*)h.data_ptr(), h.stride(0),
                       (const long*)nullptr, (const int*)nullptr,
                       idx.data_ptr<int>(), (const bf16_t*)w_up.data_ptr(), B,
                       top, W, ff);
  hipLaunchKernelGGL((moe_table_gemm_kernel<0>), dim3((W + 63) / 64, E),
                     dim3(256), 0, stream, (bf16_t*)y.data_ptr(),
                     (const bf16_t*)act.data_ptr(), (long)ff,
                     (const long*)nullptr, (const int*)nullptr,
                     idx.data_ptr<int>(), (const bf16_t*)w_down.data_ptr(), B,
                     top, ff, W);
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------------------ router
// One wave per token, four tokens a block.  s = softmax(logits) over all E
// router outputs, or (act 1) the logistic function of every logit;
// choice = s + correction; experts form ``groups`` equal groups of
// neighbours, a group's score is the sum of its ``gtop`` largest choices,
// and only the ``keep`` groups with the largest score stay eligible (the
// others count as minus infinity); the ``top`` largest eligible choices
// win, ties to the lower index.  Writes the indices and the UNcorrected s
// at them.
constexpr int ROUTE_MAX_E = 512;

DEV_INLINE void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, WAVE_SIZE);
    const int oi = __shfl_xor(i, off, WAVE_SIZE);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

__global__ __launch_bounds__(256) void moe_route_kernel(
    int* __restrict__ idx, float* __restrict__ wout,
    const float* __restrict__ logits, long ldl,
    const float* __restrict__ correction, long N, int E, int top, int groups,
    int keep, int act, int gtop) {
  __shared__ float s_sh[4][ROUTE_MAX_E], c_sh[4][ROUTE_MAX_E];
  __shared__ float g_sh[4][ROUTE_MAX_E];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long n0 = (long)blockIdx.x * 4 + wid;
  const bool live = n0 < N;           // idle waves shadow the last token
  const long n = live ? n0 : N - 1;
  float* s = s_sh[wid];
  float* c = c_sh[wid];
  float* gb = g_sh[wid];
  const float* z = logits + n * ldl;
  if (act == 1) {
    for (int e = lane; e < E; e += 64) {
      const float p = sigmoidf_acc(z[e]);
      s[e] = p;
      c[e] = p + correction[e];
    }
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_reduce_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(z[e] - mx);
      s[e] = p;
      sum += p;
    }
    sum = wave_reduce_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += 64) {
      const float p = s[e] * inv;
      s[e] = p;
      c[e] = p + correction[e];
    }
  }
  __syncthreads();
  if (groups > 1) {
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
      // sum of the gtop largest choices of the group: pick them one by one,
      // each below the last pick in (value, -index) order
      float b = 0.f, lv = INFINITY;
      int li = -1;
      const int take = gtop < per ? gtop : per;
      for (int r = 0; r < take; ++r) {
        float bv = -INFINITY;
        int bi = -1;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float v = c[e];
          const bool below = v < lv || (v == lv && e > li);
          if (below && (bi < 0 || v > bv)) {
            bv = v;
            bi = e;
          }
        }
        b += bv;
        lv = bv;
        li = bi;
      }
      gb[g] = b;
    }
    __syncthreads();
    // mark the best ``keep`` groups: their best becomes +inf
    for (int r = 0; r < keep; ++r) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += 64) {
        const float v = gb[g];
        if (v != INFINITY && (v > bv || (v == bv && g < bi))) {
          bv = v;
          bi = g;
        }
      }
      wave_argmax(bv, bi);
      if (lane == 0 && bi != 0x7fffffff) gb[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
      if (gb[e / per] != INFINITY) c[e] = -INFINITY;
    __syncthreads();
  }
  for (int r = 0; r < top; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = c[e];
      if (v > bv || (v == bv && e < bi && v != -INFINITY)) {
        bv = v;
        bi = e;
      }
    }
    wave_argmax(bv, bi);
    if (bi == 0x7fffffff) bi = 0;     // fewer eligible experts than top
    if (lane == 0) {
      if (live) {
        idx[n * top + r] = bi;
        wout[n * top + r] = s[bi];
      }
      c[bi] = -INFINITY;
    }
    __syncthreads();
  }
}

void seq_moe_route(torch::Tensor idx, torch::Tensor w, torch::Tensor logits,
                   torch::Tensor correction, int64_t groups, int64_t keep,
                   int64_t act, int64_t group_top) {
  CHECK_I32(idx);
  CHECK_F32(w);
  CHECK_F32(correction);
  TORCH_CHECK(logits.is_cuda() && logits.dim() == 2 &&
              logits.stride(1) == 1 && logits.dtype() == torch::kFloat32);
  const long N = logits.size(0);
  const int E = logits.size(1);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == N && w.sizes() == idx.sizes());
  const int top = idx.size(1);
  TORCH_CHECK(E >= 1 && E <= ROUTE_MAX_E, "router outputs above 512");
  TORCH_CHECK(correction.numel() == E && top >= 1 && top <= E);
  TORCH_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups);
  TORCH_CHECK((act == 0 || act == 1) && group_top >= 1);
  if (N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL(moe_route_kernel, dim3((N + 3) / 4), dim3(256), 0, stream,
                     idx.data_ptr<int>(), w.data_ptr<float>(),
                     logits.data_ptr<float>(), logits.stride(0),
                     correction.data_ptr<float>(), N, E, top, (int)groups,
                     (int)keep, (int)act, (int)group_top);
  HIP_CHECK_KERNEL();
}

// out[n, d] = sum_k w'[n,k] * (idx[n,k] < E ? ys[n*top+k, d] : h[n, d])
//             (+ shared[n, d]),  w' = scale * w / (sum_k w + weight_eps)
template <typename T>
__global__ void moe_weighted_combine_kernel(
    T* __restrict__ out, const T* __restrict__ ys, const int* __restrict__ idx,
    const float* __restrict__ w, const T* __restrict__ h, long ldh,
    const T* __restrict__ shared, long lds_, int top, int E, float weight_eps,
    long rows, int D, float scale) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < rows * D; i += stride) {
    const long n = i / D;
    const int d = i % D;
    float wsum = 0.f;
    for (int k = 0; k < top; ++k) wsum += w[n * top + k];
    const float inv = scale / (wsum + weight_eps);
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const float v = idx[n * top + k] < E ? ldf(ys + (n * top + k) * D + d)
                                           : ldf(h + n * ldh + d);
      acc += w[n * top + k] * inv * v;
    }
    if (shared) acc += ldf(shared + n * lds_ + d);
    stf(out + i, acc);
  }
}

void seq_moe_weighted_combine(torch::Tensor out, torch::Tensor ys,
                              torch::Tensor idx, torch::Tensor w,
                              torch::Tensor h, torch::Tensor shared,
                              int64_t E, double weight_eps, double scale) {
  CHECK_I32(idx);
  CHECK_F32(w);
  CHECK_ROWS(h);
  const long N = h.size(0);
  const int D = h.size(1);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == N && w.sizes() == idx.sizes());
  const int top = idx.size(1);
  auto ty = h.scalar_type();
  TORCH_CHECK(ys.is_cuda() && ys.is_contiguous() && ys.dim() == 2 &&
              ys.size(0) == N * top && ys.size(1) == D &&
              ys.scalar_type() == ty);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.size(0) == N &&
              out.size(1) == D && out.scalar_type() == ty);
  const bool has_shared = shared.defined() && shared.numel() > 0;
  if (has_shared) {
    CHECK_ROWS(shared);
    TORCH_CHECK(shared.size(0) == N && shared.size(1) == D &&
                shared.scalar_type() == ty);
  }
  if (N == 0) return;
  const long nblk = std::min<long>((N * D + 255) / 256, MAX_RESIDENT_BLOCKS * 4);
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(ty, { hipLaunchKernelGGL((moe_weighted_combine_kernel<T>), dim3(nblk), dim3(256), 0, stream,
      (T*)out.data_ptr(), (const T*)ys.data_ptr(), idx.data_ptr<int>(),
      w.data_ptr<float>(), (const T*)h.data_ptr(), h.stride(0),
      has_shared ? (const T*)shared.data_ptr() : nullptr,
      has_shared ? shared.stride(0) : 0, top, (int)E, (float)weight_eps, N,
      D, (float)scale); });
  HIP_CHECK_KERNEL();
}
