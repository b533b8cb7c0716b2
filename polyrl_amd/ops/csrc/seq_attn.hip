// Windowed latent attention with a softmax sink over a paged latent cache.
//
// Every head of a token scores against the SAME cached row per key
// (normed latent c_j of R numbers followed by the rotated shared key part
// of rd numbers): score = (q_lat . c_j + q_rot . kr_j) * scale, and the
// weighted sum is over c_j again (the value up-projection follows outside).
// The query already carries the key up-projection (q_lat = W_uk^T q).
//
// One launch serves prefill portions and decode tokens: a row is a token
// with its own position and sequence; its keys are positions
// max(0, pos-window+1) .. pos of that sequence, found through the page
// table.  Grid = (token, head); one wave per block.  The lanes split the
// row's R+rd numbers (coalesced row reads, NCH = ceil((R+rd)/64) numbers a
// lane); KB keys are scored per iteration so their 6-step wave reductions
// interleave; the softmax is online in fp32 and starts from the sink:
// m = sink_h, l = 1, o = 0, which puts exp(sink_h) into the denominator
// exactly once and gives the sink no value.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

template <typename T, int NCH, int KB>
__global__ __launch_bounds__(64) void latent_attn_kernel(
    T* __restrict__ out,                // (N, H, R)
    const T* __restrict__ q_lat,        // (N, H, R) contiguous
    const T* __restrict__ q_rot, long ldqn, long ldqh,  // (N, H, rd) view
    const T* __restrict__ cache,        // (pages*page_size, R+rd)
    const int* __restrict__ page_table, int max_pages,
    const int* __restrict__ seq_of_tok, const int* __restrict__ positions,
    const float* __restrict__ sink, int H, int R, int rd, int page_size,
    int window, float scale) {
  const long n = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int row = R + rd;
  const int pos = positions[n];
  const int b = seq_of_tok[n];
  const int* ptab = page_table + (long)b * max_pages;
  const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;

  float q[NCH], o[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d = lane + 64 * c;
    float v = 0.f;
    if (d < R) v = ldf(q_lat + (n * H + h) * R + d);
    else if (d < row) v = ldf(q_rot + n * ldqn + h * ldqh + (d - R));
    q[c] = v * scale;
    o[c] = 0.f;
  }
  float m = sink ? sink[h] : -INFINITY, l = sink ? 1.f : 0.f;

  for (int j0 = lo; j0 <= pos; j0 += KB) {
    float kv[KB][NCH], s[KB];
#pragma unroll
    for (int t = 0; t < KB; ++t) {
      const int j = j0 + t;
      const bool ok = j <= pos;
      const int jj = ok ? j : pos;
      const long r0 = ((long)ptab[jj / page_size] * page_size + jj % page_size) * row;
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = lane + 64 * c;
        kv[t][c] = d < row ? ldf(cache + r0 + d) : 0.f;
        acc += q[c] * kv[t][c];
      }
      s[t] = acc;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
      for (int t = 0; t < KB; ++t) s[t] += __shfl_xor(s[t], off, WAVE_SIZE);
    }
    float mn = m;
#pragma unroll
    for (int t = 0; t < KB; ++t)
      if (j0 + t <= pos) mn = fmaxf(mn, s[t]);
    const float corr = expf(m - mn);
    float p[KB];
    float ls = 0.f;
#pragma unroll
    for (int t = 0; t < KB; ++t) {
      p[t] = (j0 + t <= pos) ? expf(s[t] - mn) : 0.f;
      ls += p[t];
    }
    l = l * corr + ls;
    m = mn;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      float acc = o[c] * corr;
#pragma unroll
      for (int t = 0; t < KB; ++t) acc += p[t] * kv[t][c];
      o[c] = acc;
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d = lane + 64 * c;
    if (d < R) stf(out + (n * H + h) * R + d, o[c] * inv);
  }
}

#define ATTN_LAUNCH(NCHV)                                                     \
  hipLaunchKernelGGL((latent_attn_kernel<T, NCHV, 4>), dim3(N, H), dim3(64), 0, stream,         \
      (T*)out.data_ptr(), (const T*)q_lat.data_ptr(),                         \
      (const T*)q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1),           \
      (const T*)cache.data_ptr(), page_table.data_ptr<int>(),                 \
      (int)page_table.size(1), seq_of_tok.data_ptr<int>(),                    \
      positions.data_ptr<int>(),                                              \
      has_sink ? sink.data_ptr<float>() : nullptr, H, R, rd,                  \
      (int)cache.size(1), (int)window, (float)scale)

void seq_latent_attention(torch::Tensor out, torch::Tensor q_lat,
                          torch::Tensor q_rot, torch::Tensor cache,
                          torch::Tensor page_table, torch::Tensor seq_of_tok,
                          torch::Tensor positions, int64_t window,
                          torch::Tensor sink, double scale) {
  CHECK_I32(page_table); CHECK_I32(seq_of_tok); CHECK_I32(positions);
  const bool has_sink = sink.defined() && sink.numel() > 0;
  if (has_sink) CHECK_F32(sink);
  TORCH_CHECK(q_lat.is_cuda() && q_lat.is_contiguous() && q_lat.dim() == 3);
  TORCH_CHECK(q_rot.is_cuda() && q_rot.dim() == 3 && q_rot.stride(2) == 1);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == q_lat.sizes());
  const int N = q_lat.size(0), H = q_lat.size(1), R = q_lat.size(2);
  const int rd = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == N && q_rot.size(1) == H);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == R + rd, "cache row must be rank + rot");
  auto ty = q_lat.scalar_type();
  TORCH_CHECK(q_rot.scalar_type() == ty && cache.scalar_type() == ty &&
              out.scalar_type() == ty);
  TORCH_CHECK(page_table.dim() == 2 && seq_of_tok.numel() == N &&
              positions.numel() == N && (!has_sink || sink.numel() == H) &&
              window >= 1);
  if (N == 0) return;
  const int nch = (R + rd + 63) / 64;
  TORCH_CHECK(nch <= 12, "latent row above 768 numbers not supported");
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(ty, {
    switch (nch) {
      case 1: ATTN_LAUNCH(1); break;
      case 2: ATTN_LAUNCH(2); break;
      case 3: ATTN_LAUNCH(3); break;
      case 4: ATTN_LAUNCH(4); break;
      case 5: case 6: ATTN_LAUNCH(6); break;
      case 7: case 8: ATTN_LAUNCH(8); break;
      case 9: case 10: ATTN_LAUNCH(10); break;
      default: ATTN_LAUNCH(12); break;
    }
  });
  HIP_CHECK_KERNEL();
}
