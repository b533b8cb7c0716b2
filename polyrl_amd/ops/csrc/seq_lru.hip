// Real-gated linear recurrence over packed rows (fp32 state, in place).
//
// Per channel c of block b (C channels in B equal blocks of bw), for the
// rows of one sequence in order:
//   r = sigmoid(gr + br), i = sigmoid(gi + bi)       (gr, gi: the block-
//   log a = -mult * r * softplus(lam[c])              diagonal products,
//   a = exp(log a)                                    computed before)
//   S <- a * S + sqrt(1 - a^2) * i * u
//   out = S * gelu_tanh(y)
// Everything between the loads and the store is fp32; 1 - a^2 is taken as
// -expm1(2 log a), which keeps its digits when the decay is close to one.
//
// A channel's chain is sequential over a sequence's tokens, a step being one
// multiply-add; all the transcendental work of a token is independent of the
// chain.  Short portions (decode steps, small chunks) run as one thread per
// (sequence, channel) walking its rows.  Long portions are cut into segments
// of SEG tokens that run in parallel: pass 1 walks every segment from a zero
// state and keeps its end value and the product of its decays, pass 2 walks
// the segments again, each thread first folding the summaries of the
// segments before its own into the state it starts from (a copy that pass 1
// took: the last segment overwrites the state while others may still start).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

struct LruStep {
  float a, d;
};

template <typename T>
DEV_INLINE LruStep lru_step(const T* __restrict__ u, long ldu,
                            const float* __restrict__ gates, long n, long N,
                            int bw, int blk, int k, int c, float br, float bi,
                            float neg_sp) {
  const float* g = gates + ((long)blk * N + n) * (2 * bw);
  const float r = sigmoidf_acc(g[k] + br);
  const float ig = sigmoidf_acc(g[bw + k] + bi);
  const float log_a = neg_sp * r;
  LruStep s;
  s.a = expf(log_a);
  s.d = sqrtf(-expm1f(2.f * log_a)) * ig * ldf(u + n * ldu + c);
  return s;
}

// MODE 0: whole portion per thread, state read and written, output written.
// MODE 1: segment summaries from a zero state (no output, no state write).
// MODE 2: output of a segment, starting from the state folded with the
//         summaries of the earlier segments; the last segment writes the
//         state.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ u, long ldu,
    const float* __restrict__ gates, const float* __restrict__ gate_bias,
    const float* __restrict__ lam, const T* __restrict__ y, long ldy,
    float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slot, long N, int C, int bw, float mult,
    int seg, float* __restrict__ sum_a, float* __restrict__ sum_s,
    int max_segs) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int b = blockIdx.y;
  if (c >= C) return;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  const int sg = MODE == 0 ? 0 : blockIdx.z;
  const int t0 = MODE == 0 ? q0 : q0 + sg * seg;
  if (t0 >= q1) return;
  const int t1 = MODE == 0 ? q1 : (t0 + seg < q1 ? t0 + seg : q1);
  const int blk = c / bw, k = c % bw;
  const float br = gate_bias[blk * 2 * bw + k];
  const float bi = gate_bias[blk * 2 * bw + bw + k];
  const float neg_sp = -mult * softplusf_acc(lam[c]);
  float* sp = state + (long)state_slot[b] * C + c;
  float S = 0.f;
  if (MODE == 0) S = *sp;
  if (MODE == 2) {
    const long base = ((long)b * (max_segs + 1)) * C + c;
    S = sum_s[base + (long)max_segs * C];
    for (int j = 0; j < sg; ++j)
      S = sum_a[base + (long)j * C] * S + sum_s[base + (long)j * C];
  }
  float A = 1.f;
  for (int n = t0; n < t1; ++n) {
    const LruStep st = lru_step<T>(u, ldu, gates, n, N, bw, blk, k, c, br, bi,
                                   neg_sp);
    S = st.a * S + st.d;
    if (MODE == 1) A *= st.a;
    if (MODE != 1)
      stf(out + (long)n * C + c, S * gelu_tanhf_acc(ldf(y + (long)n * ldy + c)));
  }
  if (MODE == 1) {
    const long at = ((long)b * (max_segs + 1) + sg) * C + c;
    sum_a[at] = A;
    sum_s[at] = S;
    if (sg == 0) sum_s[at + (long)max_segs * C] = *sp;
  }
  if (MODE == 0 || (MODE == 2 && t1 == q1)) *sp = S;
}

void seq_rglru_scan(torch::Tensor out, torch::Tensor u, torch::Tensor gates,
                    torch::Tensor gate_bias, torch::Tensor lam,
                    torch::Tensor y_lin, torch::Tensor state,
                    torch::Tensor cu_q, torch::Tensor state_slot,
                    double decay_mult, int64_t max_rows) {
  CHECK_ROWS(u);
  CHECK_ROWS(y_lin);
  CHECK_F32(gates);
  CHECK_F32(gate_bias);
  CHECK_F32(lam);
  CHECK_F32(state);
  CHECK_I32(cu_q);
  CHECK_I32(state_slot);
  const long N = u.size(0);
  const int C = u.size(1);
  if (max_rows <= 0 || max_rows > N) max_rows = N;
  TORCH_CHECK(gate_bias.dim() == 2 && gate_bias.size(1) % 2 == 0);
  const int B = gate_bias.size(0), bw = gate_bias.size(1) / 2;
  TORCH_CHECK(B * bw == C, "gate blocks must cover the channels");
  TORCH_CHECK(gates.dim() == 3 && gates.size(0) == B && gates.size(1) == N &&
              gates.size(2) == 2 * bw, "gates must be (blocks, rows, 2*bw)");
  TORCH_CHECK(lam.numel() == C && y_lin.size(0) == N && y_lin.size(1) == C);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == C);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.size(0) == N &&
              out.size(1) == C);
  auto ty = u.scalar_type();
  TORCH_CHECK(y_lin.scalar_type() == ty && out.scalar_type() == ty);
  const int nseq = state_slot.numel();
  TORCH_CHECK(cu_q.numel() == nseq + 1);
  if (N == 0 || nseq == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  const dim3 blk(256);
  const int cx = (C + 255) / 256;
  // segments pay once a sequence's rows are many and the plain grid small
  constexpr int SEG = 64;
  const int segs = (int)((max_rows + SEG - 1) / SEG);
  const bool cut = max_rows >= 4 * SEG;
  torch::Tensor sum_a, sum_s;
  if (cut) {
    sum_a = torch::empty({nseq, segs + 1, C}, state.options());
    sum_s = torch::empty({nseq, segs + 1, C}, state.options());
  }
#define LRU_ARGS                                                              \
  (T*)out.data_ptr(), (const T*)u.data_ptr(), u.stride(0),                    \
      gates.data_ptr<float>(), gate_bias.data_ptr<float>(),                   \
      lam.data_ptr<float>(), (const T*)y_lin.data_ptr(), y_lin.stride(0),     \
      state.data_ptr<float>(), cu_q.data_ptr<int>(),                          \
      state_slot.data_ptr<int>(), N, C, bw, (float)decay_mult, SEG,           \
      cut ? sum_a.data_ptr<float>() : nullptr,                                \
      cut ? sum_s.data_ptr<float>() : nullptr, segs
  SEQ_DISPATCH_T(ty, {
    if (!cut) {
      hipLaunchKernelGGL((rglru_scan_kernel<T, 0>), dim3(cx, nseq), blk, 0,
                         stream, LRU_ARGS);
    } else {
      hipLaunchKernelGGL((rglru_scan_kernel<T, 1>), dim3(cx, nseq, segs), blk,
                         0, stream, LRU_ARGS);
      hipLaunchKernelGGL((rglru_scan_kernel<T, 2>), dim3(cx, nseq, segs), blk,
                         0, stream, LRU_ARGS);
    }
  });
#undef LRU_ARGS
  HIP_CHECK_KERNEL();
}
