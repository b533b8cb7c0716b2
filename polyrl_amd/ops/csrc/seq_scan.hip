// Recurrent scans of the hybrid decoders, one launch for prefill portions
// and decode tokens alike (a decode token is a portion of length 1):
//
//   delta rule : S <- diag(w) S - (a*u)(u^T S) + k v^T ,  o = S^T r
//   gated linear attention: S <- diag(w) S + k v^T     ,  o = S^T q
//   state space: S <- exp(-exp(A) dt) S + dt B x^T     ,  y = S^T C + D x
//
// State columns are independent in both recurrences, so the state matrix
// (rows = key/state channel, columns = value channel) is spread over a wave
// as 16 columns x 4 row-groups: a lane keeps RPL = rows/4 state entries of
// one column in VGPRs for the whole portion, the two per-token reductions
// over rows (u^T S and S^T r, or S^T C) are two xor-shuffles inside the
// 4-lane group, and a wave never synchronises with another.  The grid is
// (sequence, head, 64-column block); HBM traffic is the state once in and
// once out per portion plus the token inputs.
//
// Per-token inputs of a lane's rows are contiguous and come in with 16-byte
// loads when the layout allows (scalar loads otherwise); the inputs of token
// t+1 are requested before the arithmetic of token t.  The delta rule's
// decay and removal rate cost three exponentials per row: the 16 column
// lanes of a row group would all compute the same ones, so each computes
// one sixteenth and the group exchanges them by lane shuffles.  Gated
// linear attention stages whole tiles of tokens in LDS instead (below).
// All state math is fp32 for bf16 or fp32 inputs.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

constexpr int RG = 4;            // lanes sharing one column (row groups)
constexpr int COLS_PER_WAVE = 16;

// dst[i] = p[i] for i < RPL (rows row0.. of `rows` in total); 16-byte loads
// when the caller has checked alignment and rows == RG * RPL
template <typename T, int RPL>
DEV_INLINE void load_rows(float (&dst)[RPL], const T* p, int row0, int rows,
                          bool vec) {
  if (vec) {
    if constexpr (sizeof(T) == 2 && RPL % 8 == 0) {
#pragma unroll
      for (int j = 0; j < RPL / 8; ++j) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(p + 8 * j);
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[8 * j + e] = bf2f(v.v[e]);
      }
      return;
    } else if constexpr (sizeof(T) == 4 && RPL % 4 == 0) {
#pragma unroll
      for (int j = 0; j < RPL / 4; ++j) {
        const f32x4v v = *reinterpret_cast<const f32x4v*>(p + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[4 * j + e] = v.v[e];
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) dst[i] = row0 + i < rows ? ldf(p + i) : 0.f;
}

// host check for load_rows' vector form: every lane's first row address
// (view base + token row + column offset + head/group offset + row0) is
// 16-byte aligned and no lane owns padding rows
template <typename T>
static bool rows_vectorizable(const torch::Tensor& t, long col_off, int rows,
                              int rpl) {
  const int per = 16 / (int)sizeof(T);
  return rows == RG * rpl && rpl % per == 0 &&
         ((uintptr_t)t.data_ptr() % 16 == 0) && t.stride(0) % per == 0 &&
         col_off % per == 0 && rows % per == 0;
}

// ------------------------------------------------------------- delta rule
template <int RPL>
struct DeltaIn {
  static constexpr int NC = (RPL + 15) / 16;   // rows whose gates I compute
  float r[RPL], k[RPL];
  float wl[NC], al[NC];
  float v;
};

template <typename T, int RPL>
DEV_INLINE void delta_load(DeltaIn<RPL>& in, const T* r, const T* k,
                           const T* v, const T* wl, const T* al, long ldr,
                           long ldk, long ldv, long ldw, long lda, long n,
                           int hoff_k, int row0, int Dk, int vcol, bool colok,
                           int ci, bool vec) {
  load_rows<T, RPL>(in.r, r + n * ldr + hoff_k + row0, row0, Dk, vec);
  load_rows<T, RPL>(in.k, k + n * ldk + hoff_k + row0, row0, Dk, vec);
#pragma unroll
  for (int c = 0; c < DeltaIn<RPL>::NC; ++c) {
    const int i = ci + 16 * c;
    const bool ok = i < RPL && row0 + i < Dk;
    in.wl[c] = ok ? ldf(wl + n * ldw + hoff_k + row0 + i) : 0.f;
    in.al[c] = ok ? ldf(al + n * lda + hoff_k + row0 + i) : 0.f;
  }
  in.v = colok ? ldf(v + n * ldv + vcol) : 0.f;
}

template <typename T, int RPL>
__global__ __launch_bounds__(256) void delta_rule_kernel(
    float* __restrict__ out,            // (N, H*Dv) fp32, un-normalised o
    const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ wl, const T* __restrict__ al, long ldr, long ldk,
    long ldv, long ldw, long lda, const float* __restrict__ w0,
    const float* __restrict__ a_bias, float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ state_slot, int H,
    int Dk, int Dv, float decay_scale, float key_eps, bool vec) {
  constexpr int NC = DeltaIn<RPL>::NC;
  const int cblocks = (Dv + 63) / 64;
  const int b = blockIdx.x / (H * cblocks);
  const int h = (blockIdx.x / cblocks) % H;
  const int cb = blockIdx.x % cblocks;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int ci = lane / RG;                       // column index in the wave
  const int col = cb * 64 + wid * COLS_PER_WAVE + ci;
  const int rg = lane % RG;
  const int row0 = rg * RPL;
  const bool colok = col < Dv;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  // a whole wave past the last column has nothing to do (wave-uniform)
  if (cb * 64 + wid * COLS_PER_WAVE >= Dv) return;

  float* S = state + (((long)state_slot[b] * H + h) * Dk) * Dv;
  float s[RPL], w0c[NC], abc[NC];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    s[i] = (colok && row < Dk) ? S[(long)row * Dv + col] : 0.f;
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int i = ci + 16 * c;
    const bool ok = i < RPL && row0 + i < Dk;
    w0c[c] = ok ? w0[h * Dk + row0 + i] : 0.f;
    abc[c] = ok ? a_bias[h * Dk + row0 + i] : 0.f;
  }
  const int hoff_k = h * Dk;
  const int vcol = h * Dv + col;

  DeltaIn<RPL> cur, nxt;
  delta_load<T, RPL>(cur, r, k, v, wl, al, ldr, ldk, ldv, ldw, lda, q0,
                     hoff_k, row0, Dk, vcol, colok, ci, vec);
  for (int n = q0; n < q1; ++n) {
    if (n + 1 < q1)
      delta_load<T, RPL>(nxt, r, k, v, wl, al, ldr, ldk, ldv, ldw, lda, n + 1,
                         hoff_k, row0, Dk, vcol, colok, ci, vec);
    // my share of the gates: rows ci, ci+16, .. of this row group
    float decm[NC], remm[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      decm[c] = expf(-decay_scale * sigmoidf_acc(cur.wl[c] + w0c[c]));
      remm[c] = sigmoidf_acc(cur.al[c] + abc[c]);
    }
    // unit key: |k|^2 over the head's Dk rows = sum over the 4 row groups
    float kk = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) kk += cur.k[i] * cur.k[i];
    kk = lanegroup_sum<RG>(kk);
    const float kinv = rsqrtf(kk + key_eps);
    float p = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) p += cur.k[i] * s[i];
    p = lanegroup_sum<RG>(p) * kinv;               // u^T S (old state)
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      const int src = (i % 16) * RG + rg;          // lane that owns row i
      const float dec = __shfl(decm[i / 16], src, WAVE_SIZE);
      const float rem = __shfl(remm[i / 16], src, WAVE_SIZE);
      s[i] = dec * s[i] - rem * (cur.k[i] * kinv) * p + cur.k[i] * cur.v;
      o += s[i] * cur.r[i];
    }
    o = lanegroup_sum<RG>(o);
    if (colok && rg == 0) out[(long)n * H * Dv + vcol] = o;
    cur = nxt;
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    if (colok && row < Dk) S[(long)row * Dv + col] = s[i];
  }
}

#define DELTA_LAUNCH(RPLV)                                                   \
  hipLaunchKernelGGL((delta_rule_kernel<T, RPLV>), dim3(grid), dim3(256), 0, stream,           \
      out.data_ptr<float>(), (const T*)r.data_ptr(), (const T*)k.data_ptr(), \
      (const T*)v.data_ptr(), (const T*)w_lin.data_ptr(),                    \
      (const T*)a_lin.data_ptr(), r.stride(0), k.stride(0), v.stride(0),     \
      w_lin.stride(0), a_lin.stride(0), w0.data_ptr<float>(),                \
      a_bias.data_ptr<float>(), state.data_ptr<float>(),                     \
      cu_q.data_ptr<int>(), state_slot.data_ptr<int>(), H, Dk, Dv,           \
      (float)decay_scale, (float)key_eps,                                    \
      rows_vectorizable<T>(r, 0, Dk, RPLV) &&                                \
          rows_vectorizable<T>(k, 0, Dk, RPLV))

void seq_delta_rule(torch::Tensor out, torch::Tensor r, torch::Tensor k,
                    torch::Tensor v, torch::Tensor w_lin, torch::Tensor a_lin,
                    torch::Tensor w0, torch::Tensor a_bias,
                    torch::Tensor state, torch::Tensor cu_q,
                    torch::Tensor state_slot, double decay_scale,
                    double key_eps) {
  CHECK_ROWS(r); CHECK_ROWS(k); CHECK_ROWS(v); CHECK_ROWS(w_lin);
  CHECK_ROWS(a_lin);
  CHECK_F32(w0); CHECK_F32(a_bias); CHECK_F32(state); CHECK_F32(out);
  CHECK_I32(cu_q); CHECK_I32(state_slot);
  TORCH_CHECK(state.dim() == 4);
  const int H = state.size(1), Dk = state.size(2), Dv = state.size(3);
  const long N = r.size(0);
  TORCH_CHECK(r.size(1) == H * Dk && k.size(1) == H * Dk &&
              w_lin.size(1) == H * Dk && a_lin.size(1) == H * Dk &&
              v.size(1) == H * Dv, "delta rule operand widths");
  TORCH_CHECK(k.size(0) == N && v.size(0) == N && w_lin.size(0) == N &&
              a_lin.size(0) == N && out.size(0) == N &&
              out.size(1) == H * Dv);
  TORCH_CHECK(w0.numel() == H * Dk && a_bias.numel() == H * Dk);
  auto dt = r.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              w_lin.scalar_type() == dt && a_lin.scalar_type() == dt);
  TORCH_CHECK(Dk <= 256, "delta rule: key dim above 256 not supported");
  const int B = state_slot.numel();
  TORCH_CHECK(cu_q.numel() == B + 1);
  if (N == 0 || B == 0) return;
  const int grid = B * H * ((Dv + 63) / 64);
  const int rpl = (Dk + RG - 1) / RG;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(dt, {
    if (rpl <= 4) DELTA_LAUNCH(4);
    else if (rpl <= 8) DELTA_LAUNCH(8);
    else if (rpl <= 16) DELTA_LAUNCH(16);
    else if (rpl <= 32) DELTA_LAUNCH(32);
    else DELTA_LAUNCH(64);
  });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------- gated linear attention
// decay of key channel i: sigmoid(z_i + zb_i)^(1/tau)
//   = exp(inv_tau * log_sigmoid(z_i + zb_i)), fp32
//
// Same lane mapping as above, but the token inputs do not come to the lanes
// one token at a time (a dependent global load per token is what bounds a
// long portion): the block stages TT tokens at once in LDS -- scaled queries,
// keys and the decays, each computed once per (token, channel) instead of
// once per column block -- and the waves then walk the tile out of LDS, where
// the 16 column lanes of a row group read the same words (broadcast).  A
// thread's words of the next tile are requested into registers before the
// current tile is walked.
// sum over the four lanes 4j .. 4j+3 (the row groups of one column) by two
// quad permutes in the VALU data path: partner lane^2, then lane^1
DEV_INLINE float quad_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));  // [2,3,0,1]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));  // [1,0,3,2]
  return x;
}

// tokens per LDS tile: at most 32, and the tile within 48 KB
constexpr int gla_tile_tokens(int dkp) {
  const int fit = 48 * 1024 / (4 * (3 * dkp + 64));
  return fit < 32 ? fit : 32;
}

template <typename T, int RPL>
__global__ __launch_bounds__(256) void gla_scan_kernel(
    float* __restrict__ out,            // (N, H*Dv) fp32, un-normalised o
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ zl, long ldq, long ldk, long ldv, long ldz,
    const float* __restrict__ z_bias, float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ state_slot, int H,
    int Dk, int Dv, float q_scale, float inv_tau) {
  constexpr int DKP = RG * RPL;         // key rows incl. padding
  constexpr int TT = gla_tile_tokens(DKP);
  constexpr int NIT = (TT * DKP + 255) / 256;   // staged words per thread
  constexpr int NVI = (TT * 64 + 255) / 256;
  __shared__ __attribute__((aligned(16))) float q_s[TT * DKP];  // * q_scale
  __shared__ __attribute__((aligned(16))) float k_s[TT * DKP];
  __shared__ __attribute__((aligned(16))) float d_s[TT * DKP];  // decays
  __shared__ float v_s[TT * 64];        // this block's columns
  const int cblocks = (Dv + 63) / 64;
  const int b = blockIdx.x / (H * cblocks);
  const int h = (blockIdx.x / cblocks) % H;
  const int cb = blockIdx.x % cblocks;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int ci = lane / RG;                       // column index in the wave
  const int col = cb * 64 + wid * COLS_PER_WAVE + ci;
  const int rg = lane % RG;
  const int row0 = rg * RPL;
  const bool colok = col < Dv;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;                           // the whole block
  // a wave past the last column only helps to stage the tiles
  const bool wave_live = cb * 64 + wid * COLS_PER_WAVE < Dv;

  float* S = state + (((long)state_slot[b] * H + h) * Dk) * Dv;
  float s[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    s[i] = (colok && row < Dk) ? S[(long)row * Dv + col] : 0.f;
  }
  const int hoff_k = h * Dk;
  const int vcol = h * Dv + col;

  // a tile's words of this thread, requested one tile ahead of their use
  float rq[NIT], rk[NIT], rz[NIT], rv[NVI];
  auto fetch = [&](int n0) {
    const int cnt = q1 - n0 < TT ? q1 - n0 : TT;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      if (it * 256 >= cnt * DKP) break;         // block-uniform
      const int idx = threadIdx.x + it * 256;
      const int t = idx / DKP, r = idx % DKP;
      const bool ok = t < cnt && r < Dk;
      const long n = n0 + t;
      rq[it] = ok ? ldf(q + n * ldq + hoff_k + r) : 0.f;
      rk[it] = ok ? ldf(k + n * ldk + hoff_k + r) : 0.f;
      rz[it] = ok ? ldf(zl + n * ldz + hoff_k + r) + z_bias[hoff_k + r]
                  : INFINITY;
    }
#pragma unroll
    for (int it = 0; it < NVI; ++it) {
      if (it * 256 >= cnt * 64) break;
      const int idx = threadIdx.x + it * 256;
      const int t = idx >> 6, c = cb * 64 + (idx & 63);
      rv[it] = (t < cnt && c < Dv)
                   ? ldf(v + (long)(n0 + t) * ldv + h * Dv + c) : 0.f;
    }
  };
  fetch(q0);
  for (int n0 = q0; n0 < q1; n0 += TT) {
    const int cnt = q1 - n0 < TT ? q1 - n0 : TT;
    __syncthreads();                    // the tile before this one is used up
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int idx = threadIdx.x + it * 256;
      if (idx < cnt * DKP) {
        q_s[idx] = rq[it] * q_scale;
        k_s[idx] = rk[it];
        d_s[idx] = expf(-inv_tau * softplusf_acc(-rz[it]));
      }
    }
#pragma unroll
    for (int it = 0; it < NVI; ++it) {
      const int idx = threadIdx.x + it * 256;
      if (idx < cnt * 64) v_s[idx] = rv[it];
    }
    __syncthreads();
    if (n0 + TT < q1) fetch(n0 + TT);   // in flight while this tile is walked
    if (!wave_live) continue;
    static_assert(RG == 4, "quad_sum adds the four row groups");
    auto step = [&](int t) {
      const float* qr = q_s + t * DKP + row0;
      const float* kr = k_s + t * DKP + row0;
      const float* dr = d_s + t * DKP + row0;
      const float vv = v_s[t * 64 + wid * COLS_PER_WAVE + ci];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        s[i] = dr[i] * s[i] + kr[i] * vv;
        o += s[i] * qr[i];
      }
      o = quad_sum(o);
      if (colok && rg == 0) out[(long)(n0 + t) * H * Dv + vcol] = o;
    };
    int t = 0;
    for (; t + 4 <= cnt; t += 4) {      // four tokens' LDS reads in flight
#pragma unroll
      for (int u = 0; u < 4; ++u) step(t + u);
    }
    for (; t < cnt; ++t) step(t);
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    if (colok && row < Dk) S[(long)row * Dv + col] = s[i];
  }
}

#define GLA_LAUNCH(RPLV)                                                     \
  hipLaunchKernelGGL((gla_scan_kernel<T, RPLV>), dim3(grid), dim3(256), 0,   \
      stream, out.data_ptr<float>(), (const T*)q.data_ptr(),                 \
      (const T*)k.data_ptr(), (const T*)v.data_ptr(),                        \
      (const T*)z_lin.data_ptr(), q.stride(0), k.stride(0), v.stride(0),     \
      z_lin.stride(0), z_bias.data_ptr<float>(), state.data_ptr<float>(),    \
      cu_q.data_ptr<int>(), state_slot.data_ptr<int>(), H, Dk, Dv,           \
      (float)q_scale, (float)inv_tau)

void seq_gla_scan(torch::Tensor out, torch::Tensor q, torch::Tensor k,
                  torch::Tensor v, torch::Tensor z_lin, torch::Tensor z_bias,
                  torch::Tensor state, torch::Tensor cu_q,
                  torch::Tensor state_slot, double q_scale, double inv_tau) {
  CHECK_ROWS(q); CHECK_ROWS(k); CHECK_ROWS(v); CHECK_ROWS(z_lin);
  CHECK_F32(z_bias); CHECK_F32(state); CHECK_F32(out);
  CHECK_I32(cu_q); CHECK_I32(state_slot);
  TORCH_CHECK(state.dim() == 4);
  const int H = state.size(1), Dk = state.size(2), Dv = state.size(3);
  const long N = q.size(0);
  TORCH_CHECK(q.size(1) == H * Dk && k.size(1) == H * Dk &&
              z_lin.size(1) == H * Dk && v.size(1) == H * Dv,
              "gated linear attention operand widths");
  TORCH_CHECK(k.size(0) == N && v.size(0) == N && z_lin.size(0) == N &&
              out.size(0) == N && out.size(1) == H * Dv);
  TORCH_CHECK(z_bias.numel() == H * Dk);
  auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              z_lin.scalar_type() == dt);
  TORCH_CHECK(Dk <= 512, "gated linear attention: key dim above 512 not supported");
  const int B = state_slot.numel();
  TORCH_CHECK(cu_q.numel() == B + 1);
  if (N == 0 || B == 0) return;
  const int grid = B * H * ((Dv + 63) / 64);
  const int rpl = (Dk + RG - 1) / RG;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(dt, {
    if (rpl <= 4) GLA_LAUNCH(4);
    else if (rpl <= 8) GLA_LAUNCH(8);
    else if (rpl <= 16) GLA_LAUNCH(16);
    else if (rpl <= 32) GLA_LAUNCH(32);
    else if (rpl <= 64) GLA_LAUNCH(64);
    else GLA_LAUNCH(128);
  });
  HIP_CHECK_KERNEL();
}

// ------------------------------------------------------------ state space
template <int RPL>
struct SsmIn {
  float Bv[RPL], Cv[RPL];
  float x, dt, z;
};

template <typename T, int RPL>
DEV_INLINE void ssm_load(SsmIn<RPL>& in, const T* xbc, long ldx, const T* dt,
                         long ldd, const T* z, long ldz, long n, int xcol,
                         int boff, int coff, int row0, int Ns, int h,
                         bool colok, bool vec) {
  load_rows<T, RPL>(in.Bv, xbc + n * ldx + boff + row0, row0, Ns, vec);
  load_rows<T, RPL>(in.Cv, xbc + n * ldx + coff + row0, row0, Ns, vec);
  in.x = colok ? ldf(xbc + n * ldx + xcol) : 0.f;
  in.z = colok ? ldf(z + n * ldz + xcol) : 0.f;
  in.dt = ldf(dt + n * ldd + h);
}

template <typename T, int RPL>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    float* __restrict__ out,            // (N, H*P) fp32: y * silu(z)
    const T* __restrict__ xbc, long ldx, const T* __restrict__ dt, long ldd,
    const T* __restrict__ z, long ldz, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip,
    float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slot, int H, int Ns, int P, int G,
    bool vec) {
  const int cblocks = (P + 63) / 64;
  const int b = blockIdx.x / (H * cblocks);
  const int h = (blockIdx.x / cblocks) % H;
  const int cb = blockIdx.x % cblocks;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int col = cb * 64 + wid * COLS_PER_WAVE + lane / RG;
  const int rg = lane % RG;
  const int row0 = rg * RPL;
  const bool colok = col < P;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  if (cb * 64 + wid * COLS_PER_WAVE >= P) return;

  const int inner = H * P;
  const int g = h / (H / G);
  const int boff = inner + g * Ns;
  const int coff = inner + G * Ns + g * Ns;
  const int xcol = h * P + col;
  float* S = state + (((long)state_slot[b] * H + h) * Ns) * P;
  float s[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    s[i] = (colok && row < Ns) ? S[(long)row * P + col] : 0.f;
  }
  const float A = expf(a_log[h]);
  const float Dh = d_skip[h];
  const float dtb = dt_bias[h];

  SsmIn<RPL> cur, nxt;
  ssm_load<T, RPL>(cur, xbc, ldx, dt, ldd, z, ldz, q0, xcol, boff, coff, row0,
                   Ns, h, colok, vec);
  for (int n = q0; n < q1; ++n) {
    if (n + 1 < q1)
      ssm_load<T, RPL>(nxt, xbc, ldx, dt, ldd, z, ldz, n + 1, xcol, boff,
                       coff, row0, Ns, h, colok, vec);
    const float step = softplusf_acc(cur.dt + dtb);
    const float dec = expf(-A * step);
    const float sx = step * cur.x;
    float y = 0.f;
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      s[i] = dec * s[i] + cur.Bv[i] * sx;
      y += s[i] * cur.Cv[i];
    }
    y = lanegroup_sum<RG>(y);
    if (colok && rg == 0)
      out[(long)n * inner + xcol] = (y + Dh * cur.x) * siluf_acc(cur.z);
    cur = nxt;
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int row = row0 + i;
    if (colok && row < Ns) S[(long)row * P + col] = s[i];
  }
}

#define SSM_LAUNCH(RPLV)                                                     \
  hipLaunchKernelGGL((ssm_scan_kernel<T, RPLV>), dim3(grid), dim3(256), 0, stream,             \
      out.data_ptr<float>(), (const T*)xbc.data_ptr(), xbc.stride(0),        \
      (const T*)dt.data_ptr(), dt.stride(0), (const T*)z.data_ptr(),         \
      z.stride(0), dt_bias.data_ptr<float>(), a_log.data_ptr<float>(),       \
      d_skip.data_ptr<float>(), state.data_ptr<float>(),                     \
      cu_q.data_ptr<int>(), state_slot.data_ptr<int>(), H, Ns, P,            \
      (int)groups, rows_vectorizable<T>(xbc, (long)H * P, Ns, RPLV))

void seq_ssm_scan(torch::Tensor out, torch::Tensor xbc, torch::Tensor dt,
                  torch::Tensor z, torch::Tensor dt_bias, torch::Tensor a_log,
                  torch::Tensor d_skip, torch::Tensor state,
                  torch::Tensor cu_q, torch::Tensor state_slot,
                  int64_t groups) {
  CHECK_ROWS(xbc); CHECK_ROWS(dt); CHECK_ROWS(z);
  CHECK_F32(dt_bias); CHECK_F32(a_log); CHECK_F32(d_skip); CHECK_F32(state);
  CHECK_F32(out);
  CHECK_I32(cu_q); CHECK_I32(state_slot);
  TORCH_CHECK(state.dim() == 4);
  const int H = state.size(1), Ns = state.size(2), P = state.size(3);
  const long N = xbc.size(0);
  TORCH_CHECK(groups >= 1 && H % groups == 0);
  TORCH_CHECK(xbc.size(1) == H * P + 2 * groups * Ns && dt.size(1) == H &&
              z.size(1) == H * P && dt.size(0) == N && z.size(0) == N &&
              out.size(0) == N && out.size(1) == H * P,
              "state-space operand widths");
  TORCH_CHECK(dt_bias.numel() == H && a_log.numel() == H &&
              d_skip.numel() == H);
  auto ty = xbc.scalar_type();
  TORCH_CHECK(dt.scalar_type() == ty && z.scalar_type() == ty);
  TORCH_CHECK(Ns <= 256, "state size above 256 not supported");
  const int B = state_slot.numel();
  TORCH_CHECK(cu_q.numel() == B + 1);
  if (N == 0 || B == 0) return;
  const int grid = B * H * ((P + 63) / 64);
  const int rpl = (Ns + RG - 1) / RG;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(ty, {
    if (rpl <= 4) SSM_LAUNCH(4);
    else if (rpl <= 8) SSM_LAUNCH(8);
    else if (rpl <= 16) SSM_LAUNCH(16);
    else if (rpl <= 32) SSM_LAUNCH(32);
    else SSM_LAUNCH(64);
  });
  HIP_CHECK_KERNEL();
}
