// Grouped-query window attention on the matrix cores (bf16).
//
// Same operation as gqa_attn_kernel (seq_gqa.hip), which stays the fp32 /
// odd-size / single-token path.  A block is 4 waves x 16 rows: up to 64
// consecutive tokens of one sequence for one query head.  Their
// windows overlap, so the block walks the union of the visible keys in tiles
// of 32 -- first the kept first tokens that lie before the union's window
// ([0, min(keep, kmin))), then [kmin, last position] -- and masks per
// element: key j is live for the row at position p when j <= p and
// (p - j < window or j < keep).  K and V tiles of the head's key/value group
// come from the paged cache rows ([G*D keys | G*Dv values]) into LDS; QK^T
// and P.V run on v_mfma_f32_16x16x32_bf16 with fp32 accumulators; scale, the
// optional distance-bucket bias (this head's column of the table sits in
// LDS), the online softmax and the sigmoid head gate are fp32; so are the
// optional sink (the running maximum starts at the head's sink, the running
// sum at one) and the per-row query temperature folded into the score scale.
// Options: scores capped as cap * tanh(score / cap), a number per head added
// to the capped score, and weights sigmoid(score) per live key without any
// normalisation over keys (no running maximum, no rescaling); head sums as
// fp32 into a separate buffer for the pass that turns rotated values back.
// The next tiles are fetched into registers while the current ones are
// multiplied.
// K-tile bytes are XOR-swizzled by row inside each 64-byte chunk.
//
// Grid: one dimension.  Workgroups go to the 8 XCDs in turn (id mod 8), each
// with an L2 of its own, so the id is taken apart as XCD = id % 8 and, inside
// an XCD's sequence, the H/G query heads that share a key/value head follow
// each other for the same row tile: their K and V tiles are fetched into that
// XCD's L2 once and hit there for the other heads of the group.  With eight
// key/value heads or a multiple of that, every XCD takes whole key/value
// heads and walks their row tiles in order: successive tiles of a sequence
// read the same rows, which then stay in that one L2 (with few query heads
// per group -- one, for keys expanded per head -- a round-robin over the
// dies would make every die fetch every head's rows).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;

constexpr int GKV = 32;          // keys per tile
constexpr int GQA_MAX_REL = 256; // bias-table rows held in LDS
constexpr int GQA_XCDS = 8;      // accelerator dies, each with its own L2

template <int KS>
DEV_INLINE int gtile_off(int row, int byte_col) {
  return row * (KS * 64) + (byte_col ^ ((row & 3) << 4));
}

template <int KS>
__global__ __launch_bounds__(256) void gqa_attn_mfma_kernel(
    bf16_t* __restrict__ out,            // (N, H*Dv)
    const bf16_t* __restrict__ q,        // (N, H*D)
    const bf16_t* __restrict__ cache,    // (slots, G*(D+Dv))
    const int* __restrict__ page_table, int max_pages,
    const int* __restrict__ seq_of_tok, const int* __restrict__ positions,
    const int* __restrict__ tile_n0, const int* __restrict__ tile_cnt,
    int ntiles_rows, const float* __restrict__ rel, int rel_rows,
    const int* __restrict__ dist_bucket,
    const bf16_t* __restrict__ gate, long ldg, int H, int G, int D, int Dv,
    int page_size, int window, int keep, float scale,
    const float* __restrict__ sink, float qt_coef, int qt_every, float cap,
    const float* __restrict__ hbias, bool sigm, float* __restrict__ out32) {
  constexpr int DKP = KS * 32;           // padded head size in LDS
  constexpr int NVT = KS * 2;            // 16-wide output tiles
  __shared__ __attribute__((aligned(16))) bf16_t Ks[GKV * DKP];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[GKV * DKP];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][16 * GKV];
  __shared__ float rel_s[GQA_MAX_REL];

  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int l15 = lane & 15, lhi = lane >> 4;
  const int per = H / G;                 // query heads per key/value head
  const int xcd = blockIdx.x % GQA_XCDS;
  const int seq_in_xcd = blockIdx.x / GQA_XCDS;
  // (tile, kv head) unit of this block
  const int unit = G % GQA_XCDS == 0
      ? xcd * (ntiles_rows * (G / GQA_XCDS)) + seq_in_xcd / per
      : (seq_in_xcd / per) * GQA_XCDS + xcd;
  if (unit >= ntiles_rows * G) return;   // padding of the last round
  // later row tiles see more keys: they start first, the short ones fill
  // the end of the launch
  const int tile = ntiles_rows - 1 - unit % ntiles_rows;
  const int g = unit / ntiles_rows;
  const int h = g * per + seq_in_xcd % per;
  const int row = G * (D + Dv);
  const int koff = g * D, voff = G * D + g * Dv;
  const int n0 = tile_n0[tile];
  const int cnt = tile_cnt[tile];
  const int b = seq_of_tok[n0];
  const int* ptab = page_table + (long)b * max_pages;
  const int pos0 = positions[n0];
  const int pmax = pos0 + cnt - 1;
  const int kmin = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0;
  const int nk = keep < kmin ? keep : kmin;      // kept keys before kmin
  const int nkt = (nk + GKV - 1) / GKV;          // their tiles
  const int nwt = (pmax - kmin) / GKV + 1;       // window tiles

  if (rel)
    for (int i = threadIdx.x; i < rel_rows; i += 256)
      rel_s[i] = rel[(long)i * H + h];

  // ---- Q fragments (A layout): row l15 of this wave, k = ks*32 + lhi*8 ..
  bf16x8_t qfrag[KS];
  {
    const int i = wid * 16 + l15;
    const bf16_t* qp = q + ((long)(n0 + (i < cnt ? i : 0)) * H + h) * D;
    const i32x4_t zi = {0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + lhi * 8;
      qfrag[ks] = d < D ? *reinterpret_cast<const bf16x8_t*>(qp + d)
                        : __builtin_bit_cast(bf16x8_t, zi);
    }
  }
  const float hb = hbias ? hbias[h] : 0.f;
  const float inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  float m_run[4], l_run[4], rscale[4];
  int rpos[4];
  bool rok[4];
  f32x4_t o_acc[NVT];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = wid * 16 + lhi * 4 + r;
    m_run[r] = sink ? sink[h] : -1e30f;
    l_run[r] = sink ? 1.f : 0.f;
    rpos[r] = pos0 + i;
    rok[r] = i < cnt;
    rscale[r] = scale;
    if (qt_coef != 0.f)
      rscale[r] *= 1.f + qt_coef * logf((float)((rpos[r] + 1) / qt_every + 1));
  }
#pragma unroll
  for (int nt = 0; nt < NVT; ++nt) o_acc[nt] = {0.f, 0.f, 0.f, 0.f};

  // tile ti covers keys [t0, t0+32) up to jmax
  auto tile_t0 = [&](int ti) { return ti < nkt ? ti * GKV : kmin + (ti - nkt) * GKV; };
  auto tile_jmax = [&](int ti) { return ti < nkt ? nk - 1 : pmax; };

  constexpr int NV = (GKV * KS * 4 + 255) / 256;
  i32x4_t prek[NV], prev[NV];
  auto fetch = [&](int ti) {
    const int t0 = tile_t0(ti), jmax = tile_jmax(ti);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * 256;
      const int kr = v / (KS * 4);
      const int col = (v % (KS * 4)) * 8;
      const int j = t0 + kr;
      const i32x4_t z = {0, 0, 0, 0};
      prek[i] = z;
      prev[i] = z;
      if (v < GKV * KS * 4 && j <= jmax) {
        const long slot = (long)ptab[j / page_size] * page_size + j % page_size;
        const bf16_t* base = cache + slot * row;
        if (col < D) prek[i] = *reinterpret_cast<const i32x4_t*>(base + koff + col);
        if (col < Dv) prev[i] = *reinterpret_cast<const i32x4_t*>(base + voff + col);
      }
    }
  };
  const int ntiles = nkt + nwt;
  fetch(0);

  for (int ti = 0; ti < ntiles; ++ti) {
    const int t0 = tile_t0(ti), jmax = tile_jmax(ti);
    // ---- registers -> LDS tiles, then request the next tiles ------------
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * 256;
      if (v < GKV * KS * 4) {
        const int kr = v / (KS * 4);
        const int col = (v % (KS * 4)) * 8;
        *reinterpret_cast<i32x4_t*>(reinterpret_cast<char*>(Ks) +
                                    gtile_off<KS>(kr, col * 2)) = prek[i];
        *reinterpret_cast<i32x4_t*>(reinterpret_cast<char*>(Vs) +
                                    gtile_off<KS>(kr, col * 2)) = prev[i];
      }
    }
    __syncthreads();
    if (ti + 1 < ntiles) fetch(ti + 1);

    // ---- S (16 rows x 32 keys) = Q K^T ----------------------------------
    f32x4_t c[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      c[nt] = {0.f, 0.f, 0.f, 0.f};
      const int kr = nt * 16 + l15;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8_t bf = *reinterpret_cast<const bf16x8_t*>(
            reinterpret_cast<const char*>(Ks) +
            gtile_off<KS>(kr, (ks * 32 + lhi * 8) * 2));
        c[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[ks], bf, c[nt],
                                                        0, 0, 0);
      }
    }
    // ---- mask, bias, online softmax (C layout: row lhi*4+r, col l15) ----
    float p[2][4], alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float s[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int j = t0 + nt * 16 + l15;
        const int dist = rpos[r] - j;
        const bool live = rok[r] && j <= jmax && dist >= 0 &&
                          (dist < window || j < keep);
        float sv = c[nt][r] * rscale[r];
        if (rel && live) sv += rel_s[dist_bucket[dist]];
        if (cap > 0.f) sv = cap * tanhf(sv * inv_cap);
        sv += hb;
        s[nt] = live ? sv : -1e30f;
      }
      if (sigm) {
        alpha[r] = 1.f;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
          p[nt][r] = s[nt] > -1e29f ? sigmoidf_acc(s[nt]) : 0.f;
        continue;
      }
      float rm = fmaxf(s[0], s[1]);
#pragma unroll
      for (int off = 1; off < 16; off <<= 1)
        rm = fmaxf(rm, __shfl_xor(rm, off, 64));
      const float mn = fmaxf(m_run[r], rm);
      alpha[r] = __expf(m_run[r] - mn);
      m_run[r] = mn;
      float rs = 0.f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        p[nt][r] = s[nt] > -1e29f ? __expf(s[nt] - mn) : 0.f;
        rs += p[nt][r];
      }
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) rs += __shfl_xor(rs, off, 64);
      l_run[r] = l_run[r] * alpha[r] + rs;
    }
    if (!sigm) {
#pragma unroll
      for (int nt = 0; nt < NVT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[nt][r] *= alpha[r];
    }

    // ---- P: C layout -> A layout through a wave-private LDS tile --------
    bf16_t* ps = Ps[wid];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        ps[(lhi * 4 + r) * GKV + nt * 16 + l15] = f2bf(p[nt][r]);
    const bf16x8_t pa =
        *reinterpret_cast<const bf16x8_t*>(ps + l15 * GKV + lhi * 8);

    // ---- O += P V --------------------------------------------------------
#pragma unroll
    for (int nt = 0; nt < NVT; ++nt) {
      if (nt * 16 < Dv) {
        bf16x8_t bv;
        const int d2 = (nt * 16 + l15) * 2;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          bv[j] = *reinterpret_cast<const __bf16*>(
              reinterpret_cast<const char*>(Vs) +
              gtile_off<KS>(lhi * 8 + j, d2));
        o_acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, bv, o_acc[nt],
                                                            0, 0, 0);
      }
    }
    __syncthreads();   // every wave is done with the tiles before restaging
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = wid * 16 + lhi * 4 + r;
    if (!rok[r]) continue;
    const long tok = n0 + i;
    float inv = sigm ? 1.f : 1.f / l_run[r];
    if (gate && !out32) inv *= sigmoidf_acc(bf2f(gate[tok * ldg + h]));
    bf16_t* op = out + (tok * H + h) * Dv;
    float* op32 = out32 ? out32 + (tok * H + h) * Dv : nullptr;
#pragma unroll
    for (int nt = 0; nt < NVT; ++nt) {
      const int d = nt * 16 + l15;
      if (d < Dv) {
        if (op32) op32[d] = o_acc[nt][r] * inv;
        else op[d] = f2bf(o_acc[nt][r] * inv);
      }
    }
  }
}

void gqa_attention_check(torch::Tensor out, torch::Tensor q,
                         torch::Tensor cache, torch::Tensor page_table,
                         torch::Tensor seq_of_tok, torch::Tensor positions,
                         int64_t H, int64_t G, int64_t D, int64_t Dv,
                         int64_t window, int64_t keep_first,
                         torch::Tensor rel, torch::Tensor dist_bucket,
                         torch::Tensor gate, torch::Tensor sink,
                         int64_t q_temp_every);
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
                              bool sigmoid_weights, torch::Tensor v_inv_freq);
void seq_rotate_back_heads(torch::Tensor out, torch::Tensor x,
                           torch::Tensor inv_freq, torch::Tensor positions,
                           torch::Tensor gate, int64_t H);

#define GQA_MFMA_LAUNCH(KSV)                                                  \
  hipLaunchKernelGGL((gqa_attn_mfma_kernel<KSV>), grid, dim3(256), 0, stream, \
      (bf16_t*)out.data_ptr(), (const bf16_t*)q.data_ptr(),                   \
      (const bf16_t*)cache.data_ptr(), page_table.data_ptr<int>(),            \
      (int)page_table.size(1), seq_of_tok.data_ptr<int>(),                    \
      positions.data_ptr<int>(), tile_n0.data_ptr<int>(),                     \
      tile_cnt.data_ptr<int>(), ntiles,                                       \
      has_rel ? rel.data_ptr<float>() : nullptr,                              \
      has_rel ? (int)rel.size(0) : 0,                                         \
      has_rel ? dist_bucket.data_ptr<int>() : nullptr,                        \
      has_gate ? (const bf16_t*)gate.data_ptr() : nullptr,                    \
      has_gate ? gate.stride(0) : 0, (int)H, (int)G, (int)D, (int)Dv,         \
      (int)cache.size(1), (int)window, (int)keep_first, (float)scale,         \
      has_sink ? sink.data_ptr<float>() : nullptr, (float)q_temp_coef,        \
      (int)q_temp_every, (float)softcap,                                      \
      has_hb ? head_bias.data_ptr<float>() : nullptr, sigmoid_weights, o32)

void seq_gqa_window_attention_mfma(
    torch::Tensor out, torch::Tensor q, torch::Tensor tile_n0,
    torch::Tensor tile_cnt, torch::Tensor cache, torch::Tensor page_table,
    torch::Tensor seq_of_tok, torch::Tensor positions, int64_t H, int64_t G,
    int64_t D, int64_t Dv, int64_t window, int64_t keep_first,
    torch::Tensor rel, torch::Tensor dist_bucket, torch::Tensor gate,
    double scale, torch::Tensor sink, double q_temp_coef,
    int64_t q_temp_every, double softcap, torch::Tensor head_bias,
    bool sigmoid_weights, torch::Tensor v_inv_freq) {
  gqa_attention_check(out, q, cache, page_table, seq_of_tok, positions, H, G,
                      D, Dv, window, keep_first, rel, dist_bucket, gate, sink,
                      q_temp_every);
  const bool has_sink = sink.defined() && sink.numel() > 0;
  CHECK_I32(tile_n0); CHECK_I32(tile_cnt);
  TORCH_CHECK(tile_n0.numel() == tile_cnt.numel());
  const bool has_rel = rel.defined() && rel.numel() > 0;
  const bool has_gate = gate.defined() && gate.numel() > 0;
  const int ks = (int)((std::max(D, Dv) + 31) / 32);
  if (q.scalar_type() != torch::kBFloat16 || D % 8 || Dv % 8 || ks > 4 ||
      (has_rel && rel.size(0) > GQA_MAX_REL)) {
    seq_gqa_window_attention(out, q, cache, page_table, seq_of_tok, positions,
                             H, G, D, Dv, window, keep_first, rel,
                             dist_bucket, gate, scale, sink, q_temp_coef,
                             q_temp_every, softcap, head_bias,
                             sigmoid_weights, v_inv_freq);
    return;
  }
  const int ntiles = tile_n0.numel();
  if (q.size(0) == 0 || ntiles == 0) return;
  const bool has_hb = head_bias.defined() && head_bias.numel() > 0;
  if (has_hb) {
    CHECK_F32(head_bias);
    TORCH_CHECK(head_bias.numel() == H, "one bias per query head");
  }
  TORCH_CHECK(!sigmoid_weights || !has_sink, "a sink needs softmax weights");
  const bool v_rot = v_inv_freq.defined() && v_inv_freq.numel() > 0;
  torch::Tensor sums;
  float* o32 = nullptr;
  if (v_rot) {
    sums = torch::empty({q.size(0), H * Dv}, q.options().dtype(torch::kFloat32));
    o32 = sums.data_ptr<float>();
  }
  // (tile, kv head) units in rounds of one per XCD, H/G heads per unit
  const long units = (long)ntiles * G;
  const long rounds = (units + GQA_XCDS - 1) / GQA_XCDS;
  TORCH_CHECK(rounds * GQA_XCDS * (H / G) < (1L << 31), "grid too large");
  const dim3 grid((unsigned)(rounds * GQA_XCDS * (H / G)));
  auto stream = at::hip::getCurrentHIPStream();
  switch (ks) {
    case 1: GQA_MFMA_LAUNCH(1); break;
    case 2: GQA_MFMA_LAUNCH(2); break;
    case 3: GQA_MFMA_LAUNCH(3); break;
    default: GQA_MFMA_LAUNCH(4); break;
  }
  HIP_CHECK_KERNEL();
  if (v_rot) seq_rotate_back_heads(out, sums, v_inv_freq, positions, gate, H);
}
