// Windowed latent attention with a softmax sink on the matrix cores (bf16).
//
// Same operation as seq_attn.hip (which stays the fp32 / odd-size path):
// every (token, head) row scores against its sequence's cached latent rows
// inside its window and sums the latent part of those rows.  All heads share
// the cached rows, so one LDS tile of 32 keys x (R+rd) serves as K (all
// columns) and as V (the first R columns) for the block's 64 rows.
//
// A block is 4 waves x 16 rows.  mode 0 (portions): the rows are up to 64
// consecutive tokens of one sequence for head blockIdx.y; their windows
// overlap, the block walks the union and masks per element.  mode 1 (decode):
// the rows are up to 64 heads of one token.  QK^T and P.V run on
// v_mfma_f32_16x16x32_bf16 (A = Q rows / P, B = K^T / V from LDS, fp32
// accumulators); the softmax is online per row in fp32 and starts from the
// sink (m = sink_h, l = 1, O = 0).  The next tile's rows are fetched into
// registers while the current tile is multiplied.  K-tile bytes are XOR-swizzled by row
// inside each 64-byte chunk (a row is a whole number of such chunks) so the
// 16 rows of a B-fragment read spread over the banks.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;

constexpr int AKV = 32;   // keys per tile

template <int KS>
DEV_INLINE int tile_off(int row, int byte_col) {
  return row * (KS * 64) + (byte_col ^ ((row & 3) << 4));
}

template <int KS>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(
    bf16_t* __restrict__ out,            // (N, H, R)
    const bf16_t* __restrict__ q,        // (N, H, row) row = R + rd
    const bf16_t* __restrict__ cache,    // (slots, row)
    const int* __restrict__ page_table, int max_pages,
    const int* __restrict__ seq_of_tok, const int* __restrict__ positions,
    const int* __restrict__ tile_n0, const int* __restrict__ tile_cnt,
    const float* __restrict__ sink, int H, int R, int rd, int page_size,
    int window, float scale, int mode) {
  constexpr int DKP = KS * 32;           // padded row length in LDS
  constexpr int NVT = KS * 2;            // 16-wide output tiles (>= R/16)
  __shared__ __attribute__((aligned(16))) bf16_t Ks[AKV * DKP];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4][16 * AKV];

  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int l15 = lane & 15, lhi = lane >> 4;
  const int row = R + rd;
  const int n0 = tile_n0[blockIdx.x];
  const int cnt = tile_cnt[blockIdx.x];
  const int b = seq_of_tok[n0];
  const int* ptab = page_table + (long)b * max_pages;
  const int pos0 = positions[n0];
  const int h0 = mode == 0 ? blockIdx.y : blockIdx.y * 64;

  // row i of the block (0..63) -> (token, head, position, valid)
  auto row_tok = [&](int i) { return mode == 0 ? n0 + (i < cnt ? i : 0) : n0; };
  auto row_head = [&](int i) { return mode == 0 ? h0 : (h0 + i < H ? h0 + i : h0); };
  auto row_ok = [&](int i) { return mode == 0 ? i < cnt : h0 + i < H; };
  auto row_pos = [&](int i) { return mode == 0 ? pos0 + i : pos0; };

  const int pmax = mode == 0 ? pos0 + cnt - 1 : pos0;
  const int kmin = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0;

  // ---- Q fragments (A layout): row l15 of this wave, k = ks*32 + lhi*8 ..
  bf16x8_t qfrag[KS];
  {
    const int i = wid * 16 + l15;
    const bf16_t* qp = q + ((long)row_tok(i) * H + row_head(i)) * row;
    const i32x4_t zi = {0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + lhi * 8;
      qfrag[ks] = d < row ? *reinterpret_cast<const bf16x8_t*>(qp + d)
                          : __builtin_bit_cast(bf16x8_t, zi);
    }
  }
  float m_run[4], l_run[4];
  int rpos[4];
  bool rok[4];
  f32x4_t o_acc[NVT];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = wid * 16 + lhi * 4 + r;
    m_run[r] = sink ? sink[row_head(i)] : -1e30f;   // no sink: nothing yet
    l_run[r] = sink ? 1.f : 0.f;
    rpos[r] = row_pos(i);
    rok[r] = row_ok(i);
  }
#pragma unroll
  for (int nt = 0; nt < NVT; ++nt) o_acc[nt] = {0.f, 0.f, 0.f, 0.f};

  // global -> register prefetch of one tile (this thread's 16-byte vectors;
  // zero past the row end / the last key), issued one tile ahead so its
  // latency hides behind the previous tile's matrix work
  constexpr int NV = (AKV * KS * 4 + 255) / 256;
  i32x4_t pre[NV];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * 256;
      const int kr = v / (KS * 4);
      const int col = (v % (KS * 4)) * 8;
      const int j = t0 + kr;
      const i32x4_t z = {0, 0, 0, 0};
      pre[i] = z;
      if (v < AKV * KS * 4 && j <= pmax && col < row) {
        const long slot = (long)ptab[j / page_size] * page_size + j % page_size;
        pre[i] = *reinterpret_cast<const i32x4_t*>(cache + slot * row + col);
      }
    }
  };
  fetch(kmin);

  for (int t0 = kmin; t0 <= pmax; t0 += AKV) {
    // ---- registers -> swizzled LDS tile, then request the next tile ------
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * 256;
      if (v < AKV * KS * 4) {
        const int kr = v / (KS * 4);
        const int col = (v % (KS * 4)) * 8;
        *reinterpret_cast<i32x4_t*>(reinterpret_cast<char*>(Ks) +
                                    tile_off<KS>(kr, col * 2)) = pre[i];
      }
    }
    __syncthreads();
    if (t0 + AKV <= pmax) fetch(t0 + AKV);

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
            tile_off<KS>(kr, (ks * 32 + lhi * 8) * 2));
        c[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[ks], bf, c[nt],
                                                        0, 0, 0);
      }
    }
    // ---- window mask + online softmax (C layout: row lhi*4+r, col l15) --
    float p[2][4], alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float s[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int j = t0 + nt * 16 + l15;
        const bool live = rok[r] && j <= rpos[r] && j > rpos[r] - window;
        s[nt] = live ? c[nt][r] * scale : -1e30f;
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
#pragma unroll
    for (int nt = 0; nt < NVT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o_acc[nt][r] *= alpha[r];

    // ---- P: C layout -> A layout through a wave-private LDS tile --------
    bf16_t* ps = Ps[wid];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        ps[(lhi * 4 + r) * AKV + nt * 16 + l15] = f2bf(p[nt][r]);
    const bf16x8_t pa =
        *reinterpret_cast<const bf16x8_t*>(ps + l15 * AKV + lhi * 8);

    // ---- O += P V, V = first R columns of the same tile -----------------
#pragma unroll
    for (int nt = 0; nt < NVT; ++nt) {
      if (nt * 16 < R) {
        bf16x8_t bv;
        const int d2 = (nt * 16 + l15) * 2;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          bv[j] = *reinterpret_cast<const __bf16*>(
              reinterpret_cast<const char*>(Ks) +
              tile_off<KS>(lhi * 8 + j, d2));
        o_acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, bv, o_acc[nt],
                                                            0, 0, 0);
      }
    }
    __syncthreads();   // every wave is done with the tile before restaging
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = wid * 16 + lhi * 4 + r;
    if (!rok[r]) continue;
    const float inv = 1.f / l_run[r];
    bf16_t* op = out + ((long)row_tok(i) * H + row_head(i)) * R;
#pragma unroll
    for (int nt = 0; nt < NVT; ++nt) {
      const int d = nt * 16 + l15;
      if (d < R) op[d] = f2bf(o_acc[nt][r] * inv);
    }
  }
}

#define MFMA_ATTN_LAUNCH(KSV)                                                 \
  hipLaunchKernelGGL((latent_attn_mfma_kernel<KSV>), grid, dim3(256), 0,      \
                     stream, (bf16_t*)out.data_ptr(),                         \
                     (const bf16_t*)q.data_ptr(),                             \
                     (const bf16_t*)cache.data_ptr(),                         \
                     page_table.data_ptr<int>(), (int)page_table.size(1),     \
                     seq_of_tok.data_ptr<int>(), positions.data_ptr<int>(),   \
                     tile_n0.data_ptr<int>(), tile_cnt.data_ptr<int>(),       \
                     has_sink ? sink.data_ptr<float>() : nullptr, H,          \
                     (int)rank, rd,                                           \
                     (int)cache.size(1), (int)window, (float)scale, (int)mode)

void seq_latent_attention_mfma(torch::Tensor out, torch::Tensor q,
                               torch::Tensor cache, torch::Tensor page_table,
                               torch::Tensor seq_of_tok,
                               torch::Tensor positions, torch::Tensor tile_n0,
                               torch::Tensor tile_cnt, int64_t rank,
                               int64_t window, torch::Tensor sink,
                               double scale, int64_t mode) {
  CHECK_I32(page_table); CHECK_I32(seq_of_tok); CHECK_I32(positions);
  CHECK_I32(tile_n0); CHECK_I32(tile_cnt);
  const bool has_sink = sink.defined() && sink.numel() > 0;
  if (has_sink) CHECK_F32(sink);
  TORCH_CHECK(q.is_cuda() && q.is_contiguous() && q.dim() == 3 &&
              q.scalar_type() == torch::kBFloat16);
  const int N = q.size(0), H = q.size(1), row = q.size(2);
  const int rd = row - rank;
  TORCH_CHECK(rank > 0 && rd >= 0 && row % 8 == 0,
              "latent row must be a multiple of 8 numbers");
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == row && cache.scalar_type() == torch::kBFloat16);
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == torch::kBFloat16 &&
              out.dim() == 3 && out.size(0) == N && out.size(1) == H &&
              out.size(2) == rank);
  TORCH_CHECK(page_table.dim() == 2 && seq_of_tok.numel() == N &&
              positions.numel() == N && (!has_sink || sink.numel() == H) &&
              window >= 1);
  TORCH_CHECK(tile_n0.numel() == tile_cnt.numel() && (mode == 0 || mode == 1));
  const int ntiles = tile_n0.numel();
  if (N == 0 || ntiles == 0) return;
  const int ks = (row + 31) / 32;
  TORCH_CHECK(ks <= 18, "latent row above 576 numbers: use the vector path");
  const dim3 grid(ntiles, mode == 0 ? H : (H + 63) / 64);
  auto stream = at::hip::getCurrentHIPStream();
  switch (ks) {
    case 1: MFMA_ATTN_LAUNCH(1); break;
    case 2: MFMA_ATTN_LAUNCH(2); break;
    case 3: MFMA_ATTN_LAUNCH(3); break;
    case 4: MFMA_ATTN_LAUNCH(4); break;
    case 5: MFMA_ATTN_LAUNCH(5); break;
    case 6: MFMA_ATTN_LAUNCH(6); break;
    case 7: case 8: MFMA_ATTN_LAUNCH(8); break;
    case 9: MFMA_ATTN_LAUNCH(9); break;
    case 10: MFMA_ATTN_LAUNCH(10); break;
    case 11: case 12: MFMA_ATTN_LAUNCH(12); break;
    case 13: case 14: case 15: case 16: MFMA_ATTN_LAUNCH(16); break;
    default: MFMA_ATTN_LAUNCH(18); break;
  }
  HIP_CHECK_KERNEL();
}
