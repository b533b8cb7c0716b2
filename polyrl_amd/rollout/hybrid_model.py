"""Engine-side model for hybrid decoders (models/hybrid.py): per-layer weight
buffers and the no-autograd forward over a packed mixed batch (portions of
prompts beside single decode tokens) on the sequence-mixer kernels
(ops/seq.py).

The model owns no cache, no state and no loop over steps: the engine's
PagedLatentCache / StateSlots hold them and the engine's scheduler builds
the batch.  Each mixer and feed-forward kind is a small class with its own
buffers, checkpoint names and state shapes, picked per layer from the
config, so a further design composes them differently.

Precision: the residual stream, all norms, recurrent states and what enters
the recurrences stay fp32; projections run in the engine dtype (bf16 or
fp32) with fp32 accumulation.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

import polyrl_amd.ops as ops
from polyrl_amd.ops import seq
from ..models.hybrid import HybridConfig


@dataclass
class HybridBatch:
    """A packed step: rows [cu_q[b], cu_q[b+1]) are sequence b's next
    tokens at positions start[b]...; device tensors are int32 unless said."""
    tokens: torch.Tensor          # (N,) int64
    tokens_host: np.ndarray       # (N,) int64
    prev_tokens: torch.Tensor     # (N,) int64, -1 at a sequence's first token
    positions: torch.Tensor       # (N,)
    seq_of_tok: torch.Tensor      # (N,)
    cu_q: torch.Tensor            # (B+1,)
    state_slot: torch.Tensor      # (B,)
    slot_mapping: torch.Tensor    # (N,) cache row of each token
    page_table: torch.Tensor      # (B, max_pages)
    attn_tiles: Optional[tuple] = None   # ops.seq.attention_tiles(lens)
    max_q: int = 0                # rows of the longest portion (0 = unknown)
    ctx_lens: Optional[List[int]] = None   # tokens each sequence holds after
    #                                        this step (host; None = unknown)


_TUNED = False


def set_tuned_products(on: bool) -> None:
    """Route the next forward's projections through the per-shape pinned
    hipBLASLt path (worth its one-off search only for the few, recurring
    shapes of pure decode steps)."""
    global _TUNED
    _TUNED = bool(on)


def _mm(x: torch.Tensor, w: torch.Tensor,
        b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x @ w.T [+ b] (vendor matrix product, fp32 accumulation; the
    bias joins the accumulator before the result is rounded)."""
    if b is not None:
        return torch.addmm(b, x, w.t())
    if _TUNED and x.is_cuda and x.dtype == torch.bfloat16 \
            and x.shape[0] <= 512 and x.is_contiguous() \
            and w.shape[0] >= 64 and w.shape[1] >= 64:
        return ops.tuned_mm_nt(x, w)
    return x @ w.t()


class _Part:
    """Buffers of one mixer / feed-forward with their checkpoint names.

    A mixer with ``TAIL`` set can carry ``tail`` further rows (with biases)
    at the end of its fused input projection for a product that reads the
    same input (a layer's residual gate): the rows are ``tail_w`` /
    ``tail_b`` and every forward leaves their result in ``tail_out``."""
    TAIL = False
    tail_w = tail_b = tail_out = None

    def _with_tail(self, rows: int, tail: int, width, device, dtype,
                   bias: bool):
        """(w_in, b_in) of ``rows`` own rows plus ``tail`` shared ones; the
        bias exists when asked for or when there is a tail (zero on rows
        that have none)."""
        w = torch.empty(rows + tail, width, device=device, dtype=dtype)
        b = torch.zeros(rows + tail, device=device, dtype=dtype) \
            if bias or tail else None
        self._rows, self._tail = rows, tail
        if tail:
            self.tail_w, self.tail_b = w[rows:], b[rows:]
        return w, b

    def _split_tail(self, proj):
        if self._tail:
            self.tail_out = proj.narrow(1, self._rows, self._tail)

    def named(self, prefix: str) -> Dict[str, torch.Tensor]:
        raise NotImplementedError

    def state_shapes(self) -> Dict[str, tuple]:
        return {}


class DeltaRuleMixer(_Part):
    def __init__(self, spec, width, device, dtype):
        self.spec = spec
        self.n = n = spec.heads * spec.dim
        self.rank = spec.decay_rank
        z = lambda *s, dt=dtype: torch.empty(*s, device=device, dtype=dt)
        f32 = torch.float32
        # one projection for r, k, v, removal rate, output gate, decay-in
        self.w_in = z(5 * n + self.rank, width)
        self.w2 = z(n, self.rank)
        self.w0, self.a_b, self.norm = z(n, dt=f32), z(n, dt=f32), z(n, dt=f32)
        self.wo = z(width, n)

    def named(self, p):
        n = self.n
        return {p + "r": self.w_in[:n], p + "k": self.w_in[n:2 * n],
                p + "v": self.w_in[2 * n:3 * n], p + "a": self.w_in[3 * n:4 * n],
                p + "g": self.w_in[4 * n:5 * n], p + "w1": self.w_in[5 * n:],
                p + "w2": self.w2, p + "w0": self.w0, p + "a.b": self.a_b,
                p + "norm": self.norm, p + "o": self.wo}

    def state_shapes(self):
        s = self.spec
        return {"S": (s.heads, s.dim, s.dim)}

    def forward(self, h, bt, li, model, cache, states):
        n, s = self.n, self.spec
        proj = _mm(h, self.w_in)
        col = lambda i: proj.narrow(1, i * n, n)
        w_lin = _mm(seq.tanh_act(proj.narrow(1, 5 * n, self.rank)), self.w2)
        y = seq.delta_rule(col(0), col(1), col(2), w_lin, col(3), col(4),
                           self.w0, self.a_b, self.norm,
                           states.tensors[(li, "S")], bt.cu_q, bt.state_slot,
                           s.decay_scale, s.key_eps, model.cfg.norm_eps,
                           h.dtype)
        return _mm(y, self.wo)


class GLAMixer(_Part):
    """Gated linear attention (models.hybrid.GLASpec): one fused projection
    for queries, keys, values, the output gate and the low-rank decay input;
    the scan keeps one fp32 (dim, vdim) state per head and sequence; the
    per-head RMS norm (one weight row shared by the heads) and the SiLU
    output gate are one kernel."""

    def __init__(self, spec, width, device, dtype):
        self.spec = s = spec
        self.nk, self.nv = s.heads * s.dim, s.heads * s.vdim
        self.rank = int(s.decay_rank)
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        f32 = torch.float32
        self.w_in = z(2 * self.nk + 2 * self.nv + self.rank, width)
        self.a2 = z(self.nk, self.rank)
        self.a2_b = z(self.nk, dt=f32)
        self.norm = z(s.vdim, dt=f32)
        self.wo = z(width, self.nv)

    def named(self, p):
        nk, nv = self.nk, self.nv
        return {p + "q": self.w_in[:nk], p + "k": self.w_in[nk:2 * nk],
                p + "v": self.w_in[2 * nk:2 * nk + nv],
                p + "g": self.w_in[2 * nk + nv:2 * nk + 2 * nv],
                p + "a1": self.w_in[2 * nk + 2 * nv:],
                p + "a2": self.a2, p + "a2.b": self.a2_b,
                p + "norm": self.norm, p + "o": self.wo}

    def state_shapes(self):
        s = self.spec
        return {"S": (s.heads, s.dim, s.vdim)}

    def forward(self, h, bt, li, model, cache, states):
        s, nk, nv = self.spec, self.nk, self.nv
        proj = _mm(h, self.w_in)
        z_lin = _mm(proj.narrow(1, 2 * nk + 2 * nv, self.rank), self.a2)
        o = seq.gla_scan(proj.narrow(1, 0, nk), proj.narrow(1, nk, nk),
                         proj.narrow(1, 2 * nk, nv), z_lin, self.a2_b,
                         states.tensors[(li, "S")], bt.cu_q, bt.state_slot,
                         s.dim ** -0.5, 1.0 / s.tau)
        y = seq.group_rmsnorm(o, self.norm, s.heads, model.cfg.norm_eps,
                              h.dtype, gate=proj.narrow(1, 2 * nk + nv, nv),
                              gate_act="silu")
        return _mm(y, self.wo)


class RGLRUMixer(_Part):
    """Real-gated linear recurrence (models.hybrid.RGLRUSpec): one fused
    projection (with biases) for the GELU branch and the convolved branch;
    the stateful convolution; the block-diagonal gate products as one
    batched fp32 product over the blocks (decay-gate rows then input-gate
    rows of a block); one kernel for gates, decay, recurrence and the
    product with the GELU branch.  State per sequence: the recurrence's
    vector (fp32) and the convolution's last taps-1 inputs."""

    TAIL = True

    def __init__(self, spec, width, device, dtype, tail=0):
        self.spec = s = spec
        C, B = s.width, s.blocks
        self.bw = bw = C // B
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        f32 = torch.float32
        self.w_in, self.b_in = self._with_tail(2 * C, tail, width, device,
                                               dtype, True)
        self.conv = z(C, s.conv, dt=f32)
        self.conv_b = z(C, dt=f32)
        self.w_gate = z(B, 2 * bw, bw, dt=f32)
        self.b_gate = z(B, 2 * bw, dt=f32)
        self.lam = z(C, dt=f32)
        self.wo = z(width, C)

    def named(self, p):
        C, bw = self.spec.width, self.bw
        return {p + "y": self.w_in[:C], p + "x": self.w_in[C:2 * C],
                p + "y.b": self.b_in[:C], p + "x.b": self.b_in[C:2 * C],
                p + "conv": self.conv, p + "conv.b": self.conv_b,
                p + "ra": self.w_gate[:, :bw], p + "ri": self.w_gate[:, bw:],
                p + "ra.b": self.b_gate[:, :bw],
                p + "ri.b": self.b_gate[:, bw:],
                p + "lam": self.lam, p + "o": self.wo}

    def state_shapes(self):
        s = self.spec
        out = {"S": (s.width,)}
        if s.conv > 1:
            out["conv"] = (s.conv - 1, s.width)
        return out

    def forward(self, h, bt, li, model, cache, states):
        s = self.spec
        C, B, bw, N = s.width, s.blocks, self.bw, h.shape[0]
        proj = _mm(h, self.w_in, self.b_in)
        self._split_tail(proj)
        u = seq.causal_conv_state(proj.narrow(1, C, C), self.conv,
                                  self.conv_b,
                                  model._state(states, (li, "conv"), C),
                                  bt.cu_q, bt.state_slot, bt.seq_of_tok,
                                  False, False, h.dtype)
        gates = torch.bmm(u.float().view(N, B, bw).transpose(0, 1),
                          self.w_gate.transpose(1, 2))      # (B, N, 2bw)
        y = seq.rglru_scan(u, gates, self.b_gate, self.lam,
                           proj.narrow(1, 0, C), states.tensors[(li, "S")],
                           bt.cu_q, bt.state_slot, s.decay_mult, h.dtype,
                           max_rows=bt.max_q)
        return _mm(y, self.wo)


class SSMMixer(_Part):
    def __init__(self, spec, width, device, dtype):
        self.spec = spec
        z = lambda *s, dt=dtype: torch.empty(*s, device=device, dtype=dt)
        f32 = torch.float32
        inner, ch = spec.inner, spec.conv_channels
        self.w_in = z(inner + ch + spec.heads, width)
        self.conv = z(ch, spec.conv, dt=f32)
        self.conv_b = z(ch, dt=f32)
        self.dt_bias, self.a_log, self.d = (z(spec.heads, dt=f32),
                                            z(spec.heads, dt=f32),
                                            z(spec.heads, dt=f32))
        self.norm = z(inner, dt=f32)
        self.wo = z(width, inner)

    def named(self, p):
        return {p + "in": self.w_in, p + "conv": self.conv,
                p + "conv.b": self.conv_b, p + "dt_bias": self.dt_bias,
                p + "A_log": self.a_log, p + "D": self.d,
                p + "norm": self.norm, p + "o": self.wo}

    def state_shapes(self):
        s = self.spec
        out = {"S": (s.heads, s.state, s.vdim)}
        if s.conv > 1:
            out["conv"] = (s.conv - 1, s.conv_channels)
        return out

    def forward(self, h, bt, li, model, cache, states):
        s = self.spec
        inner, ch = s.inner, s.conv_channels
        proj = _mm(h, self.w_in)
        conv_state = model._state(states, (li, "conv"), ch)
        xbc = seq.causal_conv_state(proj.narrow(1, inner, ch), self.conv,
                                    self.conv_b, conv_state, bt.cu_q,
                                    bt.state_slot, bt.seq_of_tok, False, True,
                                    h.dtype)
        y = seq.ssm_scan(xbc, proj.narrow(1, inner + ch, s.heads),
                         proj.narrow(1, 0, inner), self.dt_bias, self.a_log,
                         self.d, states.tensors[(li, "S")], bt.cu_q,
                         bt.state_slot, s.groups)
        y = seq.group_rmsnorm(y, self.norm, s.norm_groups, model.cfg.norm_eps,
                              h.dtype)
        return _mm(y, self.wo)


class LatentAttnMixer(_Part):
    TAIL = True

    def __init__(self, spec, width, device, dtype, tail=0):
        self.spec = s = spec
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        f32 = torch.float32
        self.nq = s.heads * (s.dim + s.rot_dim)
        self.nv = s.heads * s.vdim
        self.owner = s.kv_from is None
        self.row = s.kv_rank + s.rot_dim
        # rows of the fused input projection: the queries (or their latent),
        # the output gate (per entry or per head) and (if owned) the latent
        self.n0 = s.q_rank if s.q_rank > 0 else self.nq
        self.ng = self.nv if s.gate == "element" else s.heads
        self.w_in, self.b_in = self._with_tail(
            self.n0 + self.ng + (self.row if self.owner else 0), tail, width,
            device, dtype, False)
        self.dq_norm = z(s.q_rank, dt=f32) if s.q_rank > 0 else None
        self.uq = z(self.nq, s.q_rank) if s.q_rank > 0 else None
        self.dkv_norm = z(s.kv_rank, dt=f32) if self.owner else None
        self.uk = z(s.heads * s.dim, s.kv_rank)
        self.uv = z(s.heads * s.vdim, s.kv_rank)
        self.sink = z(s.heads, dt=f32) if s.sink else None
        self.wo = z(width, self.nv)
        self.amp, self.interleaved = 1.0, False
        if s.rope is not None:
            f, self.amp = s.rope.inv_freq_and_amp()
            self.inv_freq = torch.tensor(f, dtype=torch.float64).float() \
                .to(device)
            self.interleaved = s.rope.interleaved
        else:
            self.inv_freq = seq.rope_inv_freq(s.rope_dims, s.rope_base,
                                              device)

    def named(self, p):
        a, b = self.n0, self.n0 + self.ng
        out = {p + "g": self.w_in[a:b],
               p + "uk": self.uk, p + "uv": self.uv, p + "o": self.wo}
        if self.uq is not None:
            out.update({p + "dq": self.w_in[:a], p + "dq.norm": self.dq_norm,
                        p + "uq": self.uq})
        else:
            out[p + "q"] = self.w_in[:a]
        if self.sink is not None:
            out[p + "sink"] = self.sink
        if self.owner:
            out[p + "dkv"] = self.w_in[b:b + self.row]
            out[p + "dkv.norm"] = self.dkv_norm
        return out

    def forward(self, h, bt, li, model, cache, states):
        s = self.spec
        N, H = h.shape[0], s.heads
        proj = _mm(h, self.w_in, self.b_in)
        self._split_tail(proj)
        rows = cache.rows[li if self.owner else s.kv_from]
        if self.owner:
            seq.latent_kv_store(proj.narrow(1, self.n0 + self.ng, self.row),
                                s.kv_rank, self.dkv_norm, model.cfg.norm_eps,
                                bt.positions, self.inv_freq, rows,
                                bt.slot_mapping, self.amp, self.interleaved)
        if self.uq is not None:
            cq = seq.group_rmsnorm(
                proj.narrow(1, 0, self.n0).float().contiguous(),
                self.dq_norm, 1, model.cfg.norm_eps, h.dtype)
            q = _mm(cq, self.uq)
        else:
            q = proj.narrow(1, 0, self.nq)
        q = q.unflatten(1, (H, s.dim + s.rot_dim))
        seq.rope_partial_(q, s.dim, self.inv_freq, bt.positions, self.amp,
                          self.interleaved)
        if self._expand_pays(h, bt, q):
            return _mm(self._attend_expanded(q, proj, rows, bt), self.wo)
        # absorb the key up-projection into the query: (q . W_uk c) =
        # (W_uk^T q) . c, so every head scores against the cached latent
        q_lat = torch.bmm(q[:, :, :s.dim].transpose(0, 1),
                          self.uk.view(H, s.dim, s.kv_rank)).transpose(0, 1)
        o_lat = seq.latent_window_attention(
            q_lat.contiguous(), q[:, :, s.dim:], rows, bt.page_table,
            bt.seq_of_tok, bt.positions, s.window, self.sink, s.scale,
            h.dtype, tiles=bt.attn_tiles)
        # ... and the value up-projection after the weighted sum
        o = torch.bmm(o_lat.transpose(0, 1),
                      self.uv.view(H, s.vdim, s.kv_rank).transpose(1, 2))
        o = o.transpose(0, 1).reshape(N, self.nv)
        gate = proj.narrow(1, self.n0, self.ng)
        o = seq.sigmoid_mul(o, gate) if s.gate == "element" else \
            seq.sigmoid_mul_heads(o, gate)
        return _mm(o, self.wo)

    def _expand_pays(self, h, bt, q) -> bool:
        """Steps that hold a prompt portion attend in the expanded form when
        the matrix-core grouped-query kernel serves the head sizes and the
        sequences' contexts are not much larger than the step itself: scoring
        against per-head keys of dim + rot_dim numbers costs a fraction of
        scoring every head against the whole latent row."""
        s = self.spec
        return (bt.ctx_lens is not None and h.is_cuda
                and bt.attn_tiles is not None and bt.attn_tiles[2] == 0
                and seq.gqa_mfma_supported(q, s.dim + s.rot_dim, s.vdim)
                and sum(bt.ctx_lens) <= max(4 * h.shape[0], 4096))


    def _attend_expanded(self, q, proj, rows, bt):
        """Keys [W_uk c | shared rotated part] and values W_uv c of every cached
        row the step can see, written as temporary K/V rows (one page run per
        sequence), then grouped-query attention with one key/value head per
        query head.  Returns the gated head outputs (N, H*Dv)."""
        s = self.spec
        H, D, Dr, Dv, R = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank
        N, dev = q.shape[0], q.device
        ps = rows.shape[1]
        lens = np.asarray(bt.ctx_lens, dtype=np.int64)
        pages = -(-lens // ps)
        base = np.concatenate([[0], np.cumsum(pages)[:-1]])       # first page
        seq_i = np.repeat(np.arange(len(lens)), lens)
        pos = np.concatenate([np.arange(n) for n in lens]) if len(lens) else \
            np.zeros(0, dtype=np.int64)
        seq_d = torch.from_numpy(seq_i).to(dev)
        pos_d = torch.from_numpy(pos).to(dev)
        src = bt.page_table[seq_d, pos_d // ps].long() * ps + pos_d % ps
        dst = torch.from_numpy(base[seq_i] * ps + pos).to(dev)
        lat = rows.view(-1, rows.shape[-1])[src]                   # (T, R + Dr)
        c = lat[:, :R]
        nk = H * (D + Dr)
        tmp = torch.empty(int(pages.sum()) * ps, nk + H * Dv, device=dev,
                          dtype=q.dtype)
        keys = torch.empty(c.shape[0], H, D + Dr, device=dev, dtype=q.dtype)
        keys[:, :, :D] = _mm(c, self.uk).view(-1, H, D)
        keys[:, :, D:] = lat[:, R:].unsqueeze(1)
        tmp[dst, :nk] = keys.view(-1, nk)
        tmp[dst, nk:] = _mm(c, self.uv)
        ptab = torch.from_numpy(
            (base[:, None] + np.arange(max(int(pages.max()), 1))[None, :])
            .astype(np.int32)).to(dev)
        gate = proj.narrow(1, self.n0, self.ng)
        o = seq.gqa_window_attention(
            q.reshape(N, nk).contiguous(), tmp.view(-1, ps, nk + H * Dv), ptab,
        bt.seq_of_tok,
            bt.positions, H, H, D + Dr, Dv, s.window, 0, None, None,
            gate if s.gate == "head" else None, s.scale, q.dtype,
            tiles=bt.attn_tiles, sink=self.sink)
        return o if s.gate == "head" else seq.sigmoid_mul(o, gate)


class WindowAttnMixer(_Part):
    """Grouped-query attention over a sliding window of paged K/V rows
    (models.hybrid.WindowAttnSpec): one fused projection for queries, keys,
    values (unless the keys serve as values) and the per-head gate; one
    kernel norms, rotates and writes the cache rows; one attends."""
    TAIL = True

    def __init__(self, spec, width, device, dtype, tail=0):
        self.spec = s = spec
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        f32 = torch.float32
        self.nq, self.nk = s.heads * s.dim, s.kv_heads * s.dim
        self.nv = 0 if s.values_from_keys else s.kv_heads * s.vdim
        self.ng = s.heads if s.head_gate else 0
        self.row = s.kv_heads * (s.dim + s.vdim)
        # (the head gate has no bias: its entries stay zero)
        self.w_in, self.b_in = self._with_tail(
            self.nq + self.nk + self.nv + self.ng, tail, width, device, dtype,
            s.qkv_bias)
        self.sink = z(s.heads, dt=f32) if s.sink else None
        self.head_bias = z(s.heads, dt=f32) if s.head_bias else None
        self.v_inv_freq = seq.rope_inv_freq(s.vdim, s.value_rope_base,
                                            device) \
            if s.value_rope_base > 0 else None
        self.q_norm = z(self.nq, dt=f32) if s.qk_norm else None
        self.k_norm = z(self.nk, dt=f32) if s.qk_norm else None
        self.wo = z(width, s.heads * s.vdim)
        self.inv_freq, self.amp = None, 1.0
        if s.rope is not None:
            f, self.amp = s.rope.inv_freq_and_amp()
            self.inv_freq = torch.tensor(f, dtype=torch.float64).float() \
                .to(device)
        self.rel = self.dist_bucket = None
        if s.bias_far > 0:
            self.rel = z(int(s.bias_rows), s.heads, dt=f32)
            self.dist_bucket = torch.tensor(
                s.bucket_of_distance(), dtype=torch.int32).to(device)

    def named(self, p):
        a, b = self.nq, self.nq + self.nk
        s_bias = self.spec.qkv_bias
        out = {p + "q": self.w_in[:a], p + "k": self.w_in[a:b],
               p + "o": self.wo}
        if self.nv:
            out[p + "v"] = self.w_in[b:b + self.nv]
        if self.ng:
            out[p + "g"] = self.w_in[b + self.nv:b + self.nv + self.ng]
        if self.q_norm is not None:
            out[p + "q.norm"] = self.q_norm
            out[p + "k.norm"] = self.k_norm
        if self.rel is not None:
            out[p + "rel"] = self.rel
        if s_bias:
            out[p + "q.b"] = self.b_in[:a]
            out[p + "k.b"] = self.b_in[a:b]
            if self.nv:
                out[p + "v.b"] = self.b_in[b:b + self.nv]
        if self.sink is not None:
            out[p + "sink"] = self.sink
        if self.head_bias is not None:
            out[p + "pb"] = self.head_bias
        return out

    def forward(self, h, bt, li, model, cache, states):
        s = self.spec
        a, b = self.nq, self.nq + self.nk
        proj = _mm(h, self.w_in, self.b_in)
        self._split_tail(proj)
        rows = cache.rows[li]
        q = seq.gqa_prepare_store(
            proj.narrow(1, 0, a), proj.narrow(1, a, self.nk),
            proj.narrow(1, b, self.nv) if self.nv else None,
            self.q_norm, self.k_norm, model.cfg.norm_eps, self.inv_freq,
            self.amp, bt.positions, rows, bt.slot_mapping, s.heads,
            s.kv_heads, s.dim, s.vdim, head_unit=s.head_unit_norm,
            v_inv_freq=self.v_inv_freq)
        o = seq.gqa_window_attention(
            q, rows, bt.page_table, bt.seq_of_tok, bt.positions, s.heads,
            s.kv_heads, s.dim, s.vdim, s.window, s.keep_first, self.rel,
            self.dist_bucket,
            proj.narrow(1, b + self.nv, self.ng) if self.ng else None,
            s.scale, h.dtype, tiles=bt.attn_tiles, sink=self.sink,
            q_temp_coef=s.q_temp_coef, q_temp_every=s.q_temp_every,
            softcap=s.softcap, head_bias=self.head_bias,
            sigmoid_weights=s.weights == "sigmoid",
            v_inv_freq=self.v_inv_freq)
        return _mm(o, self.wo)


class DenseFF(_Part):
    """Gated feed-forward, gate and up as one product: silu(gate) * up, or
    the clamped form (models.hybrid.FFSpec.act); optional biases."""

    def __init__(self, spec, width, vocab, device, dtype):
        self.spec = spec
        self.ff = spec.ff
        self.w_gu = torch.empty(2 * spec.ff, width, device=device, dtype=dtype)
        self.w_down = torch.empty(width, spec.ff, device=device, dtype=dtype)
        self.b_gu = self.b_down = None
        if spec.bias:
            self.b_gu = torch.empty(2 * spec.ff, device=device, dtype=dtype)
            self.b_down = torch.empty(width, device=device, dtype=dtype)

    def named(self, p):
        out = {p + "gate": self.w_gu[:self.ff], p + "up": self.w_gu[self.ff:],
               p + "down": self.w_down}
        if self.b_gu is not None:
            out.update({p + "gate.b": self.b_gu[:self.ff],
                        p + "up.b": self.b_gu[self.ff:],
                        p + "down.b": self.b_down})
        return out

    def forward(self, h, res, bt):
        f = self.spec
        gu = _mm(h, self.w_gu, self.b_gu)
        gate, up = gu.narrow(1, 0, self.ff), gu.narrow(1, self.ff, self.ff)
        if f.act == "clamped":
            act = seq.clamped_glu(gate, up, f.limit, f.gate_slope, f.up_shift)
        else:
            act = seq.silu_mul_any(gate, up)
        # added by the caller's next norm
        return _mm(act, self.w_down, self.b_down)


class TableMoE(_Part):
    """Experts chosen by a table over token ids (no router network): the
    host knows every token's experts before the step runs, so rows are
    sorted by expert there and the device runs one dense product per
    expert that has rows."""

    def __init__(self, spec, width, vocab, device, dtype):
        self.ff, self.E, self.top = spec.ff, spec.experts, spec.top
        self.w_gu = torch.empty(spec.experts, 2 * spec.ff, width,
                                device=device, dtype=dtype)
        self.w_down = torch.empty(spec.experts, width, spec.ff,
                                  device=device, dtype=dtype)
        self.table = torch.zeros(vocab, spec.top, device=device,
                                 dtype=torch.int32)
        self._table_host: Optional[np.ndarray] = None
        self._slots: Dict[int, torch.Tensor] = {}

    def named(self, p):
        out = {p + "table": self.table}
        for e in range(self.E):
            out[f"{p}e{e}.gate"] = self.w_gu[e, :self.ff]
            out[f"{p}e{e}.up"] = self.w_gu[e, self.ff:]
            out[f"{p}e{e}.down"] = self.w_down[e]
        return out

    def route(self, tokens_host: np.ndarray):
        if self._table_host is None:
            self._table_host = self.table.cpu().numpy()
        flat = self._table_host[tokens_host].reshape(-1)
        order = np.argsort(flat, kind="stable")
        counts = np.bincount(flat, minlength=self.E)
        inv = np.empty(order.size, dtype=np.int32)
        inv[order] = np.arange(order.size, dtype=np.int32)
        return (order // self.top).astype(np.int64), counts, \
            inv.reshape(-1, self.top)

    def _slot_index(self, n: int, device) -> torch.Tensor:
        t = self._slots.get(n)
        if t is None:
            t = self._slots[n] = torch.arange(
                n * self.top, dtype=torch.int32, device=device
            ).view(n, self.top)
        return t

    def forward(self, h, res, bt):
        if h.shape[0] <= 256 and \
                seq.moe_table_ffn_supported(h, self.top, self.ff):
            # decode-sized bf16 batch: routing, both products and the
            # activation run in two launches, weight-read bound
            y = seq.moe_table_ffn(h, bt.tokens, self.table, self.w_gu,
                                  self.w_down)
            seq.moe_combine_(res, y, self._slot_index(h.shape[0], h.device),
                             1.0 / self.top)
            return None
        src, counts, inv = self.route(bt.tokens_host)
        dev = h.device
        xs = h.index_select(0, torch.from_numpy(src).to(dev))
        ys = torch.empty(xs.shape[0], h.shape[1], device=dev, dtype=h.dtype)
        o = 0
        for e in np.nonzero(counts)[0].tolist():
            c = int(counts[e])
            gu = _mm(xs[o:o + c], self.w_gu[e])
            act = seq.silu_mul_any(gu.narrow(1, 0, self.ff),
                                   gu.narrow(1, self.ff, self.ff))
            ys[o:o + c] = _mm(act, self.w_down[e])
            o += c
        seq.moe_combine_(res, ys, torch.from_numpy(inv).to(dev),
                         1.0 / self.top)
        return None                       # already in the residual


class RoutedMoE(_Part):
    """Experts chosen by an fp32 router (softmax or per-logit sigmoid
    scores) with a selection-only correction and group-limited choice;
    experts W_down gelu(W_up h) or, gated, W_down (silu(W_gate h) * W_up h)
    with the gate rows stored ahead of the up rows; trailing identity
    experts return the input; a shared expert runs for every token.
    Returns the sublayer output (N, width)."""

    def __init__(self, spec, width, vocab, device, dtype):
        self.spec = f = spec
        self.E, self.top, self.ff = f.experts, f.top, f.ff
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        f32 = torch.float32
        self.gated = f.expert_act == "silu_gated"
        self.w_up = z(f.experts, (2 if self.gated else 1) * f.ff, width)
        self.w_down = z(f.experts, width, f.ff)
        self.router = z(f.experts + f.identity, width, dt=f32)
        self.correction = z(f.experts + f.identity, dt=f32)
        self.s_up = z(f.shared_ff, width) if f.shared_ff else None
        self.s_down = z(width, f.shared_ff) if f.shared_ff else None

    def named(self, p):
        out = {p + "router": self.router, p + "correction": self.correction}
        for e in range(self.E):
            if self.gated:
                out[f"{p}e{e}.gate"] = self.w_up[e, :self.ff]
                out[f"{p}e{e}.up"] = self.w_up[e, self.ff:]
            else:
                out[f"{p}e{e}.up"] = self.w_up[e]
            out[f"{p}e{e}.down"] = self.w_down[e]
        if self.s_up is not None:
            out[p + "shared.up"] = self.s_up
            out[p + "shared.down"] = self.s_down
        return out

    def experts_large(self, h, idx):
        """Rows sorted by expert on the device, one vendor product pair per
        live expert (prompt-sized or fp32 batches); one host sync for the
        row counts.  Each expert's products run over its rows rounded up to
        a multiple of 64 (256 from 512 rows on), reading on into the next
        expert's rows of the sorted copy: the vendor library then sees a
        handful of shapes instead of a new one per call (a new shape costs
        more on the host than the product takes on the GPU).  The surplus
        rows' results are dropped."""
        N, top = idx.shape
        S, W = N * top, h.shape[1]
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)     # identity slots last
        counts = torch.bincount(flat, minlength=self.E + 1)[:self.E].tolist()
        xs = h.new_zeros(S + 256, W)
        torch.index_select(h, 0, order // top, out=xs[:S])
        ys_sorted = torch.empty(S, W, device=h.device, dtype=h.dtype)
        o = 0
        for e, c in enumerate(counts):
            if c:
                step = 64 if c < 512 else 256
                cp = -(-c // step) * step
                act = self._act(_mm(xs[o:o + cp], self.w_up[e]))
                ys_sorted[o:o + c] = _mm(act, self.w_down[e])[:c]
                o += c
        ys = torch.empty_like(ys_sorted)
        ys[order] = ys_sorted           # identity rows stay unread
        return ys

    def _act(self, a):
        if self.gated:
            return seq.silu_mul_any(a.narrow(1, 0, self.ff),
                                    a.narrow(1, self.ff, self.ff))
        return seq.gelu_erf(a)

    def forward(self, h, res, bt):
        f = self.spec
        logits = _mm(h.float(), self.router)
        idx, w = seq.moe_route(logits, self.correction, f.top, f.group_count,
                               f.group_keep, f.router_act, f.group_top)
        if h.shape[0] <= 256 and self.E and \
                seq.moe_routed_ffn_supported(h, self.top, self.ff):
            ys = seq.moe_routed_ffn(h, idx, self.w_up, self.w_down,
                                    self.gated)
        elif self.E:
            ys = self.experts_large(h, idx.long())
        else:
            ys = h.new_empty(h.shape[0] * f.top, h.shape[1])
        shared = None
        if self.s_up is not None:
            shared = _mm(seq.gelu_erf(_mm(h, self.s_up)), self.s_down)
        return seq.moe_weighted_combine(ys, idx, w, h, shared, self.E,
                                        f.weight_eps, h.dtype, f.route_scale)


_MIXERS = {"general_delta": DeltaRuleMixer, "mamba2": SSMMixer,
           "gla": GLAMixer, "rglru": RGLRUMixer,
           "latent_attention": LatentAttnMixer, "attention": WindowAttnMixer}
_FFS = {"dense": DenseFF, "moe": TableMoE, "routed_moe": RoutedMoE}


class HybridLayer:
    def __init__(self, cfg: HybridConfig, li: int, device, dtype):
        L = cfg.layers[li]
        W = cfg.hidden_size
        f32 = torch.float32
        self.norm1 = torch.empty(1, device=device, dtype=f32)
        self.norm2 = torch.empty(1, device=device, dtype=f32)
        self.canon = torch.empty(W, cfg.canon_taps, device=device, dtype=f32)
        self.mixer = _MIXERS[L.mixer.kind](L.mixer, W, device, dtype)
        self.ff = None if L.ff is None else \
            _FFS[L.ff.kind](L.ff, W, cfg.vocab_size, device, dtype)
        d = cfg.token_side_dim
        self.side_gate = torch.empty(d, W, device=device, dtype=dtype)
        self.side_proj = torch.empty(W, d, device=device, dtype=dtype)
        self.side_norm = torch.empty(W, device=device, dtype=f32)

    def named(self, p: str) -> Dict[str, torch.Tensor]:
        out = {p + "norm1": self.norm1, p + "canon1": self.canon}
        if self.side_gate.shape[0] > 0:
            out.update({p + "side.gate": self.side_gate,
                        p + "side.proj": self.side_proj,
                        p + "side.norm": self.side_norm})
        out.update(self.mixer.named(p + "mix."))
        if self.ff is not None:
            out[p + "norm2"] = self.norm2
            out.update(self.ff.named(p + "mlp."))
        return out


class SandwichLayer:
    """x += norm(mixer(norm(x))), x += norm(ff(norm(x))): four per-channel
    norm weights stored as offsets from ``cfg.norm_offset``."""

    def __init__(self, cfg: HybridConfig, li: int, device, dtype):
        L = cfg.layers[li]
        W = cfg.hidden_size
        z = lambda: torch.empty(W, device=device, dtype=torch.float32)
        self.norm1, self.norm1b = z(), z()
        self.mixer = _MIXERS[L.mixer.kind](L.mixer, W, device, dtype)
        self.ff = None if L.ff is None else \
            _FFS[L.ff.kind](L.ff, W, cfg.vocab_size, device, dtype)
        self.norm2, self.norm2b = (z(), z()) if self.ff is not None \
            else (None, None)

    def named(self, p: str) -> Dict[str, torch.Tensor]:
        out = {p + "norm1": self.norm1, p + "norm1b": self.norm1b}
        out.update(self.mixer.named(p + "mix."))
        if self.ff is not None:
            out[p + "norm2"] = self.norm2
            out[p + "norm2b"] = self.norm2b
            out.update(self.ff.named(p + "mlp."))
        return out


class PreNormLayer:
    """x += m * mixer(norm1(x)), x += m * ff(norm2(x)), then the token-side
    input (also times m); per-channel norm weights."""

    def __init__(self, cfg: HybridConfig, li: int, device, dtype):
        L = cfg.layers[li]
        W = cfg.hidden_size
        f32 = torch.float32
        self.norm1 = torch.empty(W, device=device, dtype=f32)
        self.mixer = _MIXERS[L.mixer.kind](L.mixer, W, device, dtype)
        self.ff = None if L.ff is None else \
            _FFS[L.ff.kind](L.ff, W, cfg.vocab_size, device, dtype)
        self.norm2 = torch.empty(W, device=device, dtype=f32) \
            if self.ff is not None else None
        d = cfg.token_side_dim
        self.side_gate = torch.empty(d, W, device=device, dtype=dtype)
        self.side_proj = torch.empty(W, d, device=device, dtype=dtype)
        self.side_norm = torch.empty(W, device=device, dtype=f32)

    def named(self, p: str) -> Dict[str, torch.Tensor]:
        out = {p + "norm1": self.norm1}
        if self.side_gate.shape[0] > 0:
            out.update({p + "side.gate": self.side_gate,
                        p + "side.proj": self.side_proj,
                        p + "side.norm": self.side_norm})
        out.update(self.mixer.named(p + "mix."))
        if self.ff is not None:
            out[p + "norm2"] = self.norm2
            out.update(self.ff.named(p + "mlp."))
        return out


class ParallelLayer:
    """x += mixer(norm1(x)) + ff(norm2(x)), both norms of the same x
    (per-channel weights); optionally each sublayer's result passes a
    sigmoid gate W h + b computed from the sublayer's own input."""

    def __init__(self, cfg: HybridConfig, li: int, device, dtype):
        L = cfg.layers[li]
        W = cfg.hidden_size
        f32 = torch.float32
        z = lambda *a, dt=dtype: torch.empty(*a, device=device, dtype=dt)
        self.norm1 = z(W, dt=f32)
        cls = _MIXERS[L.mixer.kind]
        # the mixer's gate reads the mixer's input: its rows ride at the end
        # of the mixer's fused input projection where the mixer allows it
        self.fused_gate = cfg.gated_residual and cls.TAIL
        self.mixer = cls(L.mixer, W, device, dtype, tail=W) \
            if self.fused_gate else cls(L.mixer, W, device, dtype)
        self.ff = None if L.ff is None else \
            _FFS[L.ff.kind](L.ff, W, cfg.vocab_size, device, dtype)
        self.norm2 = z(W, dt=f32) if self.ff is not None else None
        self.rg1 = self.rg1_b = self.rg2 = self.rg2_b = None
        if cfg.gated_residual:
            self.rg1, self.rg1_b = (self.mixer.tail_w, self.mixer.tail_b) \
                if self.fused_gate else (z(W, W), z(W))
            if self.ff is not None:
                self.rg2, self.rg2_b = z(W, W), z(W)

    def named(self, p: str) -> Dict[str, torch.Tensor]:
        out = {p + "norm1": self.norm1}
        out.update(self.mixer.named(p + "mix."))
        if self.rg1 is not None:
            out.update({p + "rg1": self.rg1, p + "rg1.b": self.rg1_b})
        if self.ff is not None:
            out[p + "norm2"] = self.norm2
            out.update(self.ff.named(p + "mlp."))
            if self.rg2 is not None:
                out.update({p + "rg2": self.rg2, p + "rg2.b": self.rg2_b})
        return out


class HybridInferenceModel:
    """Weights + packed forward of a hybrid decoder for the rollout engine
    (same weight-update surface as InferenceModel: ``_name_map``,
    ``load_state_dict``, ``update_named``)."""

    def __init__(self, cfg: HybridConfig, device="cuda",
                 dtype=torch.bfloat16, tp_ctx=None):
        from ..parallel.tp import TPContext
        self.tp = tp_ctx if tp_ctx is not None else TPContext(None)
        assert self.tp.size == 1, \
            "hybrid decoders run one replica per GPU (tp=1)"
        self.cfg = cfg
        self.device = device
        self.dtype = dtype
        for L in cfg.layers:                 # sizes the config leaves open
            if L.mixer.kind == "general_delta" and L.mixer.decay_rank is None:
                L.mixer.decay_rank = max(8, cfg.hidden_size // 12 // 8 * 8)
            if L.mixer.kind == "attention" and L.mixer.bias_far > 0 \
                    and L.mixer.bias_rows is None:
                raise ValueError("the distance-bias table's rows come from "
                                 "the checkpoint: call resolve_shapes first")
            if L.mixer.kind == "gla" and L.mixer.decay_rank is None:
                raise ValueError("the decay projection's rank comes from "
                                 "the checkpoint: call resolve_shapes first")
        self.sandwich = cfg.layer_style == "sandwich"
        self.prenorm = cfg.layer_style == "prenorm"
        self.parallel = cfg.layer_style == "parallel"
        layer_cls = SandwichLayer if self.sandwich else \
            PreNormLayer if self.prenorm else \
            ParallelLayer if self.parallel else HybridLayer
        self.layers = [layer_cls(cfg, li, device, dtype)
                       for li in range(cfg.num_hidden_layers)]
        self.runs = cfg.run_order()
        W = cfg.hidden_size
        self.embed = torch.empty(cfg.vocab_size, W, device=device, dtype=dtype)
        self.side_embed = torch.empty(
            cfg.vocab_size, cfg.num_hidden_layers * cfg.token_side_dim,
            device=device, dtype=dtype)
        self.final_norm = torch.empty(
            W if self.sandwich or self.prenorm or self.parallel else 1,
            device=device, dtype=torch.float32)
        self.lm_head = torch.empty(cfg.vocab_size, W, device=device,
                                   dtype=dtype)
        self._name_map: Dict[str, torch.Tensor] = {
            "embed": self.embed, "final.norm": self.final_norm,
            "head": self.lm_head}
        if cfg.token_side_dim > 0:
            self._name_map["side.embed"] = self.side_embed
        self.pair_embed = self.loop_step = self.pos_inv_freq = None
        if cfg.bigram is not None:
            self.pair_embed = torch.empty(cfg.bigram.buckets + 1, W,
                                          device=device, dtype=dtype)
            self._name_map["bigram"] = self.pair_embed
        if cfg.loop_step:
            self.loop_step = torch.empty(cfg.loop[2], W, device=device,
                                         dtype=torch.float32)
            self._name_map["loop.step"] = self.loop_step
        if cfg.sin_pos_base > 0:
            self.pos_inv_freq = seq.sinusoid_inv_freq(W, cfg.sin_pos_base,
                                                      device)
        for li, lw in enumerate(self.layers):
            self._name_map.update(lw.named(f"l{li}."))
        self.capture_layers: Optional[List[torch.Tensor]] = None

    # ---------------------------------------------------------- geometry
    @classmethod
    def resolve_shapes(cls, cfg: HybridConfig, shapes: Dict[str, tuple]):
        """Fill sizes that only a tensor's shape gives (the rank of the
        decay projection) from a checkpoint's name -> shape map."""
        for li, L in enumerate(cfg.layers):
            if L.mixer.kind == "general_delta":
                shp = shapes.get(f"l{li}.mix.w1")
                if shp is not None:
                    L.mixer.decay_rank = int(shp[0])
            if L.mixer.kind == "gla":
                shp = shapes.get(f"l{li}.mix.a1")
                if shp is not None:
                    L.mixer.decay_rank = int(shp[0])
            if L.mixer.kind == "attention" and L.mixer.bias_far > 0:
                shp = shapes.get(f"l{li}.mix.rel")
                if shp is not None:
                    L.mixer.bias_rows = int(shp[0])
        return cfg

    def graph_safe_decode(self, B: int) -> bool:
        """Whether a decode step of B single tokens runs without a decision
        on the host (so it can be captured in a graph): pre-norm stacks
        always; parallel stacks when every routed feed-forward takes the
        fused expert kernels (bf16, sizes in multiples of 32, a batch the
        kernels' slot list holds)."""
        if self.prenorm:
            return True
        if not self.parallel:
            return False
        for L in self.layers:
            f = L.ff
            if f is None:
                continue
            if not isinstance(f, RoutedMoE) or f.E == 0 or \
                    self.dtype != torch.bfloat16 or B > 256 or \
                    B * f.top > 1024 or self.cfg.hidden_size % 32 or \
                    f.ff % 32:
                return False
        return True

    def cache_row_dims(self) -> Dict[int, int]:
        """Cache row size per layer RUN that owns paged rows (a looped
        layer owns one set of rows per pass)."""
        out = {}
        for ri, li in enumerate(self.runs):
            m = self.layers[li].mixer
            if isinstance(m, WindowAttnMixer) or \
                    (isinstance(m, LatentAttnMixer) and m.owner):
                out[ri] = m.row
        return out

    def state_shapes(self) -> Dict[tuple, tuple]:
        out = {}
        for ri, li in enumerate(self.runs):
            L = self.layers[li]
            if self.cfg.canon_taps > 1:
                out[(ri, "canon")] = (self.cfg.canon_taps - 1,
                                      self.cfg.hidden_size)
            for k, shp in L.mixer.state_shapes().items():
                out[(ri, k)] = shp
        return out

    # ------------------------------------------------------------ weights
    def weight_bytes(self) -> int:
        return sum(v.numel() * v.element_size()
                   for v in self._name_map.values())

    def _invalidate_host_copies(self):
        for L in self.layers:
            if isinstance(L.ff, TableMoE):
                L.ff._table_host = None

    @torch.no_grad()
    def load_state_dict(self, sd: Dict[str, torch.Tensor], strict: bool = True):
        missing = []
        for name, buf in self._name_map.items():
            src = sd.get(name)
            if src is None:
                missing.append(name)
                continue
            if tuple(src.shape) != tuple(buf.shape) and \
                    src.numel() == buf.numel() and src.dim() == 0:
                src = src.reshape(buf.shape)
            if tuple(src.shape) != tuple(buf.shape):
                raise ValueError(f"{name}: checkpoint shape "
                                 f"{tuple(src.shape)} != {tuple(buf.shape)}")
            buf.copy_(src.to(device=buf.device, dtype=buf.dtype))
        self._invalidate_host_copies()
        if strict and missing:
            raise KeyError(f"missing weights: {sorted(missing)[:5]} ...")

    @torch.no_grad()
    def update_named(self, name: str, tensor: torch.Tensor) -> bool:
        buf = self._name_map.get(name)
        if buf is None:
            return False
        buf.copy_(tensor.reshape(buf.shape).to(device=buf.device,
                                               dtype=buf.dtype))
        self._invalidate_host_copies()
        return True

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        """Random weights of plausible scale (benchmarks, smoke tests)."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        for name, buf in self._name_map.items():
            if buf.dtype == torch.int32:
                E = self._moe_of(name).E
                t = torch.stack([torch.randperm(E, generator=g)[:buf.shape[1]]
                                 for _ in range(buf.shape[0])]).int() \
                    if buf.shape[0] <= 4096 else \
                    torch.rand(buf.shape[0], E, generator=g).argsort(1)[
                        :, :buf.shape[1]].int()
                buf.copy_(t)
            elif self.prenorm and name.endswith(
                    ("norm1", "norm2", "final.norm", ".norm")):
                buf.copy_(1.0 + torch.randn(buf.shape, generator=g) * 0.1)
            elif self.prenorm and name.endswith("a2.b"):
                buf.copy_(2.0 + torch.randn(buf.shape, generator=g))
            elif self.prenorm and (name.endswith(".b")
                                   or name == "loop.step"):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.1)
            elif name == "bigram":
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.5)
            elif self.parallel and name.endswith(
                    ("norm1", "norm2", "final.norm", ".norm")):
                buf.copy_(1.0 + torch.randn(buf.shape, generator=g) * 0.1)
            elif self.parallel and name.endswith(".lam"):
                buf.copy_(torch.randn(buf.shape, generator=g) - 3.0)
            elif self.parallel and name.endswith(".b"):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.2)
            elif name.endswith("mix.pb"):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.5 - 4.0)
            elif self.sandwich and name.endswith(
                    ("norm1", "norm2", "norm1b", "norm2b", "final.norm")):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.1)
            elif name.endswith(("mix.rel", "mlp.correction")):
                buf.copy_(torch.randn(buf.shape, generator=g) *
                          (0.5 if name.endswith("rel") else 0.02))
            elif name.endswith(("norm1", "norm2", "final.norm", ".norm",
                                "mix.D")):
                buf.fill_(1.0)
            elif name.endswith(("A_log", "dt_bias", "w0", "a.b", "sink",
                                "conv.b")):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.5)
            elif name.endswith(("canon1", "mix.conv")):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.3)
            elif name == "embed" and self.cfg.embed_scale != 1.0:
                buf.copy_(torch.randn(buf.shape, generator=g)
                          / self.cfg.embed_scale)
            elif name in ("embed", "side.embed"):
                buf.copy_(torch.randn(buf.shape, generator=g))
            else:
                fan = buf.shape[-1]
                buf.copy_(torch.randn(buf.shape, generator=g) / fan ** 0.5)
        self._invalidate_host_copies()

    @staticmethod
    def _state(states, key, channels: int) -> torch.Tensor:
        """A convolution's history; a one-tap convolution keeps none."""
        t = states.tensors.get(key)
        if t is None:
            t = states.tensors[key] = torch.zeros(
                states.num_slots, 0, channels, dtype=torch.float32,
                device=states.device)
        return t

    def _moe_of(self, name: str):
        return self.layers[int(name.split(".")[0][1:])].ff

    # ------------------------------------------------------------ forward
    @torch.no_grad()
    def forward_batch(self, bt: HybridBatch, cache, states) -> torch.Tensor:
        """Packed rows through every layer; returns the fp32 residual
        stream (N, width) before the final norm.  Writes this step's cache
        rows and advances the sequences' recurrent states in place."""
        if self.sandwich:
            return self._forward_sandwich(bt, cache, states)
        if self.prenorm:
            return self._forward_prenorm(bt, cache, states)
        if self.parallel:
            return self._forward_parallel(bt, cache, states)
        cfg, dt = self.cfg, self.dtype
        eps = cfg.norm_eps
        res = self.embed[bt.tokens].float()
        pending = None                      # mixer/ff output not yet added
        d = cfg.token_side_dim
        for li, L in enumerate(self.layers):
            h = seq.add_rmsnorm_f32res(res, pending, L.norm1, eps, dt)
            h = seq.causal_conv_state(
                h, L.canon, None, self._state(states, (li, "canon"),
                                              cfg.hidden_size),
                bt.cu_q, bt.state_slot, bt.seq_of_tok, True, False, dt)
            pending = L.mixer.forward(h, bt, li, self, cache, states)
            if L.ff is not None:
                h = seq.add_rmsnorm_f32res(res, pending, L.norm2, eps, dt)
                pending = L.ff.forward(h, res, bt)
            x = seq.residual_add_cast(res, pending, dt)
            pending = None
            if d > 0:
                gate = _mm(x, L.side_gate)
                gated = seq.gelu_tanh_mul_rows(gate, self.side_embed,
                                               bt.tokens, li * d)
                seq.add_scaled_unit_rms(res, _mm(gated, L.side_proj),
                                        L.side_norm, eps)
            if self.capture_layers is not None:
                self.capture_layers.append(res.clone())
        return res

    def _forward_sandwich(self, bt: HybridBatch, cache, states):
        """Layer runs of the sandwich style.  Each joint between two
        sublayers is one fused pass: add the normed sublayer output to the
        fp32 residual and norm the result for the next sublayer."""
        cfg, dt = self.cfg, self.dtype
        eps, off = cfg.norm_eps, cfg.norm_offset
        res = self.embed[bt.tokens].float()
        runs = self.runs
        h = seq.add_rmsnorm_f32res(res, None, self.layers[runs[0]].norm1,
                                   eps, dt, off) if runs else None
        for ri, li in enumerate(runs):
            L = self.layers[li]
            nxt = self.layers[runs[ri + 1]].norm1 \
                if ri + 1 < len(runs) else None
            y = L.mixer.forward(h, bt, ri, self, cache, states)
            if L.ff is not None:
                h = seq.add_unit_rms_then_norm(res, y, L.norm1b, L.norm2,
                                               eps, dt, off)
                y = L.ff.forward(h, res, bt)
                post = L.norm2b
            else:
                post = L.norm1b
            if nxt is not None:
                h = seq.add_unit_rms_then_norm(res, y, post, nxt, eps, dt,
                                               off)
            else:
                seq.add_scaled_unit_rms(res, y, post, eps, off)
            if self.capture_layers is not None:
                self.capture_layers.append(res.clone())
        return res

    def embed_rows(self, bt: HybridBatch) -> torch.Tensor:
        """The fp32 embedding output of a packed batch: scaled table row,
        hashed pair row, sinusoid of the position (each if configured)."""
        cfg = self.cfg
        bg = cfg.bigram
        return seq.embed_compose(
            self.embed, bt.tokens, cfg.embed_scale, self.pair_embed,
            bt.prev_tokens, bg.mul_prev if bg else 0, bg.mul_cur if bg else 0,
            bg.buckets if bg else 0, bt.positions, self.pos_inv_freq)

    def _forward_prenorm(self, bt: HybridBatch, cache, states):
        """Layer runs of the pre-norm style.  What a sublayer or the
        token-side input adds to the fp32 stream (times the residual
        multiplier) stays pending until the next norm, which adds it in the
        same pass over the row; what a looped span's pass adds at its start
        (the embedding output again, the pass's vector) joins that pass
        too."""
        cfg, dt = self.cfg, self.dtype
        eps, m, d = cfg.norm_eps, cfg.residual_mult, cfg.token_side_dim
        starts = cfg.pass_starts()
        x0 = self.embed_rows(bt)
        res = x0.clone() if cfg.loop_reinject and len(starts) > 1 else x0
        pending = side = None     # sublayer output / (side output, weight)

        def settle():
            nonlocal pending, side
            if side is not None:
                seq.add_scaled_unit_rms(res, side[0], side[1], eps, scale=m)
            elif pending is not None:
                seq.residual_add_cast(res, pending, torch.float32, scale=m)
            pending = side = None

        for ri, li in enumerate(self.runs):
            L = self.layers[li]
            rep = starts.get(ri)
            extra = x0 if rep and cfg.loop_reinject else None
            vec = self.loop_step[rep] \
                if rep is not None and self.loop_step is not None else None
            if side is not None:
                h = seq.add_unit_rms_then_norm(res, side[0], side[1], L.norm1,
                                               eps, dt, scale=m, extra=extra,
                                               extra_vec=vec)
            else:
                h = seq.add_rmsnorm_f32res(res, pending, L.norm1, eps, dt,
                                           scale=m, extra=extra,
                                           extra_vec=vec)
            side = None
            pending = L.mixer.forward(h, bt, ri, self, cache, states)
            if L.ff is not None:
                h = seq.add_rmsnorm_f32res(res, pending, L.norm2, eps, dt,
                                           scale=m)
                pending = L.ff.forward(h, res, bt)
            if d > 0:
                x = seq.residual_add_cast(res, pending, dt, scale=m)
                pending = None
                gated = seq.gelu_tanh_mul_rows(_mm(x, L.side_gate),
                                               self.side_embed, bt.tokens,
                                               li * d)
                side = (_mm(gated, L.side_proj), L.side_norm)
            if self.capture_layers is not None:
                settle()
                self.capture_layers.append(res.clone())
        settle()
        return res

    def _norms(self, res, y1, g1, y2, g2, w1, w2):
        """A parallel layer's joint: the pending (gated) sublayer outputs
        join the fp32 stream and the new row is normed once for each of
        the next layer's sublayers."""
        cfg = self.cfg
        if cfg.norm_kind == "layer":
            return seq.gated_add_layernorm(res, y1, g1, y2, g2, w1, w2,
                                           cfg.norm_eps, self.dtype)
        for y, g in ((y1, g1), (y2, g2)):
            if y is not None:
                seq.residual_add_cast(
                    res, y if g is None else seq.sigmoid_mul(y, g),
                    torch.float32)
        if w1 is None:
            return None, None
        rms = lambda w: seq.add_rmsnorm_f32res(res, None, w, cfg.norm_eps,
                                               self.dtype, cfg.norm_offset)
        return rms(w1), None if w2 is None else rms(w2)

    def _forward_parallel(self, bt: HybridBatch, cache, states):
        """Layer runs of the parallel style: both sublayers of a run read
        norms of the same stream; their outputs (and gates) stay pending
        until the next run's norms, which add them in the same pass over
        the row."""
        res = self.embed[bt.tokens].float()
        y1 = g1 = y2 = g2 = None
        for ri, li in enumerate(self.runs):
            L = self.layers[li]
            h1, h2 = self._norms(res, y1, g1, y2, g2, L.norm1, L.norm2)
            y1 = L.mixer.forward(h1, bt, ri, self, cache, states)
            g1 = L.mixer.tail_out if L.fused_gate else \
                _mm(h1, L.rg1, L.rg1_b) if L.rg1 is not None else None
            y2 = g2 = None
            if L.ff is not None:
                y2 = L.ff.forward(h2, res, bt)
                g2 = _mm(h2, L.rg2, L.rg2_b) if L.rg2 is not None else None
            if self.capture_layers is not None:
                self._norms(res, y1, g1, y2, g2, None, None)
                y1 = g1 = y2 = g2 = None
                self.capture_layers.append(res.clone())
        self._norms(res, y1, g1, y2, g2, None, None)
        return res

    @torch.no_grad()
    def logits(self, res_rows: torch.Tensor) -> torch.Tensor:
        """Final norm + head on residual rows -> fp32 logits."""
        if self.cfg.norm_kind == "layer":
            h = seq.gated_add_layernorm(
                res_rows.contiguous(), None, None, None, None,
                self.final_norm, None, self.cfg.norm_eps, self.dtype)[0]
        else:
            h = seq.add_rmsnorm_f32res(res_rows.contiguous(), None,
                                       self.final_norm, self.cfg.norm_eps,
                                       self.dtype, self.cfg.norm_offset)
        out = _mm(h, self.lm_head).float()
        if self.cfg.logit_scale != 1.0:
            out = out * self.cfg.logit_scale
        return out
