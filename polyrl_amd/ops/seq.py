"""Sequence-mixer ops for hybrid decoders: fp32-residual norms (plain and
offset weights, fused joints, scaled branches, the gated layer-norm joint of
parallel layers), the composed embedding (scaled row + hashed pair row +
sinusoid), stateful causal convolutions, the generalised delta rule, gated
linear attention, the selective state-space scan, the real-gated linear
recurrence, windowed or causal latent attention with an optional softmax
sink, grouped-query (window or causal; softmax or sigmoid weights) attention
over paged K/V rows, and table-routed or router-chosen expert feed-forwards.

Same policy as the rest of ``polyrl_amd.ops``: on a HIP device the in-tree
extension is REQUIRED (csrc/seq_*.hip, templated on the activation type:
bf16 or fp32); CPU tensors run the PyTorch forms in seq_ref.py.  What the
recurrences consume (decays, step sizes, gates, unit keys, states) and all
norms, scores and softmax weights are fp32 inside the kernels for either
activation type.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import seq_ref as R


_SEQ_EXT = None
_SEQ_ERR: Optional[str] = None
try:
    from polyrl_amd import _hip_seq as _SEQ_EXT  # type: ignore
except Exception as e:  # pragma: no cover - import-environment dependent
    _SEQ_ERR = repr(e)


def seq_extension_loaded() -> bool:
    return _SEQ_EXT is not None


def _ext():
    if _SEQ_EXT is None:
        raise RuntimeError(
            "polyrl_amd._hip_seq extension is required on GPU but failed to "
            f"load ({_SEQ_ERR}). Build it in-tree: "
            "PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace")
    return _SEQ_EXT


def add_rmsnorm_f32res(res: torch.Tensor, y: Optional[torch.Tensor],
                       weight: torch.Tensor, eps: float,
                       out_dtype: torch.dtype,
                       offset: float = 0.0, scale: float = 1.0,
                       extra: Optional[torch.Tensor] = None,
                       extra_vec: Optional[torch.Tensor] = None
                       ) -> torch.Tensor:
    """res (N, D) fp32 += scale * y [+ extra (N, D) fp32] [+ extra_vec (D,)
    fp32] in place, then RMS-norm(res) * (offset + weight) -> out_dtype.
    ``weight`` holds one number (for all coordinates) or D."""
    if res.is_cuda:
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        e = torch.Tensor()
        _ext().seq_add_rmsnorm(out, res, y if y is not None else e,
                               weight, eps, 0, offset, e, scale,
                               extra if extra is not None else e,
                               extra_vec if extra_vec is not None else e)
        return out
    return R.add_rmsnorm_f32res(res, y, weight, eps, out_dtype, offset, scale,
                                extra, extra_vec)


def residual_add_cast(res: torch.Tensor, y: Optional[torch.Tensor],
                      out_dtype: torch.dtype,
                      scale: float = 1.0) -> torch.Tensor:
    """res += scale * y in place; returns res in out_dtype (res itself for
    fp32)."""
    if res.is_cuda:
        if y is None and out_dtype == torch.float32:
            return res
        out = res if out_dtype == torch.float32 else \
            torch.empty(res.shape, dtype=out_dtype, device=res.device)
        e = torch.Tensor()
        _ext().seq_add_rmsnorm(out, res, y if y is not None else e,
                               e, 0.0, 1, 0.0, e, scale, e, e)
        return out
    return R.residual_add_cast(res, y, out_dtype, scale)


def add_scaled_unit_rms(res: torch.Tensor, y: torch.Tensor,
                        weight: torch.Tensor, eps: float,
                        offset: float = 0.0, scale: float = 1.0) -> None:
    """res += scale * y / rms(y) * (offset + weight), in place (weight (D,)
    fp32)."""
    if res.is_cuda:
        e = torch.Tensor()
        _ext().seq_add_rmsnorm(res, res, y, weight, eps, 2, offset, e, scale,
                               e, e)
        return
    R.add_scaled_unit_rms(res, y, weight, eps, offset, scale)


def sinusoid_inv_freq(width: int, base: float, device) -> torch.Tensor:
    """f_i = base^(-2i/width) for the ceil(width/2) sin/cos pairs of a
    position vector, rounded once to fp32."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return (base ** (-2.0 * i / width)).float().to(device)


def embed_compose(table, tokens, scale: float, pair_table, prev_tokens,
                  mul_prev: int, mul_cur: int, buckets: int, positions,
                  inv_freq) -> torch.Tensor:
    """The fp32 embedding output (N, D): table[token] * scale
    [+ pair_table[(prev * mul_prev + token * mul_cur) mod buckets], row
    ``buckets`` where prev < 0 (a sequence's first token)]
    [+ the sinusoid of the position: with angles a_i = fp32(p) * inv_freq[i],
    sines sit at the even entries (2i) and cosines at the odd ones]."""
    if table.is_cuda:
        out = torch.empty(tokens.shape[0], table.shape[1],
                          dtype=torch.float32, device=table.device)
        if tokens.shape[0]:
            e = torch.Tensor()
            _ext().seq_embed_compose(
                out, table, tokens, scale,
                pair_table if pair_table is not None else e,
                prev_tokens if pair_table is not None else e,
                mul_prev, mul_cur, buckets, positions,
                inv_freq if inv_freq is not None else e)
        return out
    return R.embed_compose(table, tokens, scale, pair_table, prev_tokens,
                           mul_prev, mul_cur, buckets, positions, inv_freq)


def add_unit_rms_then_norm(res: torch.Tensor, y: torch.Tensor,
                           w_post: torch.Tensor, w_next: torch.Tensor,
                           eps: float, out_dtype: torch.dtype,
                           offset: float = 0.0, scale: float = 1.0,
                           extra: Optional[torch.Tensor] = None,
                           extra_vec: Optional[torch.Tensor] = None
                           ) -> torch.Tensor:
    """The joint between two normed sublayers in one pass over the row:
    res += scale * y / rms(y) * (offset + w_post) [+ extra (N, D) fp32]
    [+ extra_vec (D,) fp32] in place, then returns
    res / rms(res) * (offset + w_next) as out_dtype."""
    if res.is_cuda:
        out = torch.empty(res.shape, dtype=out_dtype, device=res.device)
        e = torch.Tensor()
        _ext().seq_add_rmsnorm(out, res, y, w_post, eps, 3, offset, w_next,
                               scale, extra if extra is not None else e,
                               extra_vec if extra_vec is not None else e)
        return out
    return R.add_unit_rms_then_norm(res, y, w_post, w_next, eps, out_dtype,
                                    offset, scale, extra, extra_vec)


def causal_conv_state(x, w, bias, state, cu_q, state_slot, seq_of_tok,
                      add_input: bool, act_silu: bool,
                      out_dtype) -> torch.Tensor:
    """Depthwise causal convolution over each sequence's rows with the last
    taps-1 inputs carried in ``state`` (slots, taps-1, C) fp32.
    y_t = sum_j w[:, j] x_(t-taps+1+j) [+ bias] [+ x_t], optional SiLU.
    ``x`` may be a column slice (row-strided view)."""
    if x.is_cuda:
        out = torch.empty(x.shape[0], w.shape[0], dtype=out_dtype,
                          device=x.device)
        if x.shape[0]:
            _ext().seq_causal_conv(out, x, w,
                                   bias if bias is not None else torch.Tensor(),
                                   state, cu_q, state_slot, seq_of_tok,
                                   add_input, act_silu)
        return out
    return R.causal_conv_state(x, w, bias, state, cu_q, state_slot,
                               seq_of_tok, add_input, act_silu, out_dtype)


def delta_rule(r, k, v, w_lin, a_lin, g, w0, a_bias, norm_w, state, cu_q,
               state_slot, decay_scale: float, key_eps: float, eps: float,
               out_dtype) -> torch.Tensor:
    """Generalised delta rule over packed rows; ``state`` (slots, H, Dk, Dv)
    fp32 in place.  Per head: w = exp(-decay_scale*sigmoid(w_lin + w0)),
    a = sigmoid(a_lin + a_bias), u = k/sqrt(|k|^2+key_eps),
    S <- diag(w) S - (a*u)(u^T S) + k v^T, o = S^T r; returns
    o/rms_head(o) * norm_w * sigmoid(g).  Inputs may be column slices."""
    if r.is_cuda:
        slots, H, Dk, Dv = state.shape
        out = torch.empty(r.shape[0], H * Dv, dtype=out_dtype, device=r.device)
        if r.shape[0]:
            o = torch.empty(r.shape[0], H * Dv, dtype=torch.float32,
                            device=r.device)
            _ext().seq_delta_rule(o, r, k, v, w_lin, a_lin, w0, a_bias, state,
                                  cu_q, state_slot, decay_scale, key_eps)
            # per-head unit RMS, plain weight, sigmoid output gate
            _ext().seq_group_rmsnorm(out, o, norm_w, H, eps, g, 1)
        return out
    return R.delta_rule(r, k, v, w_lin, a_lin, g, w0, a_bias, norm_w, state,
                        cu_q, state_slot, decay_scale, key_eps, eps, out_dtype)


def ssm_scan(xbc, dt, z, dt_bias, a_log, d_skip, state, cu_q, state_slot,
             groups: int) -> torch.Tensor:
    """Selective state-space scan; ``state`` (slots, H, N, P) fp32 in place.
    step = softplus(dt + dt_bias); S <- exp(-exp(a_log)*step) S + step B x^T;
    y = S^T C + d_skip*x; returns y * silu(z) as fp32 (N, H*P)."""
    if xbc.is_cuda:
        slots, H, Ns, P = state.shape
        out = torch.empty(xbc.shape[0], H * P, dtype=torch.float32,
                          device=xbc.device)
        if xbc.shape[0]:
            _ext().seq_ssm_scan(out, xbc, dt, z, dt_bias, a_log, d_skip,
                                state, cu_q, state_slot, groups)
        return out
    return R.ssm_scan(xbc, dt, z, dt_bias, a_log, d_skip, state, cu_q,
                      state_slot, groups)


def group_rmsnorm(y, weight, groups: int, eps: float, out_dtype,
                  gate=None, gate_act: str = "sigmoid"):
    """RMS-norm each of ``groups`` equal parts of a row by its own root mean
    square, times weight ((D,), or (D/groups,) shared by the groups), times
    sigmoid(gate) or silu(gate) when a gate (N, D) is given."""
    if y.is_cuda:
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        if y.shape[0]:
            _ext().seq_group_rmsnorm(
                out, y, weight, groups, eps,
                gate if gate is not None else torch.Tensor(),
                {"sigmoid": 1, "silu": 2}[gate_act])
        return out
    return R.group_rmsnorm(y, weight, groups, eps, out_dtype, gate, gate_act)


def gla_scan(q, k, v, z_lin, z_bias, state, cu_q, state_slot,
             q_scale: float, inv_tau: float) -> torch.Tensor:
    """Gated linear attention over packed rows; ``state`` (slots, H, Dk, Dv)
    fp32 in place.  Per head: decay = exp(log_sigmoid(z_lin + z_bias) *
    inv_tau) per key channel, S <- diag(decay) S + k v^T,
    o = S^T (q * q_scale).  Returns o as fp32 (N, H*Dv), not normed.
    Inputs may be column slices."""
    if q.is_cuda:
        slots, H, Dk, Dv = state.shape
        out = torch.empty(q.shape[0], H * Dv, dtype=torch.float32,
                          device=q.device)
        if q.shape[0]:
            _ext().seq_gla_scan(out, q, k, v, z_lin, z_bias, state, cu_q,
                                state_slot, q_scale, inv_tau)
        return out
    return R.gla_scan(q, k, v, z_lin, z_bias, state, cu_q, state_slot,
                      q_scale, inv_tau)


def rope_inv_freq(dims: int, base: float, device) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, rounded once to fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (base ** (-2.0 * i / dims)).float().to(device)


def rope_partial_(q, offset: int, inv_freq, positions, amp: float = 1.0,
                  interleaved: bool = False):
    """RoPE in place on q[..., offset:offset+dims] of a (N, H, Dh) tensor;
    angle = fp32(position) * inv_freq, fp32 cos/sin times ``amp``; pairs are
    (i, i + dims/2) or, ``interleaved``, (2i, 2i + 1)."""
    if q.is_cuda:
        if q.shape[0] and inv_freq.numel():
            _ext().seq_rope_partial(q, offset, inv_freq, positions, amp,
                                    interleaved)
        return q
    return R.rope_partial_(q, offset, inv_freq, positions, amp, interleaved)


def latent_kv_store(dkv, rank: int, norm_w, eps: float, positions, inv_freq,
                    cache, slot_mapping, amp: float = 1.0,
                    interleaved: bool = False) -> None:
    """Row n of dkv = [latent (rank) | shared key part]: RMS-norm the latent
    (times norm_w), rotate the key part (pairs and amplitude as in
    :func:`rope_partial_`), and write both into the paged latent cache
    (pages, page_size, rank+rot) at slot_mapping[n]."""
    if dkv.is_cuda:
        if dkv.shape[0]:
            _ext().seq_latent_kv_store(dkv, rank, norm_w, eps, positions,
                                       inv_freq, cache, slot_mapping, amp,
                                       interleaved)
        return
    R.latent_kv_store(dkv, rank, norm_w, eps, positions, inv_freq, cache,
                      slot_mapping, amp, interleaved)


def attention_tiles(lens, device):
    """Row tiles of a packed batch for the matrix-core attention kernel:
    (first row, rows) per tile of at most 64 consecutive tokens of one
    sequence, and the mode (1 when every sequence brings a single token:
    a tile is then one token and up to 64 of its heads)."""
    n0, cnt, at = [], [], 0
    for n in lens:
        for s in range(0, n, 64):
            n0.append(at + s)
            cnt.append(min(64, n - s))
        at += n
    mode = 1 if lens and max(lens) == 1 else 0
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    return i32(n0), i32(cnt), mode


def latent_window_attention(q_lat, q_rot, cache, page_table, seq_of_tok,
                            positions, window: int, sink, scale: float,
                            out_dtype, tiles=None) -> torch.Tensor:
    """Windowed attention of every row against its sequence's paged latent
    cache: score_j = (q_lat . c_j + q_rot . kr_j) * scale for
    0 <= pos - j < window; softmax whose denominator also holds exp(sink_h)
    when ``sink`` (H,) is given; returns sum_j p_j c_j, (N, H, rank).  All
    heads share the cache rows."""
    row = q_lat.shape[2] + q_rot.shape[2]
    if q_lat.is_cuda and sink is None:
        sink = torch.Tensor()
    if q_lat.is_cuda and tiles is not None and q_lat.shape[0] and \
            q_lat.dtype == torch.bfloat16 and row % 8 == 0 and row <= 576:
        out = torch.empty(q_lat.shape, dtype=out_dtype, device=q_lat.device)
        _ext().seq_latent_attention_mfma(
            out, torch.cat([q_lat, q_rot], -1), cache, page_table, seq_of_tok,
            positions, tiles[0], tiles[1], q_lat.shape[2], window, sink,
            scale, tiles[2])
        return out
    if q_lat.is_cuda:
        out = torch.empty(q_lat.shape, dtype=out_dtype, device=q_lat.device)
        if q_lat.shape[0]:
            _ext().seq_latent_attention(out, q_lat, q_rot, cache, page_table,
                                        seq_of_tok, positions, window, sink,
                                        scale)
        return out
    return R.latent_window_attention(q_lat, q_rot, cache, page_table,
                                     seq_of_tok, positions, window, sink,
                                     scale, out_dtype)


def gqa_prepare_store(q, k, v, q_norm, k_norm, eps: float, inv_freq,
                      amp: float, positions, cache, slot_mapping, H: int,
                      G: int, D: int, Dv: int, head_unit: bool = False,
                      v_inv_freq=None) -> torch.Tensor:
    """Queries and cache rows of grouped-query attention from a step's
    projections (column slices allowed).  Optional RMS norm over the WHOLE
    query row and the whole key row (weights q_norm / k_norm), then
    rotate-half RoPE on the first 2*len(inv_freq) entries of every head with
    angle fp32(position)*inv_freq and cos/sin scaled by ``amp``.  The cache
    row of a token, (pages, page_size, G*D + G*Dv) at slot_mapping[n], is
    [keys (normed, rotated) | values]; values are ``v`` or, when ``v`` is
    None, the key projection as it came in.  ``head_unit`` divides every
    query and key head by its root mean square after the rotation (no
    weight); ``v_inv_freq`` (Dv/2,) rotates every value head over all its
    entries by its position (pairs (m, m + Dv/2)) before it is cached.
    Returns the queries (N, H*D)."""
    if q.is_cuda:
        out = torch.empty(q.shape[0], H * D, dtype=q.dtype, device=q.device)
        if q.shape[0]:
            e = torch.Tensor()
            _ext().seq_gqa_prepare_store(
                out, q, k, v if v is not None else e,
                q_norm if q_norm is not None else e,
                k_norm if k_norm is not None else e, eps,
                inv_freq if inv_freq is not None else e, amp, positions,
                cache, slot_mapping, H, G, D, Dv, head_unit,
                v_inv_freq if v_inv_freq is not None else e)
        return out
    return R.gqa_prepare_store(q, k, v, q_norm, k_norm, eps, inv_freq, amp,
                               positions, cache, slot_mapping, H, G, D, Dv,
                               head_unit, v_inv_freq)


def gqa_window_attention(q, cache, page_table, seq_of_tok, positions, H: int,
                         G: int, D: int, Dv: int, window: int,
                         keep_first: int, rel, dist_bucket, gate,
                         scale: float, out_dtype, tiles=None, sink=None,
                         q_temp_coef: float = 0.0,
                         q_temp_every: int = 1, softcap: float = 0.0,
                         head_bias=None, sigmoid_weights: bool = False,
                         v_inv_freq=None) -> torch.Tensor:
    """Attention of every row against its sequence's paged K/V rows
    (layout of :func:`gqa_prepare_store`).  Row at position p sees key j if
    j <= p and (p - j < window or j < keep_first).  score = q.k * scale
    * (1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1))
    [+ rel[dist_bucket[p - j], head]]; with ``sink`` (H,) fp32 the
    denominator also holds exp(sink[h]) once; ``gate`` (N, H) multiplies
    head h's output by sigmoid(gate[n, h]).  Query head h reads key/value
    head h // (H // G).  ``softcap`` > 0 replaces the score by
    softcap * tanh(score / softcap); ``head_bias`` (H,) fp32 is added after
    that; with ``sigmoid_weights`` a visible key weighs
    sigmoid(score) instead of its softmax share (no normalisation over
    keys); ``v_inv_freq`` (Dv/2,) turns every head's sum back by the row's
    position (the inverse of the value rotation of
    :func:`gqa_prepare_store`) before the gate.  Returns (N, H*Dv)."""
    if q.is_cuda:
        out = torch.empty(q.shape[0], H * Dv, dtype=out_dtype,
                          device=q.device)
        if q.shape[0]:
            e = torch.Tensor()
            args = (cache, page_table, seq_of_tok, positions, H, G, D, Dv,
                    window, keep_first, rel if rel is not None else e,
                    dist_bucket if dist_bucket is not None else e,
                    gate if gate is not None else e, scale,
                    sink if sink is not None else e, q_temp_coef,
                    q_temp_every, softcap,
                    head_bias if head_bias is not None else e,
                    sigmoid_weights,
                    v_inv_freq if v_inv_freq is not None else e)
            if tiles is not None and tiles[2] == 0 and \
                    gqa_mfma_supported(q, D, Dv):
                _ext().seq_gqa_window_attention_mfma(out, q, tiles[0],
                                                     tiles[1], *args)
            else:
                _ext().seq_gqa_window_attention(out, q, *args)
        return out
    return R.gqa_window_attention(q, cache, page_table, seq_of_tok, positions,
                                  H, G, D, Dv, window, keep_first, rel,
                                  dist_bucket, gate, scale, out_dtype, sink,
                                  q_temp_coef, q_temp_every, softcap,
                                  head_bias, sigmoid_weights, v_inv_freq)


def gqa_mfma_supported(q, D: int, Dv: int) -> bool:
    """The matrix-core kernel serves bf16 batches that hold a prompt
    portion, with head sizes in multiples of 8 up to 128; everything else
    (fp32, odd sizes, steps of single tokens) runs one wave per row."""
    return (q.dtype == torch.bfloat16 and D % 8 == 0 and Dv % 8 == 0
            and D <= 128 and Dv <= 128)


def moe_route(logits, correction, top: int, groups: int, keep: int,
              act: str = "softmax", group_top: int = 1):
    """Router choice for every row of fp32 logits (N, E): s = softmax (or,
    ``act="sigmoid"``, the logistic function of every logit on its own),
    choice score = s + correction; experts form ``groups`` equal groups of
    neighbours, a group's score is the sum of its ``group_top`` largest
    choice scores, only the ``keep`` groups with the largest score stay
    eligible; the ``top`` largest eligible choice scores win.  Returns
    (index int32 (N, top), s at those indices fp32 (N, top))."""
    if logits.is_cuda:
        N = logits.shape[0]
        idx = torch.empty(N, top, dtype=torch.int32, device=logits.device)
        w = torch.empty(N, top, dtype=torch.float32, device=logits.device)
        if N:
            _ext().seq_moe_route(idx, w, logits, correction, groups, keep,
                                 {"softmax": 0, "sigmoid": 1}[act], group_top)
        return idx, w
    return R.moe_route(logits, correction, top, groups, keep, act, group_top)


def gelu_erf(x):
    """Exact (erf) GELU; x may be a column slice."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        if x.shape[0]:
            _ext().seq_act_mul(out, x, x, 3, 0.0, 0.0, 0.0)
        return out
    return R.gelu_erf(x)


def moe_routed_ffn_supported(h, top: int, ff: int) -> bool:
    """The fused expert path serves bf16 decode-sized batches on the GPU."""
    return moe_table_ffn_supported(h, top, ff)


def moe_routed_ffn(h, idx, w_up, w_down, gated: bool = False) -> torch.Tensor:
    """Router-chosen experts: row t*top+k of the result is expert
    idx[t, k] applied to h[t]; rows whose index is >= E (identity experts)
    are left unwritten.  Plain experts: W_down gelu_erf(W_up h) with w_up
    (E, ff, W); ``gated``: W_down (silu(W_gate h) * W_up h) with w_up
    (E, 2*ff, W) holding gate rows then up rows.  w_down (E, W, ff)."""
    if h.is_cuda:
        N, top = idx.shape
        y = torch.empty(N * top, h.shape[1], dtype=h.dtype, device=h.device)
        act = torch.empty(N * top, w_down.shape[2], dtype=h.dtype,
                          device=h.device)
        _ext().seq_moe_routed_ffn(y, act, h, idx, w_up, w_down, gated)
        return y
    return R.moe_routed_ffn(h, idx, w_up, w_down, gated)


def moe_weighted_combine(ys, idx, w, h, shared, E: int, weight_eps: float,
                         out_dtype, scale: float = 1.0) -> torch.Tensor:
    """y[n] = sum_k w'[n,k] * (ys[n*top+k] if idx[n,k] < E else h[n])
    [+ shared[n]] with w' = scale * w / (sum_k w + weight_eps), fp32
    sums."""
    if ys.is_cuda:
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        if h.shape[0]:
            _ext().seq_moe_weighted_combine(
                out, ys, idx, w, h,
                shared if shared is not None else torch.Tensor(), E,
                weight_eps, scale)
        return out
    return R.moe_weighted_combine(ys, idx, w, h, shared, E, weight_eps,
                                  out_dtype, scale)


def silu_mul_any(gate, up):
    """silu(gate) * up for bf16 or fp32 (row-strided views allowed)."""
    if gate.is_cuda:
        out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        if gate.shape[0]:
            _ext().seq_act_mul(out, gate, up, 0, 0.0, 0.0, 0.0)
        return out
    return R.silu_mul_any(gate, up)


def clamped_glu(gate, up, limit: float, slope: float, shift: float):
    """g * sigmoid(slope * g) * (u + shift) with g = min(gate, limit) and
    u = clamp(up, -limit, limit) (row-strided views allowed)."""
    if gate.is_cuda:
        out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        if gate.shape[0]:
            _ext().seq_act_mul(out, gate, up, 4, limit, slope, shift)
        return out
    return R.clamped_glu(gate, up, limit, slope, shift)


def sigmoid_mul(x, gate):
    """x * sigmoid(gate)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        if x.shape[0]:
            _ext().seq_act_mul(out, gate, x, 1, 0.0, 0.0, 0.0)
        return out
    return R.sigmoid_mul(x, gate)


def sigmoid_mul_heads(x, gate):
    """x (N, H*Dv) with head h's entries times sigmoid(gate[n, h])."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        if x.shape[0]:
            _ext().seq_sigmoid_mul_heads(out, x, gate)
        return out
    return R.sigmoid_mul_heads(x, gate)


def gated_add_layernorm(res, y1, g1, y2, g2, w1, w2, eps: float, out_dtype):
    """The joint of a layer whose two sublayers read the same stream:
    res (N, D) fp32 += y1 * sigmoid(g1) [+ y2 * sigmoid(g2)] in place (a
    missing gate means a plain add, a missing y1 no add), then the layer
    norm of the new row, (x - mean) / sqrt(var + eps), once with each of
    the weights w1 and w2 (D,) fp32: the two norms share their statistics.
    Returns (h1, h2) in out_dtype; h2 is None without w2, both without
    w1."""
    if res.is_cuda:
        if y1 is None and w1 is None:
            return None, None
        e = torch.Tensor()
        new = lambda: torch.empty(res.shape, dtype=out_dtype,
                                  device=res.device)
        h1 = new() if w1 is not None else None
        h2 = new() if w2 is not None else None
        if res.shape[0]:
            o = lambda t: t if t is not None else e
            _ext().seq_gated_add_layernorm(o(h1), o(h2), res, o(y1), o(g1),
                                           o(y2), o(g2), o(w1), o(w2), eps)
        return h1, h2
    return R.gated_add_layernorm(res, y1, g1, y2, g2, w1, w2, eps, out_dtype)


def rglru_scan(u, gates, gate_bias, lam, y_lin, state, cu_q, state_slot,
               decay_mult: float, out_dtype, max_rows: int = 0) -> torch.Tensor:
    """Real-gated linear recurrence over packed rows; ``state`` (slots, C)
    fp32 in place.  Channels form B equal blocks of bw; ``gates`` (B, N,
    2*bw) fp32 holds the block-diagonal products for the decay gate (first
    bw) and the input gate, ``gate_bias`` (B, 2*bw) their biases.  Per
    channel: r = sigmoid(.), i = sigmoid(.), log a = -decay_mult * r *
    softplus(lam), S <- a S + sqrt(1 - a^2) * i * u; returns
    S * gelu_tanh(y_lin) (N, C).  ``u`` and ``y_lin`` may be column
    slices.  ``max_rows`` bounds the rows of one sequence (0 = unknown):
    long portions are cut into segments that run in parallel."""
    if u.is_cuda:
        out = torch.empty(u.shape, dtype=out_dtype, device=u.device)
        if u.shape[0]:
            _ext().seq_rglru_scan(out, u, gates, gate_bias, lam, y_lin, state,
                                  cu_q, state_slot, decay_mult, max_rows)
        return out
    return R.rglru_scan(u, gates, gate_bias, lam, y_lin, state, cu_q,
                        state_slot, decay_mult, out_dtype)


def tanh_act(x):
    """tanh(x) (contiguous result; x may be a column slice)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        if x.shape[0]:
            _ext().seq_act_mul(out, x, x, 2, 0.0, 0.0, 0.0)
        return out
    return R.tanh_act(x)


def gelu_tanh_mul_rows(gate, table, tokens, col0: int):
    """gelu_tanh(gate) * table[tokens, col0:col0+d] for gate (N, d)."""
    if gate.is_cuda:
        out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        if gate.shape[0]:
            _ext().seq_gelu_mul_rows(out, gate, table, tokens, col0)
        return out
    return R.gelu_tanh_mul_rows(gate, table, tokens, col0)


def moe_combine_(res, y_sorted, inv_idx, scale: float) -> None:
    """res[n] += scale * sum_k y_sorted[inv_idx[n, k]] (fp32 residual)."""
    if res.is_cuda:
        if res.shape[0]:
            _ext().seq_moe_combine(res, y_sorted, inv_idx, scale)
        return
    R.moe_combine_(res, y_sorted, inv_idx, scale)


def moe_table_ffn_supported(h, top: int, ff: int) -> bool:
    """The fused expert path serves bf16 decode-sized batches on the GPU."""
    return (h.is_cuda and h.dtype == torch.bfloat16
            and h.shape[0] * top <= 1024 and h.shape[1] % 32 == 0
            and ff % 32 == 0)


def moe_table_ffn(h, tokens, table, w_gu, w_down) -> torch.Tensor:
    """Table-routed gated experts: row t*top+k of the result is expert
    table[tokens[t], k] applied to h[t] (silu(Wg h) * (Wu h), then Wd).
    w_gu (E, 2*ff, W) holds gate rows then up rows; w_down (E, W, ff)."""
    N, top = h.shape[0], table.shape[1]
    if h.is_cuda:
        y = torch.empty(N * top, h.shape[1], dtype=h.dtype, device=h.device)
        act = torch.empty(N * top, w_down.shape[2], dtype=h.dtype,
                          device=h.device)
        _ext().seq_moe_table_ffn(y, act, h, tokens, table, w_gu, w_down)
        return y
    return R.moe_table_ffn(h, tokens, table, w_gu, w_down)
