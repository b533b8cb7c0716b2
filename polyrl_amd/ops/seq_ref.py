"""PyTorch forms of the sequence-mixer ops (ops/seq.py): the CPU execution
path of the no-GPU test tier and the numerics reference of each HIP kernel in
csrc/seq_*.hip.  Batches are packed: row n belongs to sequence
``seq_of_tok[n]``; ``cu_q`` bounds each sequence's rows; recurrent state
lives in ``state[state_slot[b]]`` and is read and written in place.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def _w(weight: torch.Tensor) -> torch.Tensor:
    return weight.float().reshape(-1)


def add_rmsnorm_f32res(res, y, weight, eps, out_dtype, offset=0.0,
                       scale=1.0, extra=None, extra_vec=None):
    if y is not None:
        res.add_(y.float() * scale if scale != 1.0 else y.float())
    if extra is not None:
        res.add_(extra)
    if extra_vec is not None:
        res.add_(extra_vec.float())
    inv = torch.rsqrt(res.pow(2).mean(-1, keepdim=True) + eps)
    return (res * inv * (_w(weight) + offset)).to(out_dtype)


def residual_add_cast(res, y, out_dtype, scale=1.0):
    if y is not None:
        res.add_(y.float() * scale if scale != 1.0 else y.float())
    return res if out_dtype == torch.float32 else res.to(out_dtype)


def add_scaled_unit_rms(res, y, weight, eps, offset=0.0, scale=1.0):
    yf = y.float()
    inv = torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps)
    add = yf * inv * (_w(weight) + offset)
    res.add_(add * scale if scale != 1.0 else add)


def add_unit_rms_then_norm(res, y, w_post, w_next, eps, out_dtype, offset,
                           scale=1.0, extra=None, extra_vec=None):
    add_scaled_unit_rms(res, y, w_post, eps, offset, scale)
    return add_rmsnorm_f32res(res, None, w_next, eps, out_dtype, offset,
                              extra=extra, extra_vec=extra_vec)


def causal_conv_state(x, w, bias, state, cu_q, state_slot, seq_of_tok,
                      add_input, act_silu, out_dtype):
    taps = w.shape[1]
    C = w.shape[0]
    out = torch.empty(x.shape[0], C, dtype=out_dtype, device=x.device)
    cu = cu_q.tolist()
    wf = w.float()
    for b, slot in enumerate(state_slot.tolist()):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        xs = x[q0:q1].float()
        hist = torch.cat([state[slot], xs], 0)          # (taps-1+L, C)
        y = torch.zeros_like(xs)
        for j in range(taps):
            y += wf[:, j] * hist[j:j + (q1 - q0)]
        if bias is not None:
            y += bias.float()
        if add_input:
            y += xs
        if act_silu:
            y = y * torch.sigmoid(y)
        out[q0:q1] = y.to(out_dtype)
        if taps > 1:
            state[slot] = hist[-(taps - 1):]
    return out


def delta_rule(r, k, v, w_lin, a_lin, g, w0, a_bias, norm_w, state, cu_q,
               state_slot, decay_scale, key_eps, eps, out_dtype):
    slots, H, Dk, Dv = state.shape
    N = r.shape[0]
    out = torch.empty(N, H * Dv, dtype=torch.float32, device=r.device)
    rf = r.float().view(N, H, Dk)
    kf = k.float().view(N, H, Dk)
    vf = v.float().view(N, H, Dv)
    dec = torch.exp(-decay_scale * torch.sigmoid(
        w_lin.float() + w0.float())).view(N, H, Dk)
    rem = torch.sigmoid(a_lin.float() + a_bias.float()).view(N, H, Dk)
    unit = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + key_eps)
    cu = cu_q.tolist()
    for b, slot in enumerate(state_slot.tolist()):
        S = state[slot]                                  # (H, Dk, Dv)
        for n in range(cu[b], cu[b + 1]):
            proj = torch.einsum("hk,hkv->hv", unit[n], S)
            S = dec[n].unsqueeze(-1) * S \
                - (rem[n] * unit[n]).unsqueeze(-1) * proj.unsqueeze(1) \
                + kf[n].unsqueeze(-1) * vf[n].unsqueeze(1)
            o = torch.einsum("hk,hkv->hv", rf[n], S)
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
            out[n] = o.reshape(-1)
        state[slot] = S
    out = out * norm_w.float() * torch.sigmoid(g.float())
    return out.to(out_dtype)


def ssm_scan(xbc, dt, z, dt_bias, a_log, d_skip, state, cu_q, state_slot,
             groups):
    slots, H, Ns, P = state.shape
    N = xbc.shape[0]
    inner = H * P
    xf = xbc[:, :inner].float().view(N, H, P)
    Bf = xbc[:, inner:inner + groups * Ns].float().view(N, groups, Ns)
    Cf = xbc[:, inner + groups * Ns:].float().view(N, groups, Ns)
    per = H // groups
    Bh = Bf.repeat_interleave(per, dim=1)                # (N, H, Ns)
    Ch = Cf.repeat_interleave(per, dim=1)
    step = torch.nn.functional.softplus(dt.float() + dt_bias.float(),
                                        threshold=1e9)   # (N, H), no clamp
    decay = torch.exp(-torch.exp(a_log.float()) * step)
    y = torch.empty(N, H, P, dtype=torch.float32, device=xbc.device)
    cu = cu_q.tolist()
    for b, slot in enumerate(state_slot.tolist()):
        S = state[slot]                                  # (H, Ns, P)
        for n in range(cu[b], cu[b + 1]):
            S = decay[n].view(H, 1, 1) * S + step[n].view(H, 1, 1) * \
                Bh[n].unsqueeze(-1) * xf[n].unsqueeze(1)
            y[n] = torch.einsum("hn,hnp->hp", Ch[n], S) \
                + d_skip.float().view(H, 1) * xf[n]
        state[slot] = S
    zf = z.float()
    return y.view(N, inner) * (zf * torch.sigmoid(zf))


def group_rmsnorm(y, weight, groups, eps, out_dtype, gate=None,
                  gate_act="sigmoid"):
    N, D = y.shape
    yf = y.float().view(N, groups, D // groups)
    yf = yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps)
    wf = weight.float()
    if wf.numel() != D:                      # one weight row for all groups
        wf = wf.repeat(groups)
    out = yf.view(N, D) * wf
    if gate is not None:
        gf = gate.float()
        out = out * (torch.sigmoid(gf) if gate_act == "sigmoid"
                     else gf * torch.sigmoid(gf))
    return out.to(out_dtype)


def embed_compose(table, tokens, scale, pair_table, prev_tokens, mul_prev,
                  mul_cur, buckets, positions, inv_freq):
    x = table[tokens.long()].float() * scale
    if pair_table is not None:
        prev, cur = prev_tokens.long(), tokens.long()
        row = torch.where(prev < 0, torch.full_like(cur, buckets),
                          (prev.clamp(min=0) * mul_prev + cur * mul_cur)
                          % buckets)
        x = x + pair_table[row].float()
    if inv_freq is not None:
        D = table.shape[1]
        ang = positions.float().unsqueeze(-1) * inv_freq.float()
        pe = torch.stack([torch.sin(ang), torch.cos(ang)], -1)
        x = x + pe.reshape(x.shape[0], -1)[:, :D]
    return x


def gla_scan(q, k, v, z_lin, z_bias, state, cu_q, state_slot, q_scale,
             inv_tau):
    slots, H, Dk, Dv = state.shape
    N = q.shape[0]
    qf = q.float().view(N, H, Dk) * q_scale
    kf = k.float().view(N, H, Dk)
    vf = v.float().view(N, H, Dv)
    dec = torch.exp(torch.nn.functional.logsigmoid(
        z_lin.float() + z_bias.float()) * inv_tau).view(N, H, Dk)
    out = torch.empty(N, H * Dv, dtype=torch.float32, device=q.device)
    cu = cu_q.tolist()
    for b, slot in enumerate(state_slot.tolist()):
        S = state[slot]                                  # (H, Dk, Dv)
        for n in range(cu[b], cu[b + 1]):
            S = dec[n].unsqueeze(-1) * S \
                + kf[n].unsqueeze(-1) * vf[n].unsqueeze(1)
            out[n] = torch.einsum("hk,hkv->hv", qf[n], S).reshape(-1)
        state[slot] = S
    return out


def clamped_glu(gate, up, limit, slope, shift):
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return (g * torch.sigmoid(slope * g) * (u + shift)).to(gate.dtype)


def _rotate(x, positions, inv_freq, amp=1.0, interleaved=False,
            negate=False):
    """x (N, ..., dims) rotated over the last axis by position * inv_freq;
    pairs are (i, i + dims/2) or, interleaved, (2i, 2i + 1); cos and sin
    times ``amp``; ``negate`` turns the other way."""
    half = inv_freq.numel()
    ang = positions.float().unsqueeze(-1) * inv_freq.float()   # (N, half)
    while ang.dim() < x.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang) * amp, torch.sin(ang) * amp
    if negate:
        s = -s
    if interleaved:
        a, b = x[..., 0:2 * half:2].float(), x[..., 1:2 * half:2].float()
        return torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)
    a, b = x[..., :half].float(), x[..., half:2 * half].float()
    return torch.cat([a * c - b * s, b * c + a * s], -1)


def rope_partial_(q, offset, inv_freq, positions, amp=1.0, interleaved=False):
    dims = 2 * inv_freq.numel()
    if dims == 0:
        return q
    part = q[..., offset:offset + dims]
    part.copy_(_rotate(part, positions, inv_freq, amp, interleaved)
               .to(q.dtype))
    return q


def latent_kv_store(dkv, rank, norm_w, eps, positions, inv_freq, cache,
                    slot_mapping, amp=1.0, interleaved=False):
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = dkv[:, rank:].float().clone()
    dims = 2 * inv_freq.numel()
    if dims:
        kr[:, :dims] = _rotate(kr[:, :dims], positions, inv_freq, amp,
                               interleaved)
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping.long()] = torch.cat([c, kr], -1).to(cache.dtype)


def latent_window_attention(q_lat, q_rot, cache, page_table, seq_of_tok,
                            positions, window, sink, scale, out_dtype):
    N, H, R = q_lat.shape
    ps = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1]).float()
    out = torch.empty(N, H, R, dtype=torch.float32, device=q_lat.device)
    ptab = page_table.tolist()
    for n, (b, p) in enumerate(zip(seq_of_tok.tolist(), positions.tolist())):
        lo = max(0, p - window + 1)
        rows = torch.tensor([ptab[b][j // ps] * ps + j % ps
                             for j in range(lo, p + 1)], dtype=torch.long)
        kv = flat[rows]                                  # (L, R + rd)
        s = (q_lat[n].float() @ kv[:, :R].t()
             + q_rot[n].float() @ kv[:, R:].t()) * scale   # (H, L)
        if sink is not None:
            s = torch.cat([s, sink.float().view(H, 1)], 1)
            pr = torch.softmax(s, -1)[:, :-1]
        else:
            pr = torch.softmax(s, -1)
        out[n] = pr @ kv[:, :R]
    return out.to(out_dtype)


def silu_mul_any(gate, up):
    gf = gate.float()
    return (gf * torch.sigmoid(gf) * up.float()).to(gate.dtype)


def sigmoid_mul(x, gate):
    return (x.float() * torch.sigmoid(gate.float())).to(x.dtype)


def tanh_act(x):
    return torch.tanh(x.float()).to(x.dtype)


def gelu_tanh_mul_rows(gate, table, tokens, col0):
    zf = gate.float()
    c = math.sqrt(2.0 / math.pi)
    act = 0.5 * zf * (1.0 + torch.tanh(c * (zf + 0.044715 * zf ** 3)))
    e = table[tokens.long(), col0:col0 + gate.shape[1]].float()
    return (act * e).to(gate.dtype)


def moe_combine_(res, y_sorted, inv_idx, scale):
    res.add_(y_sorted.float()[inv_idx.long()].sum(1) * scale)


def moe_table_ffn(h, tokens, table, w_gu, w_down):
    N, top = h.shape[0], table.shape[1]
    ff = w_down.shape[2]
    y = torch.empty(N * top, h.shape[1], dtype=h.dtype, device=h.device)
    for t in range(N):
        for k, e in enumerate(table[tokens[t]].tolist()):
            gu = w_gu[e].float() @ h[t].float()
            a = (gu[:ff] * torch.sigmoid(gu[:ff]) * gu[ff:]).to(h.dtype)
            y[t * top + k] = (w_down[e].float() @ a.float()).to(h.dtype)
    return y


def gelu_erf(x):
    xf = x.float()
    return (0.5 * xf * (1.0 + torch.erf(xf * (1.0 / math.sqrt(2.0))))
            ).to(x.dtype)


def gqa_prepare_store(q, k, v, q_norm, k_norm, eps, inv_freq, amp, positions,
                      cache, slot_mapping, H, G, D, Dv, head_unit=False,
                      v_inv_freq=None):
    N = q.shape[0]
    qf, kf = q.float(), k.float()
    vf = kf if v is None else v.float()
    if q_norm is not None:
        qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) \
            * q_norm.float()
        kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) \
            * k_norm.float()
    qf, kf = qf.reshape(N, H, D).clone(), kf.reshape(N, G, D).clone()
    half = 0 if inv_freq is None else inv_freq.numel()
    if half:
        ang = positions.float().unsqueeze(-1) * inv_freq.float()
        c = (torch.cos(ang) * amp).unsqueeze(1)
        s = (torch.sin(ang) * amp).unsqueeze(1)
        for t in (qf, kf):
            a, b = t[..., :half].clone(), t[..., half:2 * half].clone()
            t[..., :half] = a * c - b * s
            t[..., half:2 * half] = b * c + a * s
    if head_unit:
        qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps)
        kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps)
    if v_inv_freq is not None and v_inv_freq.numel():
        vf = _rotate(vf.reshape(N, G, Dv), positions, v_inv_freq)
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping.long()] = torch.cat(
        [kf.reshape(N, G * D), vf.reshape(N, G * Dv)], -1).to(cache.dtype)
    return qf.reshape(N, H * D).to(q.dtype)


def gqa_window_attention(q, cache, page_table, seq_of_tok, positions, H, G,
                         D, Dv, window, keep_first, rel, dist_bucket, gate,
                         scale, out_dtype, sink=None, q_temp_coef=0.0,
                         q_temp_every=1, softcap=0.0, head_bias=None,
                         sigmoid_weights=False, v_inv_freq=None):
    N = q.shape[0]
    ps = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1]).float()
    out = torch.empty(N, H, Dv, dtype=torch.float32, device=q.device)
    ptab = page_table.tolist()
    qf = q.float().view(N, H, D)
    per = H // G
    for n, (b, p) in enumerate(zip(seq_of_tok.tolist(), positions.tolist())):
        lo = max(0, p - window + 1)
        js = list(range(0, min(keep_first, lo))) + list(range(lo, p + 1))
        rows = torch.tensor([ptab[b][j // ps] * ps + j % ps for j in js],
                            dtype=torch.long)
        kv = flat[rows]
        kk = kv[:, :G * D].view(-1, G, D).repeat_interleave(per, 1)
        vv = kv[:, G * D:].view(-1, G, Dv).repeat_interleave(per, 1)
        sc = scale
        if q_temp_coef != 0.0:
            sc = scale * (1.0 + q_temp_coef
                          * math.log((p + 1) // q_temp_every + 1))
        s = torch.einsum("hd,jhd->hj", qf[n], kk) * sc
        if rel is not None:
            dist = torch.tensor([p - j for j in js], dtype=torch.long)
            s = s + rel.float()[dist_bucket.long()[dist]].t()
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if head_bias is not None:
            s = s + head_bias.float().view(H, 1)
        if sigmoid_weights:
            pr = torch.sigmoid(s)
        elif sink is not None:
            pr = torch.softmax(
                torch.cat([s, sink.float().view(H, 1)], 1), -1)[:, :-1]
        else:
            pr = torch.softmax(s, -1)
        o = torch.einsum("hj,jhv->hv", pr, vv)
        if v_inv_freq is not None and v_inv_freq.numel():
            o = _rotate(o.unsqueeze(0), torch.tensor([p]), v_inv_freq,
                        negate=True)[0]
        if gate is not None:
            o = o * torch.sigmoid(gate[n].float()).unsqueeze(-1)
        out[n] = o
    return out.view(N, H * Dv).to(out_dtype)


def moe_route(logits, correction, top, groups, keep, act="softmax",
              group_top=1):
    s = torch.softmax(logits.float(), -1) if act == "softmax" \
        else torch.sigmoid(logits.float())
    choice = s + correction.float()
    N, E = s.shape
    if groups > 1:
        per = choice.view(N, groups, E // groups)
        best = per.topk(min(group_top, E // groups), -1).values.sum(-1)
        kept = best.topk(keep, -1).indices
        open_ = torch.zeros(N, groups, dtype=torch.bool, device=s.device)
        open_.scatter_(1, kept, True)
        choice = choice.masked_fill(
            ~open_.repeat_interleave(E // groups, 1), float("-inf"))
    idx = choice.topk(top, -1).indices
    return idx.int(), s.gather(1, idx)


def moe_routed_ffn(h, idx, w_up, w_down, gated=False):
    N, top = idx.shape
    E = w_up.shape[0]
    y = torch.zeros(N * top, h.shape[1], dtype=h.dtype, device=h.device)
    flat = idx.reshape(-1)
    for e in torch.unique(flat).tolist():
        if e >= E:
            continue
        sl = (flat == e).nonzero().squeeze(1)
        a = h[sl // top] @ w_up[e].t()
        if gated:
            ff = w_down.shape[2]
            a = silu_mul_any(a[:, :ff], a[:, ff:])
        else:
            a = gelu_erf(a)
        y[sl] = a @ w_down[e].t()
    return y


def moe_weighted_combine(ys, idx, w, h, shared, E, weight_eps, out_dtype,
                         scale=1.0):
    N, top = idx.shape
    wn = w.float() / (w.float().sum(-1, keepdim=True) + weight_eps) * scale
    rows = ys.float().view(N, top, -1)
    ident = (idx >= E).unsqueeze(-1)
    rows = torch.where(ident, h.float().unsqueeze(1).expand_as(rows), rows)
    y = (rows * wn.unsqueeze(-1)).sum(1)
    if shared is not None:
        y = y + shared.float()
    return y.to(out_dtype)


def sigmoid_mul_heads(x, gate):
    N, H = gate.shape
    return (x.float().view(N, H, -1)
            * torch.sigmoid(gate.float()).unsqueeze(-1)
            ).view(N, -1).to(x.dtype)


def gated_add_layernorm(res, y1, g1, y2, g2, w1, w2, eps, out_dtype):
    if y1 is not None:
        add = y1.float() * torch.sigmoid(g1.float()) if g1 is not None \
            else y1.float()
        if y2 is not None:
            add = add + (y2.float() * torch.sigmoid(g2.float())
                         if g2 is not None else y2.float())
        res.add_(add)
    if w1 is None:
        return None, None
    d = res - res.mean(-1, keepdim=True)
    unit = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps)
    return ((unit * w1.float()).to(out_dtype),
            None if w2 is None else (unit * w2.float()).to(out_dtype))


def gelu_tanh(z):
    c = math.sqrt(2.0 / math.pi)
    return 0.5 * z * (1.0 + torch.tanh(c * (z + 0.044715 * z ** 3)))


def rglru_scan(u, gates, gate_bias, lam, y_lin, state, cu_q, state_slot,
               decay_mult, out_dtype):
    N, C = u.shape
    B, bw = gate_bias.shape[0], gate_bias.shape[1] // 2
    g = gates.float() + gate_bias.float().unsqueeze(1)       # (B, N, 2bw)
    r = torch.sigmoid(g[..., :bw]).permute(1, 0, 2).reshape(N, C)
    i = torch.sigmoid(g[..., bw:]).permute(1, 0, 2).reshape(N, C)
    log_a = -decay_mult * r * torch.nn.functional.softplus(
        lam.float(), threshold=1e9)
    a = torch.exp(log_a)
    drive = torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.float()
    y = gelu_tanh(y_lin.float())
    out = torch.empty(N, C, dtype=torch.float32, device=u.device)
    cu = cu_q.tolist()
    for b, slot in enumerate(state_slot.tolist()):
        S = state[slot]
        for n in range(cu[b], cu[b + 1]):
            S = a[n] * S + drive[n]
            out[n] = S * y[n]
        state[slot] = S
    return out.to(out_dtype)
