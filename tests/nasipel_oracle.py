"""Plain, slow implementation of the Nasipel design for the tests.

One function per mechanism, written from the design's equations; whole
sequences only (no cache, no batching, no paging, no recurrent state that
outlives a call).  It shares no code with ``polyrl_amd``: the engine, its
cache manager and its kernels are compared against these functions.

Conventions: ``W`` maps tensor names to torch tensors, linear weights are
[out, in] and applied as ``W @ x``; ``cfg`` is the parsed config dict.
Everything runs in ``DT`` (float64 by default).
"""
import math

import torch

DT = torch.float64


def _f(t):
    return t.to(DT)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * sigmoid(z)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, biased variance, no bias term."""
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * _f(w)


# ------------------------------------------------------------- rotation
def frequencies(dims, base, scaling=None):
    """Per-pair frequencies f_i = base^(-2i/dims) and the amplitude of
    cos/sin; with a 'scaling' entry the long-wave pairs slow down."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / \
            (2 * math.log(base))
    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def turn(vec, pos, freqs, amp, interleaved):
    """Rotate the first 2*len(freqs) entries of a vector by pos * freqs.
    Pairs are (i, i + half) or, interleaved, (2i, 2i + 1)."""
    out = vec.clone()
    half = len(freqs)
    for i, f in enumerate(freqs):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + half)
        c, s = math.cos(pos * f) * amp, math.sin(pos * f) * amp
        out[a] = vec[a] * c - vec[b] * s
        out[b] = vec[b] * c + vec[a] * s
    return out


# ------------------------------------------------------------ attention
def sigmoid_attention(W, p, m, h, eps):
    """Grouped-query attention whose weights are sigmoid(capped score +
    a number per head), not normalised; q and k are rotated, then divided
    by their root mean square; values turn with their position and the
    head's sum turns back by the query's."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), \
        int(m["vdim"])
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    fq, amp = frequencies(dims, base, rot.get("scaling")) if dims \
        else ([], 1.0)
    fv, _ = frequencies(Dv, base)
    cap = float(m.get("softcap") or 0.0)
    q = (h @ _f(W[p + "q"]).t()).view(T, H, D)
    k = (h @ _f(W[p + "k"]).t()).view(T, G, D)
    v = (h @ _f(W[p + "v"]).t()).view(T, G, Dv)
    pb = _f(W[p + "pb"])
    qs = [[unit_rms(turn(q[t, a], t, fq, amp, False), eps) for a in range(H)]
          for t in range(T)]
    ks = [[unit_rms(turn(k[t, g], t, fq, amp, False), eps) for g in range(G)]
          for t in range(T)]
    vs = [[turn(v[t, g], t, fv, 1.0, False) for g in range(G)]
          for t in range(T)]
    K = [torch.stack([ks[t][g] for t in range(T)]) for g in range(G)]
    V = [torch.stack([vs[t][g] for t in range(T)]) for g in range(G)]
    out = torch.zeros(T, H * Dv, dtype=DT)
    for i in range(T):
        for a in range(H):
            g = a // (H // G)
            s = (K[g][:i + 1] @ qs[i][a]) * float(m["scale"])   # keys 0..i
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            w = sigmoid(s + pb[a])                  # one weight per key
            acc = (w.unsqueeze(1) * V[g][:i + 1]).sum(0)
            out[i, a * Dv:(a + 1) * Dv] = turn(acc, -i, fv, 1.0, False)
    return out @ _f(W[p + "o"]).t()


def latent_attention(W, p, m, h, eps):
    """Softmax attention through a shared latent: queries through a normed
    latent of their own; one rotated key part for all heads; a sigmoid
    gate per head on the output."""
    T = h.shape[0]
    H, D, Dr, Dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), \
        int(m["vdim"]), int(m["kv_rank"])
    rot = m["rot"]
    f, amp = frequencies(int(rot["dims"]), float(rot["base"]),
                         rot.get("scaling"))
    cq = unit_rms(h @ _f(W[p + "dq"]).t(), eps) * _f(W[p + "dq.norm"])
    q = (cq @ _f(W[p + "uq"]).t()).view(T, H, D + Dr)
    dkv = h @ _f(W[p + "dkv"]).t()
    c = unit_rms(dkv[:, :R], eps) * _f(W[p + "dkv.norm"])
    kn = (c @ _f(W[p + "uk"]).t()).view(T, H, D)
    vv = (c @ _f(W[p + "uv"]).t()).view(T, H, Dv)
    kr = torch.stack([turn(dkv[t, R:], t, f, amp, True) for t in range(T)])
    gate = sigmoid(h @ _f(W[p + "g"]).t())                # (T, H)
    out = torch.zeros(T, H * Dv, dtype=DT)
    for i in range(T):
        for a in range(H):
            qr = turn(q[i, a, D:], i, f, amp, True)
            s = (kn[:i + 1, a] @ q[i, a, :D] + kr[:i + 1] @ qr) \
                * float(m["scale"])
            w = torch.softmax(s, 0)
            out[i, a * Dv:(a + 1) * Dv] = (w.unsqueeze(1) * vv[:i + 1, a]
                                           ).sum(0) * gate[i, a]
    return out @ _f(W[p + "o"]).t()


# ------------------------------------------------------------ recurrence
def causal_conv(x, w, b):
    """Per-channel convolution over time; w[:, -1] meets the current
    token, zeros stand before the start."""
    T, taps = x.shape[0], w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] = out[t] + w[:, j] * x[src]
        out[t] = out[t] + b
    return out


def gated_linear_recurrence(W, p, m, h, decay_mult=8.0):
    """Two branches of the same width: a GELU branch, and a convolved
    branch that drives a diagonal recurrence with block-diagonal input and
    decay gates; their product leaves through the output matrix."""
    T = h.shape[0]
    C, B = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ _f(W[p + "y"]).t() + _f(W[p + "y.b"]))
    u = causal_conv(h @ _f(W[p + "x"]).t() + _f(W[p + "x.b"]),
                    _f(W[p + "conv"]), _f(W[p + "conv.b"]))
    ub = u.view(T, B, C // B)
    r = sigmoid(torch.einsum("boi,tbi->tbo", _f(W[p + "ra"]), ub)
                + _f(W[p + "ra.b"])).reshape(T, C)
    i = sigmoid(torch.einsum("boi,tbi->tbo", _f(W[p + "ri"]), ub)
                + _f(W[p + "ri.b"])).reshape(T, C)
    log_a = -decay_mult * r * softplus(_f(W[p + "lam"]))
    a = torch.exp(log_a)
    S = torch.zeros(C, dtype=DT)
    out = torch.zeros(T, C, dtype=DT)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] * a[t]) * i[t] * u[t]
        out[t] = S * y[t]
    return out @ _f(W[p + "o"]).t()


# ---------------------------------------------------------- feed-forward
def choose_experts(s, corr, top, groups, keep):
    """Indices of the chosen experts for one token: choice scores are
    s + corr; a group's score is the sum of its two best choice scores;
    only the best ``keep`` groups stay open."""
    E = s.numel()
    choice = (s + corr).tolist()
    per = E // groups
    gs = []
    for g in range(groups):
        best = sorted(choice[g * per:(g + 1) * per], reverse=True)
        gs.append(sum(best[:2]))
    open_groups = sorted(range(groups), key=lambda g: (-gs[g], g))[:keep]
    cand = [e for e in range(E) if e // per in open_groups]
    cand.sort(key=lambda e: (-choice[e], e))
    return cand[:top]


def routed_experts(W, p, f, h):
    r = f["router"]
    E, top = int(r["experts"]), int(r["top"])
    g = r.get("groups") or {}
    z = h @ _f(W[p + "router"]).t()
    s = sigmoid(z)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        idx = choose_experts(s[t], _f(W[p + "correction"]), top,
                             int(g.get("count", 1)), int(g.get("keep", 1)))
        tot = sum(float(s[t, e]) for e in idx) + 1e-20
        for e in idx:
            a = silu(_f(W[f"{p}e{e}.gate"]) @ h[t]) * \
                (_f(W[f"{p}e{e}.up"]) @ h[t])
            out[t] = out[t] + (_f(W[f"{p}e{e}.down"]) @ a) * \
                (float(s[t, e]) / tot * float(r.get("scale", 1.0)))
    return out


# ----------------------------------------------------------------- model
def mixer(W, p, L, h, eps):
    kind = L["type"]
    if kind == "attention":
        return sigmoid_attention(W, p, L["mixer"], h, eps)
    if kind == "latent_attention":
        return latent_attention(W, p, L["mixer"], h, eps)
    if kind == "rglru":
        return gated_linear_recurrence(W, p, L["mixer"], h)
    raise ValueError(kind)


def layer(W, li, L, x, eps):
    """Both sublayers read the same x; each result passes a sigmoid gate
    computed from the sublayer's own input."""
    p = f"l{li}."
    h1 = layer_norm(x, W[p + "norm1"], eps)
    add = mixer(W, p + "mix.", L, h1, eps) * \
        sigmoid(h1 @ _f(W[p + "rg1"]).t() + _f(W[p + "rg1.b"]))
    if L.get("mlp") is not None:
        h2 = layer_norm(x, W[p + "norm2"], eps)
        add = add + routed_experts(W, p + "mlp.", L["mlp"], h2) * \
            sigmoid(h2 @ _f(W[p + "rg2"]).t() + _f(W[p + "rg2.b"]))
    return x + add


def forward(cfg, W, tokens, collect=None):
    """Logits [T, vocab] of one whole sequence; ``collect`` gathers the
    stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = _f(W["embed"])[torch.tensor(tokens)]
    for li, L in enumerate(cfg["layers"]):
        x = layer(W, li, L, x, eps)
        if collect is not None:
            collect.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ _f(W["head"]).t()


# --------------------------------------------------------------- weights
def random_weights(cfg, seed=0):
    """name -> tensor for a config; values are bf16-representable so every
    engine dtype loads them exactly."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = int(cfg["width"]), int(cfg["vocab"])

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean) \
            .bfloat16().float()

    def lin(o, i, gain=1.0):
        return rnd(o, i, std=gain / math.sqrt(i))
    W = {"embed": rnd(V, Wd), "final.norm": rnd(Wd, std=0.1, mean=1.0),
         "head": lin(V, Wd)}
    for li, L in enumerate(cfg["layers"]):
        p, m, kind = f"l{li}.", L["mixer"], L["type"]
        W[p + "norm1"] = rnd(Wd, std=0.1, mean=1.0)
        W[p + "rg1"], W[p + "rg1.b"] = lin(Wd, Wd), rnd(Wd, std=0.5)
        q = p + "mix."
        if kind == "rglru":
            C, B, taps = int(m["width"]), int(m["blocks"]), int(m["conv"])
            bw = C // B
            W[q + "y"], W[q + "y.b"] = lin(C, Wd), rnd(C, std=0.3)
            W[q + "x"], W[q + "x.b"] = lin(C, Wd), rnd(C, std=0.3)
            W[q + "conv"] = rnd(C, taps, std=0.5)
            W[q + "conv.b"] = rnd(C, std=0.2)
            for n in ("ra", "ri"):
                W[q + n] = rnd(B, bw, bw, std=1.0 / math.sqrt(bw))
                W[q + n + ".b"] = rnd(B, bw, std=0.5)
            W[q + "lam"] = rnd(C, std=1.0, mean=-2.0)
            W[q + "o"] = lin(Wd, C)
        elif kind == "attention":
            H, G = int(m["heads"]), int(m["kv_heads"])
            D, Dv = int(m["dim"]), int(m["vdim"])
            W[q + "q"], W[q + "k"] = lin(H * D, Wd), lin(G * D, Wd)
            W[q + "v"] = lin(G * Dv, Wd)
            W[q + "pb"] = rnd(H, std=0.5, mean=-2.0)
            W[q + "o"] = lin(Wd, H * Dv)
        else:
            H, D, Dr = int(m["heads"]), int(m["dim"]), int(m["rot_dim"])
            Dv, R, Rq = int(m["vdim"]), int(m["kv_rank"]), int(m["q_rank"])
            W[q + "dq"] = lin(Rq, Wd)
            W[q + "dq.norm"] = rnd(Rq, std=0.1, mean=1.0)
            W[q + "uq"] = lin(H * (D + Dr), Rq, gain=2.0)
            W[q + "dkv"] = lin(R + Dr, Wd)
            W[q + "dkv.norm"] = rnd(R, std=0.1, mean=1.0)
            W[q + "uk"] = lin(H * D, R, gain=2.0)
            W[q + "uv"] = lin(H * Dv, R)
            W[q + "g"] = lin(H, Wd, gain=2.0)
            W[q + "o"] = lin(Wd, H * Dv)
        f = L.get("mlp")
        if f is None:
            continue
        W[p + "norm2"] = rnd(Wd, std=0.1, mean=1.0)
        W[p + "rg2"], W[p + "rg2.b"] = lin(Wd, Wd), rnd(Wd, std=0.5)
        E, ff = int(f["router"]["experts"]), int(f["expert"]["ff"])
        for e in range(E):
            W[f"{p}mlp.e{e}.gate"] = lin(ff, Wd)
            W[f"{p}mlp.e{e}.up"] = lin(ff, Wd)
            W[f"{p}mlp.e{e}.down"] = lin(Wd, ff)
        W[p + "mlp.router"] = lin(E, Wd, gain=3.0)
        W[p + "mlp.correction"] = rnd(E, std=0.1)
    return W
