"""Plain, slow implementation of the Vurivik design for the tests.

One function per mechanism, written from the design's equations; whole
sequences only (no cache, no batching, no paging).  It shares no code with
``polyrl_amd``: the engine, its cache manager and its kernels are compared
against these functions.

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


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * _f(w)


# ------------------------------------------------------------- embedding
def bigram_row(prev, cur, bg):
    """Row of the pair table for (previous, current); the table's last row
    serves a sequence's first token."""
    if prev is None:
        return int(bg["buckets"])
    return (prev * int(bg["mul_prev"]) + cur * int(bg["mul_cur"])) \
        % int(bg["buckets"])


def sinusoid(p, width):
    """Position vector: angles a_i = p / 10000^(2i/width); sines at the
    even places, cosines at the odd ones."""
    out = torch.zeros(width, dtype=DT)
    for i in range((width + 1) // 2):
        ang = p * 10000.0 ** (-2.0 * i / width)
        out[2 * i] = math.sin(ang)
        if 2 * i + 1 < width:
            out[2 * i + 1] = math.cos(ang)
    return out


def embed(cfg, W, tokens):
    width = int(cfg["width"])
    e = cfg["embedding"]
    rows = []
    for p, t in enumerate(tokens):
        x = _f(W["embed"][t]) * float(e["scale"])
        if e.get("bigram"):
            prev = tokens[p - 1] if p > 0 else None
            x = x + _f(W["bigram"][bigram_row(prev, t, e["bigram"])])
        rows.append(x + sinusoid(p, width))
    return torch.stack(rows)


# ------------------------------------------------- gated linear attention
def gla_decay(h, W, p, heads, dim, tau):
    """Per key channel: sigmoid(low-rank projection + bias)^(1/tau)."""
    z = _f(W[p + "a2"]) @ (_f(W[p + "a1"]) @ h) + _f(W[p + "a2.b"])
    return (sigmoid(z) ** (1.0 / tau)).view(heads, dim)


def gla_mixer(hs, W, p, m, eps):
    """hs [T, width].  State per head [dim, vdim], zero at the start:
    S <- diag(decay) S + k v^T, read out with the scaled query."""
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    tau = float(m["tau"])
    S = torch.zeros(H, D, Dv, dtype=DT)
    out = []
    for h in hs:
        q = (_f(W[p + "q"]) @ h).view(H, D) * D ** -0.5
        k = (_f(W[p + "k"]) @ h).view(H, D)
        v = (_f(W[p + "v"]) @ h).view(H, Dv)
        a = gla_decay(h, W, p, H, D, tau)
        S = a.unsqueeze(-1) * S + k.unsqueeze(-1) * v.unsqueeze(1)
        o = torch.einsum("hkv,hk->hv", S, q)
        o = unit_rms(o, eps) * _f(W[p + "norm"])         # per head, shared w
        o = o.reshape(-1) * silu(_f(W[p + "g"]) @ h)
        out.append(_f(W[p + "o"]) @ o)
    return torch.stack(out)


# -------------------------------------------------------------- attention
def query_temperature(p, qt):
    if not qt:
        return 1.0
    return 1.0 + float(qt["coef"]) * math.log(
        math.floor((p + 1) / int(qt["every"])) + 1)


def attention_mixer(hs, W, p, m):
    """Causal grouped-query softmax attention with one extra term
    exp(sink_h) in every head's denominator (nothing is added to the
    weighted sum for it)."""
    H, G = int(m["heads"]), int(m["kv_heads"])
    D, Dv = int(m["dim"]), int(m["vdim"])
    T = hs.shape[0]
    q = (hs @ _f(W[p + "q"]).t() + _f(W[p + "q.b"])).view(T, H, D)
    k = (hs @ _f(W[p + "k"]).t() + _f(W[p + "k.b"])).view(T, G, D)
    v = (hs @ _f(W[p + "v"]).t() + _f(W[p + "v.b"])).view(T, G, Dv)
    sink = _f(W[p + "sink"])
    out = torch.zeros(T, H, Dv, dtype=DT)
    for i in range(T):
        qi = q[i] * query_temperature(i, m.get("q_temp"))
        for h in range(H):
            g = h // (H // G)
            s = (k[:i + 1, g] @ qi[h]) * float(m["scale"])
            mx = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - mx)
            den = e.sum() + math.exp(float(sink[h]) - mx)
            out[i, h] = (e / den) @ v[:i + 1, g]
    return out.reshape(T, H * Dv) @ _f(W[p + "o"]).t()


# ----------------------------------------------------------- feed-forward
def dense_ff(hs, W, p, f):
    lim = float(f["limit"])
    g = (hs @ _f(W[p + "gate"]).t() + _f(W[p + "gate.b"])).clamp(max=lim)
    u = (hs @ _f(W[p + "up"]).t() + _f(W[p + "up.b"])).clamp(-lim, lim)
    y = g * sigmoid(1.702 * g) * (u + 1.0)
    return y @ _f(W[p + "down"]).t() + _f(W[p + "down.b"])


def token_side(x, W, li, tokens, d, eps):
    """Per-layer token input: y = proj(gelu_tanh(gate x) * e); returns
    y / rms(y) * w (the caller scales and adds it)."""
    e = _f(W["side.embed"][torch.tensor(tokens)][:, li * d:(li + 1) * d])
    g = gelu_tanh(x @ _f(W[f"l{li}.side.gate"]).t()) * e
    y = g @ _f(W[f"l{li}.side.proj"]).t()
    return unit_rms(y, eps) * _f(W[f"l{li}.side.norm"])


# ------------------------------------------------------------------ stack
def run_order(cfg):
    """(layer, pass number or None) for every layer run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    a, b, t = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    out = [(i, None) for i in range(a)]
    for r in range(t):
        out += [(i, r) for i in range(a, b)]
    return out + [(i, None) for i in range(b, n)]


def forward(cfg, W, tokens):
    """Returns (logits [T, vocab], residual after every layer run)."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    d = int((cfg.get("token_side") or {}).get("dim", 0))
    lp = cfg.get("loop")
    x0 = embed(cfg, W, tokens)
    x = x0.clone()
    after = []
    for li, rep in run_order(cfg):
        L = cfg["layers"][li]
        if rep is not None and li == int(lp["start"]):
            if rep > 0:
                x = x + x0
            x = x + _f(W["loop.step"][rep])
        p = f"l{li}."
        h = rms_norm(x, W[p + "norm1"], eps)
        if L["type"] == "gla":
            y = gla_mixer(h, W, p + "mix.", L["mixer"], eps)
        elif L["type"] == "attention":
            y = attention_mixer(h, W, p + "mix.", L["mixer"])
        else:
            raise ValueError(L["type"])
        x = x + mult * y
        if L.get("mlp") is not None:
            h = rms_norm(x, W[p + "norm2"], eps)
            x = x + mult * dense_ff(h, W, p + "mlp.", L["mlp"])
        if d > 0:
            x = x + mult * token_side(x, W, li, tokens, d, eps)
        after.append(x.clone())
    h = rms_norm(x, W["final.norm"], eps)
    return h @ _f(W["head"]).t(), after


def make_weights(cfg, seed=0, scale=1.0, rank=6):
    """Random weights (bf16-representable) for a config; names and shapes
    as a checkpoint holds them (``rank``: rows of the decay's first
    projection, which only the tensor's shape gives)."""
    g = torch.Generator().manual_seed(seed)
    width, V = int(cfg["width"]), int(cfg["vocab"])

    def rnd(*shape, s=None):
        s = (shape[-1] ** -0.5 if len(shape) > 1 else 0.5) if s is None else s
        return (torch.randn(*shape, generator=g) * s * scale) \
            .bfloat16().float()

    def near_one(n):
        return (1.0 + 0.2 * torch.randn(n, generator=g)).bfloat16().float()

    W = {"embed": rnd(V, width, s=0.5), "head": rnd(V, width),
         "final.norm": near_one(width)}
    bg = cfg["embedding"].get("bigram")
    if bg:
        W["bigram"] = rnd(int(bg["buckets"]) + 1, width, s=0.5)
    lp = cfg.get("loop")
    if lp:
        W["loop.step"] = rnd(int(lp["times"]), width, s=0.3)
    d = int((cfg.get("token_side") or {}).get("dim", 0))
    if d:
        W["side.embed"] = rnd(V, d * len(cfg["layers"]), s=1.0)
    for li, L in enumerate(cfg["layers"]):
        p, m = f"l{li}.", L["mixer"]
        W[p + "norm1"] = near_one(width)
        H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        if L["type"] == "gla":
            W.update({p + "mix.q": rnd(H * D, width),
                      p + "mix.k": rnd(H * D, width),
                      p + "mix.v": rnd(H * Dv, width),
                      p + "mix.g": rnd(H * Dv, width),
                      p + "mix.o": rnd(width, H * Dv),
                      p + "mix.norm": near_one(Dv),
                      p + "mix.a1": rnd(rank, width),
                      p + "mix.a2": rnd(H * D, rank),
                      p + "mix.a2.b": rnd(H * D, s=1.0) + 2.0})
        else:
            G = int(m["kv_heads"])
            W.update({p + "mix.q": rnd(H * D, width),
                      p + "mix.q.b": rnd(H * D, s=0.2),
                      p + "mix.k": rnd(G * D, width),
                      p + "mix.k.b": rnd(G * D, s=0.2),
                      p + "mix.v": rnd(G * Dv, width),
                      p + "mix.v.b": rnd(G * Dv, s=0.2),
                      p + "mix.sink": rnd(H, s=1.0),
                      p + "mix.o": rnd(width, H * Dv)})
        f = L.get("mlp")
        if f is not None:
            ff = int(f["ff"])
            W.update({p + "norm2": near_one(width),
                      p + "mlp.gate": rnd(ff, width, s=2.0 * width ** -0.5),
                      p + "mlp.gate.b": rnd(ff, s=0.3),
                      p + "mlp.up": rnd(ff, width, s=2.0 * width ** -0.5),
                      p + "mlp.up.b": rnd(ff, s=0.3),
                      p + "mlp.down": rnd(width, ff),
                      p + "mlp.down.b": rnd(width, s=0.2)})
        if d:
            W.update({p + "side.gate": rnd(d, width),
                      p + "side.proj": rnd(width, d),
                      p + "side.norm": near_one(width)})
    return W
