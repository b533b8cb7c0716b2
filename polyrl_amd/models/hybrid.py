"""Configuration of hybrid decoders: a stack whose layers each pick one
sequence mixer (recurrent, state-space, gated linear attention, a real-gated
linear recurrence, latent attention or grouped-query attention) and one
feed-forward (dense, table-routed experts, router-chosen experts, or none).

The Bizusun design is the first family described this way, Kuforax the
second, Vurivik the third, Nasipel the fourth.  Everything that
can differ between two models of a family is a field here and is read from
the checkpoint's ``config.json``; constants that the design fixes (the decay
constant of the delta rule, its key epsilon) are defaults of the mixer
parameters, so another design can set them differently.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class DeltaRuleSpec:
    """Generalised delta rule: per-channel decay and removal rate."""
    heads: int
    dim: int
    decay_rank: Optional[int] = None      # rows of w1; None = from the tensor
    decay_scale: float = math.exp(-0.5)   # w = exp(-decay_scale * sigmoid(.))
    key_eps: float = 1e-6                 # unit key: k / sqrt(sum k^2 + eps)
    kind: str = "general_delta"


@dataclass
class GLASpec:
    """Gated linear attention: a matrix state per head with one decay per
    key channel, ``decay = sigmoid(low-rank projection + bias)^(1/tau)``;
    the query is scaled by ``dim^(-1/2)``."""
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int] = None      # rows of a1; None = from the tensor
    kind: str = "gla"


@dataclass
class RGLRUSpec:
    """Recurrent block with a real-gated linear recurrent unit: a GELU
    branch and a convolved branch of ``width`` channels each; the convolved
    branch drives a per-channel recurrence whose decay gate and input gate
    are block-diagonal (``blocks`` equal blocks); decay
    ``a = exp(-decay_mult * r * softplus(lam))``, input scaled by
    ``sqrt(1 - a^2)``."""
    width: int
    blocks: int
    conv: int = 4
    decay_mult: float = 8.0
    kind: str = "rglru"


@dataclass
class SSMSpec:
    """Mamba-2 style selective state space layer."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    norm_groups: int = 1
    conv: int = 4
    kind: str = "mamba2"

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class LatentAttnSpec:
    """Multi-head attention over a shared low-rank latent, windowed or
    (``window = UNBOUNDED``) causal.  Optional parts, each a parameter: a
    normed low-rank latent for the queries (``q_rank`` > 0: tensors 'dq',
    'dq.norm', 'uq' instead of 'q'), a learned logit per head in the softmax
    denominator (``sink``), the output gate per entry (``gate="element"``,
    'g' has heads * vdim rows) or per head (``gate="head"``, 'g' has one row
    per head), and a rotation given as a :class:`RopeSpec` (``rope``:
    interleaved pairs, YaRN) instead of plain rotate-half."""
    heads: int
    dim: int              # unrotated query/key size per head
    rot_dim: int          # rotated query/key size per head (key part shared)
    vdim: int
    kv_rank: int
    window: int           # a query sees itself and window-1 tokens before it
    scale: float
    rope_base: float = 10000.0
    rope_dims: Optional[int] = None       # rotated pairs cover the first dims
    kv_from: Optional[int] = None         # reuse that layer's latent cache
    q_rank: int = 0
    sink: bool = True
    gate: str = "element"
    rope: Optional["RopeSpec"] = None
    kind: str = "latent_attention"

    def __post_init__(self):
        if self.rope is not None:
            self.rope_base, self.rope_dims = self.rope.base, self.rope.dims
        if self.rope_dims is None:
            self.rope_dims = self.rot_dim


@dataclass
class RopeSpec:
    """Rotary positions on the first ``dims`` entries of every head; pair i
    is (i, i + dims/2) (rotate-half) or, ``interleaved``, (2i, 2i + 1).
    ``factor`` > 1 switches on YaRN: pairs that turn fewer than
    ``slow`` times within ``original`` positions have their frequency divided
    by ``factor``, pairs that turn more than ``fast`` times keep it, a linear
    ramp joins the two, and cos/sin are scaled by ``amp_slope*ln(factor)+1``."""
    dims: int
    base: float = 10000.0
    factor: float = 1.0
    original: float = 0.0
    fast: float = 32.0
    slow: float = 1.0
    amp_slope: float = 0.1
    interleaved: bool = False

    def inv_freq_and_amp(self):
        """(per-pair frequencies as Python floats, cos/sin amplitude)."""
        dims, half = self.dims, self.dims // 2
        f = [self.base ** (-2.0 * i / dims) for i in range(half)]
        if self.factor == 1.0 or self.original <= 0:
            return f, 1.0

        def pair_of(turns):
            return dims * math.log(self.original / (2 * math.pi * turns)) / \
                (2 * math.log(self.base))
        lo = max(math.floor(pair_of(self.fast)), 0)
        hi = min(math.ceil(pair_of(self.slow)), dims - 1)
        out = []
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f[i] / self.factor * ramp + f[i] * (1.0 - ramp))
        return out, self.amp_slope * math.log(self.factor) + 1.0


UNBOUNDED = 1 << 30       # a window no sequence reaches


@dataclass
class WindowAttnSpec:
    """Grouped-query softmax attention over a sliding window of a paged
    K/V cache.  Optional parts, each a parameter: rotary positions
    (``rope``), first tokens that stay visible (``keep_first``), RMS norms
    over the whole query / key projection (``qk_norm``), values taken from
    the raw key projection (``values_from_keys``: no value matrix), one
    sigmoid output gate per head (``head_gate``), and a learned bias per
    (distance bucket, head) added to the scaled scores (``bias_far`` > 0:
    the bucket of distance n is n below half the table's rows, logarithmic
    steps up to ``bias_far`` above), biases on the query / key / value
    projections (``qkv_bias``), one learned logit per head that joins the
    softmax denominator and contributes no value row (``sink``), and a query
    temperature ``1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)``
    at position p.  ``window = UNBOUNDED`` is plain causal attention.
    Further parts: every query and key head divided by its root mean square
    after the rotation (``head_unit_norm``, no weight), scores capped as
    ``softcap * tanh(score / softcap)``, a learned number per head added to
    the capped score (``head_bias``, tensor 'pb'), weights
    ``sigmoid(score)`` per visible key instead of a softmax over the keys
    (``weights="sigmoid"``), and values that are rotated by their position
    over all ``vdim`` entries before they are cached, the head's sum being
    turned back by the query's position (``value_rope_base`` > 0; pairs
    (m, m + vdim/2), frequencies base^(-2m/vdim), never scaled)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    scale: float
    keep_first: int = 0
    qkv_bias: bool = False
    sink: bool = False
    q_temp_coef: float = 0.0
    q_temp_every: int = 1
    rope: Optional[RopeSpec] = None
    qk_norm: bool = False
    values_from_keys: bool = False
    head_gate: bool = False
    bias_far: float = 0.0
    bias_rows: Optional[int] = None       # rows of the table; None = tensor
    head_unit_norm: bool = False
    softcap: float = 0.0
    head_bias: bool = False
    weights: str = "softmax"
    value_rope_base: float = 0.0
    kind: str = "attention"

    def bucket_of_distance(self) -> List[int]:
        """Bias-table row for every distance 0 .. window-1."""
        rows, far = int(self.bias_rows), float(self.bias_far)
        half = rows // 2
        out = []
        for n in range(self.window):
            if n < half:
                out.append(n)
            else:
                out.append(min(rows - 1, half + int(math.floor(
                    math.log(n / half) / math.log(far / half)
                    * (rows - half)))))
        return out


@dataclass
class FFSpec:
    kind: str                 # dense | moe | routed_moe
    ff: int                   # hidden size (of one expert for moe)
    experts: int = 0
    top: int = 0
    # routed_moe: softmax router with a selection-only correction, experts
    # in equal groups of neighbours of which the best ``group_keep`` stay
    # eligible, trailing identity experts, an always-on shared expert
    identity: int = 0
    group_count: int = 1
    group_keep: int = 1
    shared_ff: int = 0
    weight_eps: float = 1e-20
    # routed_moe: the router's scores are a softmax over the experts or each
    # logit's own sigmoid; a group's score is the sum of its best
    # ``group_top`` choice scores; the normalised weights are multiplied by
    # ``route_scale``; experts are W_down gelu(W_up h) ("gelu") or
    # W_down (silu(W_gate h) * W_up h) ("silu_gated")
    router_act: str = "softmax"
    group_top: int = 1
    route_scale: float = 1.0
    expert_act: str = "gelu"
    # dense: "silu" is silu(gate) * up; "clamped" is g * sigmoid(slope * g)
    # * (u + shift) with g = min(gate, limit), u = clamp(up, -limit, limit)
    act: str = "silu"
    limit: float = 0.0
    gate_slope: float = 1.702
    up_shift: float = 1.0
    bias: bool = False        # gate / up / down projections carry biases


@dataclass
class BigramSpec:
    """Hashed pair embedding: row (prev * mul_prev + cur * mul_cur) mod
    buckets of a (buckets + 1)-row table; a sequence's first token reads
    the last row."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class HybridLayerSpec:
    mixer: object
    ff: Optional[FFSpec]


@dataclass
class HybridConfig:
    arch: str = "bizusun"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[HybridLayerSpec] = field(default_factory=list)
    norm_eps: float = 1e-6
    canon_taps: int = 4
    token_side_dim: int = 0
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 20   # no learned positions: a fence
    # "canon": norm -> convolution -> mixer, norm -> ff, token-side input
    # (scalar norm weights).  "sandwich": x += norm(mixer(norm(x))),
    # x += norm(ff(norm(x))) with per-channel weights stored as offsets
    # from ``norm_offset``.  "prenorm": x += m * mixer(norm(x)),
    # x += m * ff(norm(x)), x += m * token-side input, with per-channel
    # weights and m = ``residual_mult``.  "parallel": both sublayers read
    # the same stream, x += mixer(norm1(x)) + ff(norm2(x)).
    layer_style: str = "canon"
    # "rms": x / sqrt(mean(x^2) + eps) * w.  "layer": (x - mean) /
    # sqrt(var + eps) * w (no bias); parallel layers only.
    norm_kind: str = "rms"
    # every sublayer's result is multiplied by sigmoid(W h + b) of the
    # sublayer's own input h (tensors 'rg1', 'rg1.b', 'rg2', 'rg2.b')
    gated_residual: bool = False
    norm_offset: float = 0.0
    residual_mult: float = 1.0
    # the embedding: table row * embed_scale [+ hashed pair row]
    # [+ sinusoid of the position p: angles p * base^(-2i/width), sines at
    # the even entries, cosines at the odd ones; 0 = none]
    embed_scale: float = 1.0
    bigram: Optional[BigramSpec] = None
    sin_pos_base: float = 0.0
    # layers [start, stop) run ``times`` times in a row with the same
    # weights; every pass owns its cache rows and state
    loop: Optional[tuple] = None
    # before every pass after the first the embedding output is added to
    # the stream again (``loop_reinject``); before every pass a learned
    # vector of that pass is added (``loop_step``, tensor 'loop.step')
    loop_reinject: bool = False
    loop_step: bool = False

    # the engine's generic accessors
    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def is_hybrid(self) -> bool:
        return True

    def run_order(self) -> List[int]:
        """Layer index of every layer run, in execution order.  Caches and
        states are keyed by the run's place in this list."""
        n = len(self.layers)
        if not self.loop or self.loop[2] <= 1:
            return list(range(n))
        a, b, t = self.loop
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    def pass_starts(self) -> dict:
        """Run index -> pass number for the first run of every pass of the
        looped span (empty without a loop)."""
        if not self.loop:
            return {}
        a, b, t = self.loop
        if b <= a:
            return {}
        return {a + r * (b - a): r for r in range(t)}

    def cache_owner(self, li: int) -> Optional[int]:
        """Layer whose latent cache layer ``li`` reads (itself unless it
        shares), or None for a layer without a paged cache."""
        m = self.layers[li].mixer
        if m.kind != "latent_attention":
            return None
        return li if m.kv_from is None else m.kv_from

    def validate(self):
        for li, L in enumerate(self.layers):
            m = L.mixer
            if m.kind == "latent_attention" and m.kv_from is not None:
                src = self.layers[m.kv_from].mixer
                if not (0 <= m.kv_from < li) or \
                        src.kind != "latent_attention" or \
                        src.kv_from is not None:
                    raise ValueError(f"layer {li}: kv_from must name an "
                                     "earlier layer that owns its cache")
                if (src.kv_rank, src.rot_dim) != (m.kv_rank, m.rot_dim):
                    raise ValueError(f"layer {li}: a shared cache needs "
                                     "equal latent and rotated sizes")
            if m.kind == "gla":
                assert m.heads > 0 and m.dim > 0 and m.vdim > 0 and m.tau > 0
            if m.kind == "rglru":
                assert m.width % m.blocks == 0 and m.conv >= 1
            if m.kind == "latent_attention":
                assert m.gate in ("element", "head")
                if m.rope is not None:
                    assert m.rope.dims % 2 == 0 and m.rope.dims <= m.rot_dim
            if m.kind == "mamba2":
                assert m.heads % m.groups == 0
                assert m.inner % m.norm_groups == 0
            if m.kind == "attention":
                assert m.heads % m.kv_heads == 0 and m.window >= 1
                if m.rope is not None:
                    assert m.rope.dims % 2 == 0 and m.rope.dims <= m.dim
                    if m.rope.interleaved:
                        raise ValueError(f"layer {li}: grouped-query "
                                         "attention rotates halves")
                assert m.weights in ("softmax", "sigmoid")
                if m.weights == "sigmoid" and (m.sink or m.bias_far > 0):
                    raise ValueError(f"layer {li}: a sink or a distance "
                                     "bias needs softmax weights")
                if m.value_rope_base > 0:
                    assert m.vdim % 2 == 0 and not m.values_from_keys
                if m.bias_far > 0 and m.keep_first > 0:
                    raise ValueError(f"layer {li}: the distance bias covers "
                                     "the window only (no kept first tokens)")
            if L.ff is not None and L.ff.kind == "dense":
                assert L.ff.act in ("silu", "clamped")
                assert L.ff.act == "silu" or L.ff.limit > 0
            if L.ff is not None and L.ff.kind == "moe":
                assert 0 < L.ff.top <= L.ff.experts
            if L.ff is not None and L.ff.kind == "routed_moe":
                f = L.ff
                total = f.experts + f.identity
                assert total % f.group_count == 0
                assert 0 < f.group_keep <= f.group_count
                assert 0 < f.top <= f.group_keep * (total // f.group_count)
                assert f.router_act in ("softmax", "sigmoid")
                assert f.expert_act in ("gelu", "silu_gated")
                assert f.group_top >= 1
        assert self.norm_kind == "rms" or self.layer_style == "parallel"
        assert not self.gated_residual or self.layer_style == "parallel"
        if (self.loop_reinject or self.loop_step) and not self.loop:
            raise ValueError("pass inputs need a looped span")
        if self.loop is not None:
            a, b, t = self.loop
            assert 0 <= a <= b <= len(self.layers) and t >= 1
            if any(getattr(L.mixer, "kv_from", None) is not None
                   for L in self.layers):
                raise ValueError("shared caches and looped layers do not "
                                 "combine")
        return self


def _mixer_from_json(kind: str, m: dict):
    if kind == "general_delta":
        return DeltaRuleSpec(heads=int(m["heads"]), dim=int(m["dim"]))
    if kind == "mamba2":
        return SSMSpec(heads=int(m["heads"]), vdim=int(m["vdim"]),
                       state=int(m["state"]), groups=int(m.get("groups", 1)),
                       norm_groups=int(m.get("norm_groups", 1)),
                       conv=int(m["conv"]))
    if kind == "latent_attention":
        rot = m.get("rot", {})
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]),
            rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), window=int(m["mask"]["size"]),
            scale=float(m["scale"]),
            rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", m["rot_dim"])),
            kv_from=(None if m.get("kv_from") is None
                     else int(m["kv_from"])))
    raise ValueError(f"unknown mixer type {kind!r}")


def _ff_from_json(f: Optional[dict]) -> Optional[FFSpec]:
    if f is None:
        return None
    if f["kind"] == "dense":
        return FFSpec(kind="dense", ff=int(f["ff"]))
    if f["kind"] == "moe":
        return FFSpec(kind="moe", ff=int(f["expert"]["ff"]),
                      experts=int(f["router"]["experts"]),
                      top=int(f["router"]["top"]))
    raise ValueError(f"unknown feed-forward kind {f['kind']!r}")


def bizusun_config_from_json(d: dict) -> HybridConfig:
    """Read a Bizusun ``config.json`` (already parsed)."""
    layers = [HybridLayerSpec(_mixer_from_json(L["type"], L["mixer"]),
                              _ff_from_json(L.get("mlp")))
              for L in d["layers"]]
    return HybridConfig(
        arch="bizusun", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), layers=layers,
        norm_eps=float(d["norm"]["eps"]),
        canon_taps=int(d["canon"]["taps"]),
        token_side_dim=int(d["token_side"]["dim"]),
        logit_scale=float(d.get("logit_scale", 1.0))).validate()


def bizusun_config_to_json(cfg: HybridConfig) -> dict:
    """Inverse of :func:`bizusun_config_from_json` (checkpoint export)."""
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.kind == "general_delta":
            mj = {"heads": m.heads, "dim": m.dim}
        elif m.kind == "mamba2":
            mj = {"heads": m.heads, "vdim": m.vdim, "state": m.state,
                  "groups": m.groups, "norm_groups": m.norm_groups,
                  "conv": m.conv}
        else:
            mj = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank,
                  "mask": {"size": m.window}, "scale": m.scale,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims}}
            if m.kv_from is not None:
                mj["kv_from"] = m.kv_from
        if L.ff is None:
            fj = None
        elif L.ff.kind == "dense":
            fj = {"kind": "dense", "ff": L.ff.ff}
        else:
            fj = {"kind": "moe", "expert": {"ff": L.ff.ff},
                  "router": {"experts": L.ff.experts, "top": L.ff.top}}
        layers.append({"type": m.kind, "mixer": mj, "mlp": fj})
    return {"architecture": "Bizusun", "vocab": cfg.vocab_size,
            "width": cfg.hidden_size, "layers": layers,
            "norm": {"eps": cfg.norm_eps},
            "canon": {"taps": cfg.canon_taps},
            "token_side": {"dim": cfg.token_side_dim},
            "logit_scale": cfg.logit_scale}


def bizusun_preset(width: int, layers: int, vocab: int = 32000,
                   heads: int = 16, ff_mult: float = 2.5, experts: int = 16,
                   top: int = 2, window: int = 1024,
                   pattern=("general_delta", "mamba2", "latent_attention",
                            "latent_attention")) -> HybridConfig:
    """A Bizusun stack of realistic layer sizes (random weights): the mixer
    kinds cycle through ``pattern``; the second latent-attention layer of
    each cycle shares the first one's cache; the first layer is dense, the
    rest use table-routed experts of equal total active width."""
    hd = width // heads
    out: List[HybridLayerSpec] = []
    last_owner = None
    for li in range(layers):
        kind = pattern[li % len(pattern)]
        if kind == "general_delta":
            mixer = DeltaRuleSpec(heads=heads, dim=hd)
            last_owner = None
        elif kind == "mamba2":
            mixer = SSMSpec(heads=2 * heads, vdim=hd, state=128,
                            groups=max(1, heads // 8), norm_groups=1, conv=4)
            last_owner = None
        else:
            mixer = LatentAttnSpec(
                heads=heads, dim=hd, rot_dim=hd // 2, vdim=hd,
                kv_rank=4 * hd, window=window,
                scale=1.0 / math.sqrt(hd + hd // 2), kv_from=last_owner)
            if last_owner is None:
                last_owner = li
        dense_ff = int(width * ff_mult) // 64 * 64
        ff = FFSpec("dense", dense_ff) if li == 0 else \
            FFSpec("moe", max(64, dense_ff // top // 64 * 64), experts, top)
        out.append(HybridLayerSpec(mixer, ff))
    return HybridConfig(arch="bizusun", vocab_size=vocab, hidden_size=width,
                        layers=out, norm_eps=1e-6, canon_taps=4,
                        token_side_dim=max(8, width // 16),
                        logit_scale=1.0).validate()


def _window_attn_from_json(kind: str, m: dict) -> WindowAttnSpec:
    """Kuforax mixers: 'attention' (rotary, kept first tokens, whole-row
    query/key norms, values = raw keys, per-head gate) and 'attention_2'
    (distance-bucket bias, separate values, no rotation)."""
    mask = m["mask"]
    common = dict(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                  dim=int(m["dim"]), vdim=int(m["vdim"]),
                  window=int(mask["size"]), scale=float(m["scale"]))
    if kind == "attention":
        rot = m.get("rot")
        rope = None
        if rot and int(rot.get("dims", 0)) > 0:
            sc = rot.get("scaling") or {}
            rope = RopeSpec(dims=int(rot["dims"]), base=float(rot["base"]),
                            factor=float(sc.get("factor", 1.0)),
                            original=float(sc.get("original", 0.0)),
                            fast=float(sc.get("fast", 32.0)),
                            slow=float(sc.get("slow", 1.0)))
        if common["vdim"] != common["dim"]:
            raise ValueError("values taken from keys need vdim == dim")
        return WindowAttnSpec(**common, rope=rope,
                              keep_first=int(mask.get("keep_first", 0)),
                              qk_norm=True, values_from_keys=True,
                              head_gate=True)
    return WindowAttnSpec(**common, bias_far=float(m["bias_max"]))


def _routed_ff_from_json(f: Optional[dict]) -> Optional[FFSpec]:
    if f is None:
        return None
    if f["kind"] != "moe":
        raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
    r = f["router"]
    g = r.get("groups") or {}
    shared = f.get("shared") or {}
    return FFSpec(kind="routed_moe", ff=int(f["expert"]["ff"]),
                  experts=int(r["experts"]), top=int(r["top"]),
                  identity=int(r.get("identity", 0)),
                  group_count=int(g.get("count", 1)),
                  group_keep=int(g.get("keep", 1)),
                  shared_ff=int(shared.get("ff", 0)))


def kuforax_config_from_json(d: dict) -> HybridConfig:
    """Read a Kuforax ``config.json`` (already parsed)."""
    layers = []
    for L in d["layers"]:
        if L["type"] not in ("attention", "attention_2"):
            raise ValueError(f"unknown mixer type {L['type']!r}")
        layers.append(HybridLayerSpec(
            _window_attn_from_json(L["type"], L["mixer"]),
            _routed_ff_from_json(L.get("mlp"))))
    loop = d.get("loop")
    return HybridConfig(
        arch="kuforax", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), layers=layers,
        norm_eps=float(d["norm"]["eps"]), canon_taps=1, token_side_dim=0,
        layer_style="sandwich", norm_offset=1.0,
        loop=None if not loop else (int(loop["start"]), int(loop["stop"]),
                                    int(loop["times"]))).validate()


def kuforax_config_to_json(cfg: HybridConfig) -> dict:
    """Inverse of :func:`kuforax_config_from_json` (checkpoint export)."""
    layers = []
    for L in cfg.layers:
        m = L.mixer
        mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
              "vdim": m.vdim, "scale": m.scale, "mask": {"size": m.window}}
        if m.bias_far > 0:
            kind = "attention_2"
            mj["bias_max"] = m.bias_far
        else:
            kind = "attention"
            mj["mask"]["keep_first"] = m.keep_first
            if m.rope is not None:
                r = m.rope
                mj["rot"] = {"base": r.base, "dims": r.dims}
                if r.factor != 1.0:
                    mj["rot"]["scaling"] = {
                        "factor": r.factor, "original": r.original,
                        "fast": r.fast, "slow": r.slow}
        fj = None
        if L.ff is not None:
            f = L.ff
            fj = {"kind": "moe", "expert": {"ff": f.ff},
                  "router": {"experts": f.experts, "top": f.top,
                             "identity": f.identity,
                             "groups": {"count": f.group_count,
                                        "keep": f.group_keep}}}
            if f.shared_ff:
                fj["shared"] = {"ff": f.shared_ff}
        layers.append({"type": kind, "mixer": mj, "mlp": fj})
    out = {"architecture": "Kuforax", "vocab": cfg.vocab_size,
           "width": cfg.hidden_size, "layers": layers,
           "norm": {"eps": cfg.norm_eps}}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop[0], "stop": cfg.loop[1],
                       "times": cfg.loop[2]}
    return out


def kuforax_preset(width: int, layers: int, vocab: int = 32000,
                   heads: int = 16, kv_heads: int = 4, experts: int = 16,
                   top: int = 2, identity: int = 2, expert_ff: int = 0,
                   shared_ff: int = 0, window: int = 1024,
                   keep_first: int = 4, bias_every: int = 4,
                   loop: Optional[tuple] = None) -> HybridConfig:
    """A Kuforax stack of realistic layer sizes (random weights): every
    ``bias_every``-th layer uses the distance-bias attention, the others
    the rotary one; routed experts with a shared expert in every layer."""
    hd = width // heads
    expert_ff = expert_ff or max(64, width // 64 * 64)
    shared_ff = shared_ff or expert_ff
    total = experts + identity
    groups = 2 if total % 2 == 0 and total // 2 >= top else 1
    out = []
    for li in range(layers):
        if bias_every and li % bias_every == bias_every - 1:
            mixer = WindowAttnSpec(heads=heads, kv_heads=kv_heads, dim=hd,
                                   vdim=hd, window=window,
                                   scale=1.0 / math.sqrt(hd),
                                   bias_far=float(window), bias_rows=32)
        else:
            mixer = WindowAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=hd, vdim=hd,
                window=window, scale=1.0 / math.sqrt(hd),
                keep_first=keep_first,
                rope=RopeSpec(dims=hd // 2, base=10000.0, factor=4.0,
                              original=4096.0),
                qk_norm=True, values_from_keys=True, head_gate=True)
        ff = FFSpec("routed_moe", expert_ff, experts, top, identity=identity,
                    group_count=groups, group_keep=1 if groups > 1 else 1,
                    shared_ff=shared_ff)
        out.append(HybridLayerSpec(mixer, ff))
    return HybridConfig(arch="kuforax", vocab_size=vocab, hidden_size=width,
                        layers=out, norm_eps=1e-5, canon_taps=1,
                        token_side_dim=0, layer_style="sandwich",
                        norm_offset=1.0, loop=loop).validate()


def _vurivik_mixer_from_json(kind: str, m: dict):
    """Vurivik mixers: 'gla' (gated linear attention) and 'attention'
    (causal grouped-query attention with projection biases, a softmax sink
    and a position-dependent query temperature; no rotation)."""
    if kind == "gla":
        return GLASpec(heads=int(m["heads"]), dim=int(m["dim"]),
                       vdim=int(m["vdim"]), tau=float(m["tau"]))
    if kind == "attention":
        qt = m.get("q_temp") or {}
        return WindowAttnSpec(
            heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]), vdim=int(m["vdim"]), window=UNBOUNDED,
            scale=float(m["scale"]), qkv_bias=True, sink=True,
            q_temp_coef=float(qt.get("coef", 0.0)),
            q_temp_every=int(qt.get("every", 1)))
    raise ValueError(f"unknown mixer type {kind!r}")


def _clamped_ff_from_json(f: Optional[dict]) -> Optional[FFSpec]:
    if f is None:
        return None
    if f["kind"] != "dense":
        raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
    return FFSpec(kind="dense", ff=int(f["ff"]), act="clamped",
                  limit=float(f["limit"]), bias=True)


def vurivik_config_from_json(d: dict) -> HybridConfig:
    """Read a Vurivik ``config.json`` (already parsed)."""
    layers = [HybridLayerSpec(_vurivik_mixer_from_json(L["type"], L["mixer"]),
                              _clamped_ff_from_json(L.get("mlp")))
              for L in d["layers"]]
    emb = d.get("embedding") or {}
    bg = emb.get("bigram")
    loop = d.get("loop")
    return HybridConfig(
        arch="vurivik", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), layers=layers,
        norm_eps=float(d["norm"]["eps"]), canon_taps=1,
        token_side_dim=int((d.get("token_side") or {}).get("dim", 0)),
        layer_style="prenorm",
        residual_mult=float(d.get("residual_mult", 1.0)),
        embed_scale=float(emb.get("scale", 1.0)),
        bigram=None if not bg else BigramSpec(
            buckets=int(bg["buckets"]), mul_prev=int(bg["mul_prev"]),
            mul_cur=int(bg["mul_cur"])),
        sin_pos_base=10000.0,
        loop=None if not loop else (int(loop["start"]), int(loop["stop"]),
                                    int(loop["times"])),
        loop_reinject=bool(loop), loop_step=bool(loop)).validate()


def vurivik_config_to_json(cfg: HybridConfig) -> dict:
    """Inverse of :func:`vurivik_config_from_json` (checkpoint export)."""
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.kind == "gla":
            mj = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim,
                  "tau": m.tau}
        else:
            mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "scale": m.scale,
                  "q_temp": {"coef": m.q_temp_coef, "every": m.q_temp_every}}
        fj = None if L.ff is None else \
            {"kind": "dense", "ff": L.ff.ff, "limit": L.ff.limit}
        layers.append({"type": m.kind, "mixer": mj, "mlp": fj})
    emb = {"scale": cfg.embed_scale}
    if cfg.bigram is not None:
        emb["bigram"] = {"buckets": cfg.bigram.buckets,
                         "mul_prev": cfg.bigram.mul_prev,
                         "mul_cur": cfg.bigram.mul_cur}
    out = {"architecture": "Vurivik", "vocab": cfg.vocab_size,
           "width": cfg.hidden_size, "embedding": emb, "layers": layers,
           "norm": {"eps": cfg.norm_eps},
           "residual_mult": cfg.residual_mult,
           "token_side": {"dim": cfg.token_side_dim}}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop[0], "stop": cfg.loop[1],
                       "times": cfg.loop[2]}
    return out


def vurivik_preset(width: int, layers: int, vocab: int = 32000,
                   heads: int = 16, kv_heads: int = 4, ff_mult: float = 2.75,
                   gla_every: int = 3, gla_heads: int = 0,
                   loop: Optional[tuple] = None) -> HybridConfig:
    """A Vurivik stack of realistic layer sizes (random weights): every
    ``gla_every``-th layer is gated linear attention without a feed-forward,
    the others causal grouped-query attention with the clamped gated
    feed-forward."""
    hd = width // heads
    gh = gla_heads or max(1, heads // 2)
    out = []
    for li in range(layers):
        if gla_every and li % gla_every == gla_every - 1:
            out.append(HybridLayerSpec(
                GLASpec(heads=gh, dim=hd, vdim=2 * hd, tau=8.0,
                        decay_rank=16), None))
        else:
            out.append(HybridLayerSpec(
                WindowAttnSpec(heads=heads, kv_heads=kv_heads, dim=hd,
                               vdim=hd, window=UNBOUNDED,
                               scale=1.0 / math.sqrt(hd), qkv_bias=True,
                               sink=True, q_temp_coef=0.1, q_temp_every=1024),
                FFSpec(kind="dense", ff=int(width * ff_mult) // 64 * 64,
                       act="clamped", limit=7.0, bias=True)))
    return HybridConfig(
        arch="vurivik", vocab_size=vocab, hidden_size=width, layers=out,
        norm_eps=1e-5, canon_taps=1, token_side_dim=max(8, width // 16),
        layer_style="prenorm", residual_mult=0.6,
        embed_scale=8.0,
        bigram=BigramSpec(buckets=65521, mul_prev=257, mul_cur=13),
        sin_pos_base=10000.0, loop=loop, loop_reinject=bool(loop),
        loop_step=bool(loop)).validate()


def _rope_from_json(rot: Optional[dict], interleaved: bool = False
                    ) -> Optional[RopeSpec]:
    if not rot or int(rot.get("dims", 0)) <= 0:
        return None
    sc = rot.get("scaling") or {}
    return RopeSpec(dims=int(rot["dims"]), base=float(rot["base"]),
                    factor=float(sc.get("factor", 1.0)),
                    original=float(sc.get("original", 0.0)),
                    fast=float(sc.get("fast", 32.0)),
                    slow=float(sc.get("slow", 1.0)),
                    interleaved=interleaved)


def _nasipel_mixer_from_json(kind: str, m: dict):
    """Nasipel mixers: 'attention' (grouped-query, rotate-half rotation,
    unit q/k heads, capped scores, sigmoid weights with a per-head bias,
    rotated values), 'rglru' (gated linear recurrence) and
    'latent_attention' (causal, query latent, interleaved YaRN rotation,
    per-head output gate, no sink)."""
    if kind == "rglru":
        return RGLRUSpec(width=int(m["width"]), blocks=int(m["blocks"]),
                         conv=int(m["conv"]))
    if kind == "attention":
        rot = m.get("rot") or {}
        return WindowAttnSpec(
            heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]), vdim=int(m["vdim"]), window=UNBOUNDED,
            scale=float(m["scale"]), rope=_rope_from_json(rot),
            head_unit_norm=True, softcap=float(m.get("softcap") or 0.0),
            head_bias=True, weights="sigmoid",
            value_rope_base=float(rot.get("base", 10000.0)))
    if kind == "latent_attention":
        rope = _rope_from_json(m.get("rot"), interleaved=True)
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]),
            rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), window=UNBOUNDED,
            scale=float(m["scale"]), q_rank=int(m["q_rank"]), sink=False,
            gate="head", rope=rope)
    raise ValueError(f"unknown mixer type {kind!r}")


def _sigmoid_routed_ff_from_json(f: Optional[dict]) -> Optional[FFSpec]:
    if f is None:
        return None
    if f["kind"] != "moe":
        raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
    r = f["router"]
    g = r.get("groups") or {}
    return FFSpec(kind="routed_moe", ff=int(f["expert"]["ff"]),
                  experts=int(r["experts"]), top=int(r["top"]),
                  group_count=int(g.get("count", 1)),
                  group_keep=int(g.get("keep", 1)),
                  router_act="sigmoid", group_top=2,
                  route_scale=float(r.get("scale", 1.0)),
                  expert_act="silu_gated")


def nasipel_config_from_json(d: dict) -> HybridConfig:
    """Read a Nasipel ``config.json`` (already parsed)."""
    layers = [HybridLayerSpec(_nasipel_mixer_from_json(L["type"], L["mixer"]),
                              _sigmoid_routed_ff_from_json(L.get("mlp")))
              for L in d["layers"]]
    return HybridConfig(
        arch="nasipel", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), layers=layers,
        norm_eps=float(d["norm"]["eps"]), canon_taps=1, token_side_dim=0,
        layer_style="parallel", norm_kind="layer",
        gated_residual=True).validate()


def nasipel_config_to_json(cfg: HybridConfig) -> dict:
    """Inverse of :func:`nasipel_config_from_json` (checkpoint export)."""
    def rot_json(r):
        out = {"base": r.base, "dims": r.dims}
        if r.factor != 1.0:
            out["scaling"] = {"factor": r.factor, "original": r.original,
                              "fast": r.fast, "slow": r.slow}
        return out
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.kind == "rglru":
            mj = {"width": m.width, "blocks": m.blocks, "conv": m.conv}
        elif m.kind == "attention":
            mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "scale": m.scale, "softcap": m.softcap,
                  "rot": rot_json(m.rope) if m.rope is not None else
                  {"base": m.value_rope_base, "dims": 0}}
        else:
            mj = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank, "q_rank": m.q_rank,
                  "scale": m.scale, "rot": rot_json(m.rope)}
        fj = None
        if L.ff is not None:
            f = L.ff
            fj = {"kind": "moe", "expert": {"ff": f.ff},
                  "router": {"experts": f.experts, "top": f.top,
                             "scale": f.route_scale,
                             "groups": {"count": f.group_count,
                                        "keep": f.group_keep}}}
        layers.append({"type": m.kind, "mixer": mj, "mlp": fj})
    return {"architecture": "Nasipel", "vocab": cfg.vocab_size,
            "width": cfg.hidden_size, "layers": layers,
            "norm": {"eps": cfg.norm_eps}}


def nasipel_preset(width: int, layers: int, vocab: int = 32000,
                   heads: int = 16, kv_heads: int = 4, experts: int = 16,
                   top: int = 2, expert_ff: int = 0,
                   pattern=("rglru", "rglru", "latent_attention",
                            "attention")) -> HybridConfig:
    """A Nasipel stack of realistic layer sizes (random weights): the mixer
    kinds cycle through ``pattern``; every layer has sigmoid-routed gated
    experts in two groups of which one stays open."""
    hd = width // heads
    expert_ff = expert_ff or max(64, width // 64 * 64)
    groups = 2 if experts % 2 == 0 and experts // 2 >= top else 1
    out = []
    for li in range(layers):
        kind = pattern[li % len(pattern)]
        if kind == "rglru":
            mixer = RGLRUSpec(width=width, blocks=heads, conv=4)
        elif kind == "attention":
            mixer = WindowAttnSpec(
                heads=heads, kv_heads=kv_heads, dim=hd, vdim=hd,
                window=UNBOUNDED, scale=1.0 / math.sqrt(hd),
                rope=RopeSpec(dims=hd, base=10000.0), head_unit_norm=True,
                softcap=50.0, head_bias=True, weights="sigmoid",
                value_rope_base=10000.0)
        else:
            mixer = LatentAttnSpec(
                heads=heads, dim=hd, rot_dim=hd // 2, vdim=hd,
                kv_rank=4 * hd, window=UNBOUNDED,
                scale=1.0 / math.sqrt(hd + hd // 2), q_rank=6 * hd,
                sink=False, gate="head",
                rope=RopeSpec(dims=hd // 2, base=10000.0, factor=8.0,
                              original=4096.0, interleaved=True))
        ff = FFSpec("routed_moe", expert_ff, experts, top,
                    group_count=groups, group_keep=1, router_act="sigmoid",
                    group_top=2, route_scale=2.5, expert_act="silu_gated")
        out.append(HybridLayerSpec(mixer, ff))
    return HybridConfig(arch="nasipel", vocab_size=vocab, hidden_size=width,
                        layers=out, norm_eps=1e-5, canon_taps=1,
                        token_side_dim=0, layer_style="parallel",
                        norm_kind="layer", gated_residual=True).validate()


def read_config_dir(path: str):
    """Model config from a checkpoint folder's ``config.json``.  The
    ``architecture`` key names the family; HF-style folders
    (``model_type``) map onto the dense decoder config."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch == "Bizusun":
        return bizusun_config_from_json(d)
    if arch == "Kuforax":
        return kuforax_config_from_json(d)
    if arch == "Vurivik":
        return vurivik_config_from_json(d)
    if arch == "Nasipel":
        return nasipel_config_from_json(d)
    mt = d.get("model_type")
    if mt in ("llama", "qwen2"):
        from .registry import DecoderConfig
        return DecoderConfig(
            arch=mt, vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
            intermediate_size=d["intermediate_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=d["num_attention_heads"],
            num_key_value_heads=d.get("num_key_value_heads",
                                      d["num_attention_heads"]),
            head_dim=d.get("head_dim"),
            max_position_embeddings=d.get("max_position_embeddings", 8192),
            rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            rope_theta=d.get("rope_theta", 10000.0),
            tie_word_embeddings=d.get("tie_word_embeddings", False),
            attention_bias=d.get("attention_bias", mt == "qwen2"))
    raise ValueError(f"{path}: unknown architecture "
                     f"{arch or mt!r} in config.json")
