"""The Vurivik family in the rollout engine against the plain oracle
(tests/vurivik_oracle.py): each mixer, the feed-forward, the composed
embedding and the looped passes alone, whole prompts against token-by-token
decoding, portions down to two tokens, unequal batches, reuse of pages and
slots, keys far behind and at page borders, the steps of the query
temperature, the sink, a long-lived recurrent state, first tokens, long
decoding, odd sizes, the checkpoint-folder loader, the trace replay entry
point and greedy generation through the engine's scheduler.

Every case runs on the CPU tier (PyTorch forms of the ops, fp32) and, marked
``gpu``, on the HIP kernels in fp32 and bf16.  Configurations are small and
made here; weights are random with a fixed seed (bf16-representable), or
built so that one key, one table row or one state is loud where random
weights would hide a fault.
"""
import copy
import io
import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import vurivik_oracle as O  # noqa: E402

from polyrl_amd.models.hybrid import (vurivik_config_from_json,  # noqa: E402
                                      vurivik_config_to_json)
from polyrl_amd.rollout.engine import Engine, SamplingParams  # noqa: E402
from polyrl_amd.rollout.hybrid_model import HybridInferenceModel  # noqa: E402

CPU = ("cpu", torch.float32)
GPU32 = pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu)
GPU16 = pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)
TARGETS = [CPU, GPU32, GPU16]
VOCAB = 83


def attn(heads=4, kv=2, dim=16, vdim=24, scale=0.3, coef=0.4, every=7):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
         "scale": scale}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def gla(heads=2, dim=12, vdim=20, tau=3.0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim,
                                     "vdim": vdim, "tau": tau}}


def ff(size=40, limit=1.5):
    return {"kind": "dense", "ff": size, "limit": limit}


def config(layers, width=48, loop=None, side=5, mult=0.7, scale=3.0,
           bigram=(61, 13, 5)):
    c = {"architecture": "Vurivik", "vocab": VOCAB, "width": width,
         "embedding": {"scale": scale},
         "layers": [dict(copy.deepcopy(m), mlp=copy.deepcopy(f))
                    for m, f in layers],
         "norm": {"eps": 1e-5}, "residual_mult": mult,
         "token_side": {"dim": side}}
    if bigram:
        c["embedding"]["bigram"] = dict(zip(
            ("buckets", "mul_prev", "mul_cur"), bigram))
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


FULL = config([(attn(), ff()), (gla(), None), (attn(kv=4, dim=24, vdim=8),
                                               ff(size=24, limit=0.8)),
               (gla(heads=3, dim=8, vdim=8, tau=1.0), ff(size=16))],
              loop=(1, 3, 2))


def engine(cfg, W, target, tokens=512, slots=4, page=4, **kw):
    dev, dt = target
    c = vurivik_config_from_json(cfg)
    HybridInferenceModel.resolve_shapes(
        c, {k: tuple(v.shape) for k, v in W.items()})
    e = Engine(c, device=dev, dtype=dt, page_size=page,
               kv_token_capacity=tokens, max_running_requests=slots,
               max_num_batched_tokens=kw.pop("budget", 1 << 20), **kw)
    e.model.load_state_dict(W)
    return e


def close(got, want, target, what=""):
    """Logit rows agree: error (mean removed, RMS over the vocabulary) over
    the oracle's own spread, every row."""
    got, want = got.double().cpu(), want.double()
    assert got.shape == want.shape, f"{what}: {got.shape} vs {want.shape}"
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)
    if target[1] == torch.float32:
        assert float(err.max()) < 3e-4, f"{what}: {float(err.max()):.3g}"
        return
    assert float(err.max()) < 0.12, f"{what}: worst {float(err.max()):.3g}"
    assert float(err.median()) < 0.04, f"{what}: median {float(err.median()):.3g}"


def toks(n, seed=0, avoid=()):
    g = torch.Generator().manual_seed(seed)
    t = torch.randint(0, VOCAB, (n,), generator=g).tolist()
    return [x if x not in avoid else (x + 7) % VOCAB for x in t]


def logits_of(cfg, W, t):
    return O.forward(cfg, W, t)[0]


def run(e, rid, t, want=None, end=True):
    want = list(range(len(t))) if want is None else want
    return e.step_forced([(rid, t, want)], [rid] if end else [])


def decode_after(e, rid, t, cut):
    rows = [e.step_forced([(rid, t[:cut], list(range(cut)))], [])]
    rows += [e.step_forced([(rid, [x], [0])], []) for x in t[cut:]]
    e.step_forced([], [rid])
    return torch.cat(rows)


def in_portions(e, rid, t, sizes):
    rows, at, i = [], 0, 0
    while at < len(t):
        n = min(sizes[i % len(sizes)], len(t) - at)
        rows.append(e.step_forced([(rid, t[at:at + n], list(range(n)))], []))
        at += n
        i += 1
    e.step_forced([], [rid])
    return torch.cat(rows)


# ------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name,layers,kw", [
    ("attention", [(attn(), None)], {}),
    ("attention-one-kv-head", [(attn(kv=1), None)], {}),
    ("attention-mha-one-head", [(attn(heads=1, kv=1, dim=32, vdim=32), None)],
     {}),
    ("attention-no-temperature", [(attn(coef=None, kv=4), None)], {}),
    ("attention-temperature-every-token", [(attn(every=1, coef=0.2), None)],
     {}),
    ("attention-odd-head-sizes", [(attn(dim=20, vdim=12), None)], {}),
    ("attention-head-136", [(attn(heads=2, kv=1, dim=136, vdim=8), None)],
     {}),
    ("gla", [(gla(), None)], {}),
    ("gla-one-head-square", [(gla(heads=1, dim=16, vdim=16, tau=16.0), None)],
     {}),
    ("gla-odd-sizes-tau-1", [(gla(heads=3, dim=5, vdim=3, tau=1.0), None)],
     {}),
    ("gla-wide", [(gla(heads=1, dim=40, vdim=70, tau=2.0), None)], {}),
    ("feed-forward-tight-limit", [(attn(), ff(limit=0.3))], {}),
    ("feed-forward-loose-limit", [(gla(), ff(limit=50.0))], {}),
    ("no-token-side", [(attn(), ff()), (gla(), None)], {"side": 0}),
    ("no-pair-table", [(gla(), ff()), (attn(), None)], {"bigram": None}),
    ("unit-multiplier-unit-scale", [(attn(), ff()), (gla(), None)],
     {"mult": 1.0, "scale": 1.0}),
    ("odd-width", [(attn(), ff(size=27)), (gla(), None)], {"width": 37}),
    ("loop-whole-stack", [(attn(), ff()), (gla(), None)],
     {"loop": (0, 2, 3)}),
    ("loop-once", [(gla(), None), (attn(), ff())], {"loop": (1, 2, 1)}),
    ("loop-at-the-end", [(attn(), None), (gla(), ff()), (attn(), None)],
     {"loop": (1, 3, 2)}),
    ("no-loop", [(gla(), ff()), (attn(), ff())], {}),
])
def test_mechanism_alone(target, name, layers, kw):
    cfg = config(layers, **kw)
    W = O.make_weights(cfg, seed=3, rank=4 if "odd" in name else 6)
    t = toks(29, seed=1)
    close(run(engine(cfg, W, target), "a", t), logits_of(cfg, W, t), target,
          name)


@pytest.mark.parametrize("target", TARGETS)
def test_residual_after_every_layer_run(target):
    W = O.make_weights(FULL, seed=7)
    t = toks(17, seed=2)
    e = engine(FULL, W, target)
    e.model.capture_layers = []
    run(e, "a", t)
    _, want = O.forward(FULL, W, t)
    assert len(e.model.capture_layers) == len(want) == 6
    for i, got in enumerate(e.model.capture_layers):
        d = (got.double().cpu() - want[i]).abs().max() / want[i].abs().max()
        lim = 2e-5 if target[1] == torch.float32 else 0.05
        assert float(d) < lim, f"layer run {i}: {float(d):.3g}"


# ---------------------------------------------- schedules give one answer
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_decode_and_portions_agree_with_oracle(target):
    W = O.make_weights(FULL, seed=11)
    t = toks(41, seed=3)
    want = logits_of(FULL, W, t)
    e = engine(FULL, W, target, page=4)
    close(run(e, "whole", t), want, target, "whole")
    close(decode_after(e, "dec", t, 1), want, target, "token by token")
    close(decode_after(e, "dec9", t, 9), want, target, "prefill 9 + decode")
    for sizes in ((2,), (3, 2, 7), (16, 5), (4,), (13, 1, 1, 2)):
        close(in_portions(e, f"p{sizes}", t, sizes), want, target,
              f"portions {sizes}")
    assert e.kv.free_pages == e.kv.num_pages
    assert e.states.free_slots == e.states.num_slots


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_batch_matches_each_alone(target):
    W = O.make_weights(FULL, seed=13)
    seqs = {"a": toks(33, seed=4), "b": toks(2, seed=5), "c": toks(19, seed=6),
            "d": toks(1, seed=7)}
    want = {k: logits_of(FULL, W, v) for k, v in seqs.items()}
    e = engine(FULL, W, target, page=4)
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    plan = [{"a": 5, "b": 2, "c": 1, "d": 1}, {"a": 1, "c": 9},
            {"c": 1, "a": 20}, {"a": 1, "c": 8}, {"a": 6}]
    for step in plan:
        entries, end = [], []
        for k, n in step.items():
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        out = e.step_forced(entries, end)
        o = 0
        for k, n in step.items():
            got[k].append(out[o:o + n])
            o += n
    for k in seqs:
        assert at[k] == len(seqs[k])
        close(torch.cat(got[k]), want[k], target, f"request {k}")


@pytest.mark.parametrize("target", TARGETS)
def test_pages_and_slots_are_reused_clean(target):
    """A pool of 6 pages and 2 slots serves a stream of requests: every page
    and slot is handed out again with another request's rows and states in
    it."""
    W = O.make_weights(FULL, seed=17)
    e = engine(FULL, W, target, tokens=24, slots=2, page=4)
    for i, n in enumerate((21, 7, 13, 24, 3, 10)):
        t = toks(n, seed=20 + i)
        got = decode_after(e, f"r{i}", t, max(1, n - 3)) if i % 2 else \
            run(e, f"r{i}", t)
        close(got, logits_of(FULL, W, t), target, f"request {i}")
        assert e.kv.free_pages == e.kv.num_pages
    a, b = toks(11, seed=40), toks(12, seed=41)
    e.step_forced([("a", a[:6], []), ("b", b[:2], [])], [])
    ga = e.step_forced([("a", a[6:], list(range(5)))], ["a"])
    c = toks(9, seed=42)                     # takes a's pages and slot
    gc = e.step_forced([("c", c, list(range(9))), ("b", b[2:], [])], ["c"])
    close(ga, logits_of(FULL, W, a)[6:], target, "a")
    close(gc[:9], logits_of(FULL, W, c), target, "c in a's pages and slot")


# --------------------------------------------- faults made visible on purpose
LOUD = 5


def _loud_key_model(layer, width=32):
    """One attention layer in which token LOUD's key is loud for every
    query: channel 0 of every embedding carries a constant, channel 1 is
    set for LOUD only; the last entry of every query head reads channel 0,
    the last entry of every key head reads channel 1.  Whoever sees LOUD
    attends to it.  No pair table and no token-side input, so a token acts
    through its own row only."""
    cfg = config([(layer, None)], width=width, side=0, bigram=None,
                 scale=1.0, mult=1.0)
    W = O.make_weights(cfg, seed=23)
    m = layer["mixer"]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    W["embed"][:, 0] = 3.0
    W["embed"][:, 1] = 0.0
    W["embed"][LOUD, 1] = 6.0
    W["l0.norm1"][:] = 1.0
    for name in ("q", "k"):
        W[f"l0.mix.{name}"][:, :2] = 0.0
        W[f"l0.mix.{name}.b"].zero_()
    for h in range(H):
        W["l0.mix.q"][h * D + D - 1] = 0.0
        W["l0.mix.q"][h * D + D - 1, 0] = 4.0
    for g in range(G):
        W["l0.mix.k"][g * D + D - 1] = 0.0
        W["l0.mix.k"][g * D + D - 1, 1] = 16.0
    m["scale"] = 1.0
    return cfg, W


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("where", [0, 3, 4, 63, 64, 65])
def test_far_key_is_seen_from_hundreds_of_tokens_away(target, where):
    """Causal attention has no window: a key at the start of the sequence,
    or on either side of a page or tile border, decides the logits 300
    tokens later, in a prompt, in decoding and across portion cuts."""
    cfg, W = _loud_key_model(attn(dim=16, vdim=16, coef=None))
    n = 330
    t = toks(n, seed=9, avoid=(LOUD,))
    t[where] = LOUD
    t2 = list(t)
    t2[where] = LOUD + 1
    want = logits_of(cfg, W, t)
    d = (want - logits_of(cfg, W, t2)).abs().max(-1).values
    assert float(d[-1]) > 0.05, "test model hides the far key"
    e = engine(cfg, W, target, page=4, tokens=1024)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, n - 40), want, target, "decoded")
    close(in_portions(e, "por", t, (97, 2, 64, 5)), want, target, "portions")


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("every", [1, 4, 9, 16])
def test_query_temperature_steps(target, every):
    """The temperature grows at positions every-1, 2*every-1, ...: with a
    large coefficient a step that is one position off moves the logits, in
    prompts, in decoding and at portion cuts on either side of a step."""
    cfg = config([(attn(coef=2.5, every=every, scale=0.6), None)])
    W = O.make_weights(cfg, seed=29)
    t = toks(3 * every + 6, seed=14)
    want = logits_of(cfg, W, t)
    off = copy.deepcopy(cfg)
    off["layers"][0]["mixer"]["q_temp"]["every"] = every + 1
    d = (want - logits_of(off, W, t)).abs().max(-1).values
    assert float(d[every - 1]) > 0.05, "test model hides the step"
    e = engine(cfg, W, target, page=4)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, max(1, every - 2)), want, target,
          "decoded")
    for cut in sorted({c for s in (every, 2 * every) for c in (s - 2, s - 1, s)}):
        if 0 < cut < len(t):
            rows = [e.step_forced([("p", t[:cut], list(range(cut)))], []),
                    e.step_forced([("p", t[cut:], list(range(len(t) - cut)))],
                                  ["p"])]
            close(torch.cat(rows), want, target, f"cut at {cut}")
    close(in_portions(e, "two", t, (2,)), want, target, "in twos")


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("sink", [6.0, -6.0])
def test_sink_counts_once_in_the_denominator(target, sink):
    """A large sink takes most of the weight away from the keys (also from
    a sequence's first token, which would otherwise attend to itself with
    weight one); a very negative one leaves plain softmax."""
    cfg = config([(attn(heads=4, kv=2), None)])
    W = O.make_weights(cfg, seed=31)
    W["l0.mix.sink"][:] = torch.tensor([sink, 0.0, -sink, sink / 2])
    t = toks(70, seed=15)
    want = logits_of(cfg, W, t)
    W2 = dict(W)
    W2["l0.mix.sink"] = torch.full((4,), -60.0)
    assert float((want - logits_of(cfg, W2, t)).abs().max()) > 0.05
    e = engine(cfg, W, target, page=4)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, 3), want, target, "decoded")
    close(in_portions(e, "por", t, (2, 33)), want, target, "portions")


@pytest.mark.parametrize("target", TARGETS)
def test_recurrent_state_lives_long_and_starts_at_zero(target):
    """Decays next to one: what the first tokens wrote into the state is
    still read 200 tokens later, so a state that is lost at a portion cut,
    in decoding or in a reused slot shows; a second layer decays fast."""
    cfg = config([(gla(heads=2, dim=8, vdim=8, tau=8.0), None),
                  (gla(heads=1, dim=12, vdim=4, tau=1.0), None)], width=32)
    W = O.make_weights(cfg, seed=37)
    W["l0.mix.a2"].zero_()
    W["l0.mix.a2.b"][:] = 9.0
    W["l1.mix.a2.b"] -= 3.0
    n = 220
    t = toks(n, seed=16)
    want = logits_of(cfg, W, t)
    t2 = toks(20, seed=99) + t[20:]          # other first tokens
    d = (want - logits_of(cfg, W, t2)).abs().max(-1).values
    assert float(d[-1]) > 0.05, "test model forgets its first tokens"
    e = engine(cfg, W, target, page=4, tokens=512, slots=1)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, n - 30), want, target, "decoded")
    close(in_portions(e, "por", t, (2, 61, 3, 128)), want, target, "portions")
    short = toks(3, seed=17)                 # the slot again, from zero
    close(run(e, "again", short), logits_of(cfg, W, short), target, "again")


@pytest.mark.parametrize("target", TARGETS)
def test_pair_table_rows_at_sequence_and_portion_starts(target):
    """The pair table is loud: the last row (a sequence's first token) and
    the row picked by the token before a portion's or a decoded token's
    first row decide the logits."""
    cfg = config([(gla(), ff())], bigram=(7, 3, 2), scale=0.5)
    W = O.make_weights(cfg, seed=41)
    W["bigram"] *= 6.0
    t = toks(23, seed=18)
    want = logits_of(cfg, W, t)
    W2 = dict(W)
    W2["bigram"] = W["bigram"].clone()
    W2["bigram"][-1] = W["bigram"][0]
    assert float((want[0] - logits_of(cfg, W2, t)[0]).abs().max()) > 0.05
    e = engine(cfg, W, target, page=4)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, 1), want, target, "token by token")
    close(in_portions(e, "por", t, (2, 1, 5)), want, target, "portions")


@pytest.mark.parametrize("target", TARGETS)
def test_pass_inputs_of_the_looped_span(target):
    """Loud pass vectors and a span looped three times: each pass adds its
    own vector, every pass after the first adds the embedding output."""
    cfg = config([(attn(), None), (gla(), ff()), (attn(kv=1), None)],
                 loop=(1, 3, 3))
    W = O.make_weights(cfg, seed=43)
    W["loop.step"] *= 8.0
    t = toks(21, seed=19)
    want = logits_of(cfg, W, t)
    e = engine(cfg, W, target, page=4)
    close(run(e, "whole", t), want, target, "prompt")
    close(decode_after(e, "dec", t, 2), want, target, "decoded")
    close(in_portions(e, "por", t, (2, 7)), want, target, "portions")


@pytest.mark.parametrize("target", TARGETS)
def test_first_tokens_and_long_decoding(target):
    W = O.make_weights(FULL, seed=31)
    e = engine(FULL, W, target)
    for n in (1, 2, 3, 4):
        t = toks(n, seed=50 + n)
        close(run(e, f"s{n}", t), logits_of(FULL, W, t), target, f"len {n}")
    t = toks(120, seed=55)
    close(decode_after(e, "long", t, 2), logits_of(FULL, W, t), target,
          "118 decoded tokens")


# ------------------------------------- loader, replay entry, generation
def _save(tmp_path, cfg, W):
    from safetensors.torch import save_file
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()},
              str(d / "model.safetensors"))
    return str(d)


def test_config_round_trip():
    c = vurivik_config_from_json(FULL)
    assert c.run_order() == [0, 1, 2, 1, 2, 3]
    assert c.pass_starts() == {1: 0, 3: 1}
    assert vurivik_config_to_json(c) == FULL
    assert vurivik_config_from_json(vurivik_config_to_json(c)) == c


@pytest.mark.parametrize("target", [CPU, GPU32])
def test_folder_loader_and_trace_replay(target, tmp_path, monkeypatch, capsys):
    from polyrl_amd.models import get_model_config
    from polyrl_amd.rollout import trace_replay
    W = O.make_weights(FULL, seed=37, rank=3)
    path = _save(tmp_path, FULL, W)
    c = get_model_config(path)
    assert c.arch == "vurivik" and c.num_hidden_layers == 4
    a, b = toks(13, seed=60), toks(6, seed=61)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [7]},
                                {"id": "b", "tokens": b, "want": [0, 5]}],
         "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": a[8:9], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[9:], "want": [3]}],
         "end": ["a"]},
    ]
    monkeypatch.setattr(sys, "stdin",
                        io.StringIO("\n".join(map(json.dumps, steps)) + "\n"))
    out = tmp_path / "out"
    rc = trace_replay.main(["--model", path, "--dtype", "float32", "--out",
                            str(out), "--max-tokens", "128", "--device",
                            target[0]])
    assert rc == 0
    assert capsys.readouterr().out.split() == ["done", "0", "done", "1",
                                               "done", "2"]
    import numpy as np
    wa, wb = logits_of(FULL, W, a), logits_of(FULL, W, b)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")
                          .reshape(3, -1))
    close(g0, torch.stack([wa[7], wb[0], wb[5]]), target, "step 0")
    assert not (out / "1.f32").exists()
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")
                          .reshape(1, -1))
    close(g2, wa[12:13], target, "step 2")


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(target):
    """Engine.generate: admission, chunked prompts (token budget of 8),
    mixed steps, sampling at temperature 0, the pair row of a sampled token
    (its predecessor is the last prompt or sampled token), pages and slots
    released."""
    if target[0] == "cuda":
        from polyrl_amd.ops import seq
        assert seq.seq_extension_loaded()
    W = O.make_weights(FULL, seed=41)
    W["bigram"] *= 3.0
    e = engine(FULL, W, target, slots=3, budget=8)
    prompts = [toks(n, seed=70 + n) for n in (11, 2, 17, 5)]
    outs = e.generate(prompts, SamplingParams(temperature=0.0,
                                              max_new_tokens=5), "g")
    for p, o in zip(prompts, outs):
        ids = list(p)
        for got_tok in o.output_ids:
            logits = logits_of(FULL, W, ids)[-1]
            top2 = logits.topk(2).values
            tie = 1e-3 if target[1] == torch.float32 else \
                0.25 * float(logits.std())
            if float(top2[0] - top2[1]) > tie:      # skip near ties
                assert got_tok == int(logits.argmax())
            ids.append(got_tok)
        assert len(o.output_ids) == 5 and o.finish_reason == "length"
    assert e.kv.free_pages == e.kv.num_pages
    assert e.states.free_slots == e.states.num_slots


def test_registry_preset_runs_and_resumes_memory():
    from polyrl_amd.models import get_model_config
    c = get_model_config("vurivik-debug")
    e = Engine(c, device="cpu", dtype=torch.float32, page_size=4,
               kv_token_capacity=64, max_running_requests=2)
    e.model.init_random(seed=1)
    t = toks(9, seed=90)
    a = run(e, "a", t)
    assert a.shape == (9, c.vocab_size) and torch.isfinite(a).all()
    e.release_memory()
    assert not e.kv.rows
    e.resume_memory()
    torch.testing.assert_close(run(e, "b", t), a)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_decode_graph_replays_match_eager_steps(dt):
    """Pure decode steps replay a captured graph once their batch size has
    recurred: 40 greedy tokens (eager sampling, copies and a host sync
    between the replays) equal the run with every launch issued eagerly,
    also after the batch shrinks to another size."""
    W = O.make_weights(FULL, seed=47)
    prompts = [toks(n, seed=80 + n) for n in (9, 3, 14)]
    new = (40, 17, 40)
    outs = {}
    for graphs in (False, True):
        e = engine(FULL, W, ("cuda", dt), slots=3)
        assert e.enable_hybrid_graphs
        e.enable_hybrid_graphs = graphs
        for i, (p, n) in enumerate(zip(prompts, new)):
            e.add_request(f"g-{i}", p, SamplingParams(temperature=0.0,
                                                      max_new_tokens=n))
        got = {}
        while e.has_work():
            for o in e.step():
                got[o.rid] = o
        outs[graphs] = [got[f"g-{i}"] for i in range(3)]
        assert sorted(e._graphs) == ([2, 3] if graphs else [])
        assert e.states.free_slots == e.states.num_slots
    for a, b in zip(outs[False], outs[True]):
        assert a.output_ids == b.output_ids
        torch.testing.assert_close(torch.tensor(a.output_logprobs),
                                   torch.tensor(b.output_logprobs),
                                   rtol=1e-5, atol=1e-5)
