"""The Bizusun family in the rollout engine against the plain oracle
(tests/bizusun_oracle.py): every mixer and feed-forward alone, whole prompts
against token-by-token decoding, portions down to two tokens, unequal
batches, reuse of pages and state slots, window and page edges, long
decoding, odd sizes, the checkpoint-folder loader, the trace replay entry
point and greedy generation through the engine's scheduler.

Every case runs on the CPU tier (PyTorch forms of the ops, fp32) and, marked
``gpu``, on the HIP kernels in fp32 and bf16.  Configurations are small and
made here; weights are random with a fixed seed (bf16-representable).
"""
import copy
import io
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bizusun_oracle as O  # noqa: E402

from polyrl_amd.models.hybrid import bizusun_config_from_json  # noqa: E402
from polyrl_amd.rollout.engine import Engine, SamplingParams  # noqa: E402
from polyrl_amd.rollout.hybrid_model import HybridInferenceModel  # noqa: E402

CPU = ("cpu", torch.float32)
GPU32 = pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu)
GPU16 = pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)
TARGETS = [CPU, GPU32, GPU16]

DELTA = {"type": "general_delta", "mixer": {"heads": 3, "dim": 16}}
SSM = {"type": "mamba2", "mixer": {"heads": 4, "vdim": 12, "state": 20,
                                    "groups": 2, "norm_groups": 2, "conv": 3}}


def attn(window=7, kv_from=None, heads=3, dim=24, rot=8, vdim=20, rank=40):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim,
         "kv_rank": rank, "mask": {"size": window},
         "rot": {"base": 100.0, "dims": rot},
         "scale": 1.0 / math.sqrt(dim + rot)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


DENSE = {"kind": "dense", "ff": 72}
MOE = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 5, "top": 3}}
MOE1 = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 3, "top": 1}}


def config(layers, width=48, vocab=97, taps=3, side=10, scale=0.5):
    return {"architecture": "Bizusun", "vocab": vocab, "width": width,
            "layers": [dict(copy.deepcopy(m), mlp=copy.deepcopy(f))
                       for m, f in layers],
            "norm": {"eps": 1e-5}, "canon": {"taps": taps},
            "token_side": {"dim": side}, "logit_scale": scale}


FULL = config([(DELTA, DENSE), (attn(), MOE), (SSM, MOE1),
               (attn(kv_from=1), None), (DELTA, MOE)])


def engine(cfg, W, target, tokens=512, slots=4, page=4, **kw):
    dev, dt = target
    c = bizusun_config_from_json(cfg)
    HybridInferenceModel.resolve_shapes(
        c, {k: tuple(v.shape) for k, v in W.items()})
    e = Engine(c, device=dev, dtype=dt, page_size=page,
               kv_token_capacity=tokens, max_running_requests=slots,
               max_num_batched_tokens=kw.pop("budget", 1 << 20), **kw)
    e.model.load_state_dict(W)
    return e


def close(got, want, target, what=""):
    """Logit rows agree: error (mean removed, RMS over the vocabulary) over
    the oracle's own RMS."""
    got, want = got.double().cpu(), want.double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)
    # bf16: the oracle rounds nothing, so single rows can sit near 0.1 of
    # the logits' spread while the typical row stays below 0.02
    lim = 0.15 if target[1] == torch.bfloat16 else 2e-4
    assert float(err.max()) < lim, f"{what}: {float(err.max()):.3g} >= {lim}"
    if target[1] == torch.bfloat16 and err.numel() >= 8:
        assert float(err.median()) < 0.03, f"{what}: median {err.median()}"


def toks(n, vocab=97, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def run(e, rid, t, want=None, end=True):
    want = list(range(len(t))) if want is None else want
    return e.step_forced([(rid, t, want)], [rid] if end else [])


# ------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name,layers", [
    ("delta", [(DELTA, None)]),
    ("ssm", [(SSM, None)]),
    ("attention", [(attn(), None)]),
    ("shared-cache", [(attn(window=5), None), (attn(window=9, kv_from=0,
                                                     heads=2, dim=16,
                                                     vdim=12), None)]),
    # key (dim + rot) and value sizes in multiples of 8: bf16 prompt steps
    # attend in the expanded form on the matrix cores
    ("attention-expanded", [(attn(vdim=24), None)]),
    ("shared-cache-expanded", [(attn(window=5, vdim=16), None),
                               (attn(window=9, kv_from=0, heads=2, dim=16,
                                     vdim=8), None)]),
    ("dense", [(DELTA, DENSE)]),
    ("experts", [(DELTA, MOE)]),
    ("one-expert", [(SSM, MOE1)]),
])
def test_mechanism_alone(target, name, layers):
    cfg = config(layers)
    W = O.random_weights(cfg, seed=3)
    t = toks(23, seed=1)
    got = run(engine(cfg, W, target), "a", t)
    close(got, O.forward(cfg, W, t), target, name)


@pytest.mark.parametrize("target", TARGETS)
def test_one_tap_and_no_side_and_sizes_of_one(target):
    """Sizes that often coincide or equal one: taps 1 (no history), a conv
    of 2 taps, one head, one group, one expert of one, no side input."""
    ssm = {"type": "mamba2", "mixer": {"heads": 1, "vdim": 16, "state": 8,
                                        "groups": 1, "norm_groups": 1,
                                        "conv": 2}}
    one = {"kind": "moe", "expert": {"ff": 24},
           "router": {"experts": 1, "top": 1}}
    cfg = config([({"type": "general_delta",
                    "mixer": {"heads": 1, "dim": 20}}, one), (ssm, DENSE),
                  (attn(window=1, heads=1), None)], width=40, taps=1, side=4,
                 scale=1.0)
    W = O.random_weights(cfg, seed=5)
    t = toks(12, seed=2)
    close(run(engine(cfg, W, target), "a", t), O.forward(cfg, W, t), target)


# --------------------------------------- layers of the residual stream
@pytest.mark.parametrize("target", [CPU, GPU32])
def test_residual_after_every_layer(target):
    W = O.random_weights(FULL, seed=7)
    t = toks(17, seed=3)
    e = engine(FULL, W, target)
    e.model.capture_layers = []
    run(e, "a", t)
    _, layers = O.forward(FULL, W, t, return_layers=True)
    for li, got in enumerate(e.model.capture_layers):
        torch.testing.assert_close(got.double().cpu(), layers[li],
                                   rtol=2e-4, atol=2e-4,
                                   msg=lambda m: f"layer {li}: {m}")


# ----------------------------------- whole / decode / portions / batches
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_decode_and_portions_agree_with_oracle(target):
    W = O.random_weights(FULL, seed=11)
    t = toks(41, seed=4)
    want = O.forward(FULL, W, t)
    e = engine(FULL, W, target)
    close(run(e, "whole", t), want, target, "whole")
    # token by token from the first token on
    rows = [e.step_forced([("dec", [x], [0])], []) for x in t]
    e.step_forced([], ["dec"])
    close(torch.cat(rows), want, target, "decode")
    # portions of changing size, down to two tokens and one
    for sizes in ([2, 2, 3, 5, 2, 9, 1, 1, 2, 14], [7, 1, 33], [40, 1]):
        assert sum(sizes) == len(t)
        rows, at = [], 0
        for n in sizes:
            rows.append(e.step_forced(
                [("p", t[at:at + n], list(range(n)))], []))
            at += n
        e.step_forced([], ["p"])
        close(torch.cat(rows), want, target, f"portions {sizes}")
    assert e.kv.free_pages == e.kv.num_pages
    assert e.states.free_slots == e.states.num_slots


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_batch_matches_each_alone(target):
    W = O.random_weights(FULL, seed=13)
    seqs = {"a": toks(19, seed=5), "b": toks(3, seed=6), "c": toks(30, seed=7),
            "d": toks(1, seed=8)}
    want = {k: O.forward(FULL, W, v) for k, v in seqs.items()}
    e = engine(FULL, W, target)
    # step 1: a whole, c's first 11; step 2: b whole, c's next 2, d;
    # then a few steps of c alone beside nothing, one token at a time
    g1 = e.step_forced([("a", seqs["a"], list(range(19))),
                        ("c", seqs["c"][:11], list(range(11)))], ["a"])
    close(g1[:19], want["a"], target, "a in batch")
    close(g1[19:], want["c"][:11], target, "c first portion")
    g2 = e.step_forced([("b", seqs["b"], [0, 1, 2]),
                        ("c", seqs["c"][11:13], [0, 1]),
                        ("d", seqs["d"], [0])], ["b", "d"])
    close(g2[:3], want["b"], target, "b in batch")
    close(g2[3:5], want["c"][11:13], target, "c second portion")
    close(g2[5:], want["d"], target, "d in batch")
    rest = [e.step_forced([("c", [x], [0])], []) for x in seqs["c"][13:]]
    close(torch.cat(rest), want["c"][13:], target, "c decoded")


@pytest.mark.parametrize("target", TARGETS)
def test_pages_and_slots_are_reused_clean(target):
    """A pool of two slots and few pages: later requests get slots and
    pages that earlier ones left dirty, and must not see them."""
    W = O.random_weights(FULL, seed=17)
    e = engine(FULL, W, target, tokens=48, slots=2, page=4)
    for i in range(5):
        a, b = toks(20 + i, seed=20 + i), toks(9 + 2 * i, seed=40 + i)
        got = e.step_forced([(f"a{i}", a, [len(a) - 1]),
                             (f"b{i}", b[:4], [])], [f"a{i}"])
        close(got, O.forward(FULL, W, a)[-1:], target, f"a{i}")
        got = e.step_forced([(f"b{i}", b[4:], [len(b) - 5])], [f"b{i}"])
        close(got, O.forward(FULL, W, b)[-1:], target, f"b{i}")
    with pytest.raises(RuntimeError):       # third live request: no slot
        e.step_forced([("x", [1], []), ("y", [2], []), ("z", [3], [])], [])


# -------------------------------------------- windows, pages, far tokens
def _loud_key_model(window, vdim=20):
    """One attention layer (plus a sharer) where one token id has a huge
    rotated-key part, so whichever query still sees it attends to it: a
    window that is one token off changes the logits at its edge."""
    cfg = config([(attn(window=window, rank=24, vdim=vdim), None),
                  (attn(window=window + 3, kv_from=0, rank=24, vdim=vdim),
                   DENSE)],
                 taps=1, side=6)
    W = O.random_weights(cfg, seed=23)
    W["embed"][5] *= 12.0                   # token 5 = the loud key
    W["l0.mix.sink"] = torch.full_like(W["l0.mix.sink"], 2.5)
    return cfg, W


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("window,vdim", [(4, 20), (9, 20), (16, 20),
                                         (4, 24), (9, 24), (16, 24)])
def test_window_edge_in_prompt_and_decode(target, window, vdim):
    cfg, W = _loud_key_model(window, vdim)
    t = [x if x != 5 else 6 for x in toks(3 * window + 9, seed=9)]
    loud = window + 1                       # crosses a page edge for page=4
    t[loud] = 5
    want = O.forward(cfg, W, t)
    # the loud key must matter exactly while it is inside the window
    t2 = list(t)
    t2[loud] = 6
    other = O.forward(cfg, W, t2)
    d = (want - other).abs().max(-1).values
    assert float(d[loud + window - 1]) > 1e-2, "test model hides the edge"
    e = engine(cfg, W, target, page=4)
    close(run(e, "whole", t), want, target, "prompt")
    cut = loud + 2                          # the edge is crossed in decoding
    rows = [e.step_forced([("d", t[:cut], list(range(cut)))], [])]
    rows += [e.step_forced([("d", [x], [0])], []) for x in t[cut:]]
    close(torch.cat(rows), want, target, "decoded")
    # portions that start and end at, before and after the edge
    for first in (loud + window - 2, loud + window - 1, loud + window):
        rows = [e.step_forced([(f"p{first}", t[:first],
                                list(range(first)))], []),
                e.step_forced([(f"p{first}", t[first:],
                                list(range(len(t) - first)))], [f"p{first}"])]
        close(torch.cat(rows), want, target, f"cut at {first}")


@pytest.mark.parametrize("target", TARGETS)
def test_far_token_reaches_through_recurrent_state(target):
    """The first token decides the last logits only through the recurrent
    states (the window is shorter than the distance): a lost or stale state
    shows."""
    cfg = config([(DELTA, None), (SSM, None), (attn(window=3), None)])
    W = O.random_weights(cfg, seed=29)
    W["l0.mix.w0"] -= 6.0                   # slow decay: long memory
    W["l1.mix.A_log"] -= 4.0
    t = toks(70, seed=10)
    t2 = [(t[0] + 1) % 97] + t[1:]
    a, b = O.forward(cfg, W, t), O.forward(cfg, W, t2)
    assert float((a[-1] - b[-1]).abs().max()) > 1e-3, "no long memory"
    e = engine(cfg, W, target)
    for seq_, want in ((t, a), (t2, b)):
        rows = [e.step_forced([("r", seq_[:9], [])], [])]
        rows = [e.step_forced([("r", [x], [0])], []) for x in seq_[9:]]
        e.step_forced([], ["r"])
        close(torch.cat(rows), want[9:], target, "long decode")


@pytest.mark.parametrize("target", TARGETS)
def test_first_tokens(target):
    W = O.random_weights(FULL, seed=31)
    e = engine(FULL, W, target)
    for n in (1, 2, 3, 4):
        t = toks(n, seed=50 + n)
        close(run(e, f"s{n}", t), O.forward(FULL, W, t), target, f"len {n}")


# ------------------------------------- loader, replay entry, generation
def _save(tmp_path, cfg, W):
    from safetensors.torch import save_file
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: (v if v.dtype == torch.int32 else v.bfloat16()).contiguous()
               for k, v in W.items()}, str(d / "model.safetensors"))
    return str(d)


@pytest.mark.parametrize("target", [CPU, GPU32])
def test_folder_loader_and_trace_replay(target, tmp_path, monkeypatch, capsys):
    from polyrl_amd.models import get_model_config
    from polyrl_amd.rollout import trace_replay
    W = O.random_weights(FULL, seed=37)
    path = _save(tmp_path, FULL, W)
    c = get_model_config(path)
    assert c.arch == "bizusun" and c.num_hidden_layers == 5
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
    wa, wb = O.forward(FULL, W, a), O.forward(FULL, W, b)
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
    mixed steps, sampling at temperature 0, slots released at the end."""
    if target[0] == "cuda":
        import polyrl_amd.ops as ops
        assert ops.extension_loaded()
    W = O.random_weights(FULL, seed=41)
    e = engine(FULL, W, target, slots=3, budget=8)
    prompts = [toks(n, seed=70 + n) for n in (11, 2, 17, 5)]
    outs = e.generate(prompts, SamplingParams(temperature=0.0,
                                              max_new_tokens=5), "g")
    for p, o in zip(prompts, outs):
        ids = list(p)
        for got_tok in o.output_ids:
            logits = O.forward(FULL, W, ids)[-1]
            top2 = logits.topk(2).values
            tie = 1e-3 if target[1] == torch.float32 else \
                0.25 * float(logits.std())
            if float(top2[0] - top2[1]) > tie:      # skip near ties
                assert got_tok == int(logits.argmax())
            ids.append(got_tok)
        assert len(o.output_ids) == 5 and o.finish_reason == "length"
    assert e.kv.free_pages == e.kv.num_pages
    assert e.states.free_slots == e.states.num_slots


def test_release_and_resume_memory():
    W = O.random_weights(FULL, seed=43)
    e = engine(FULL, W, CPU)
    t = toks(9, seed=90)
    a = run(e, "a", t)
    e.release_memory()
    assert not e.kv.rows and not e.states.tensors
    e.resume_memory()
    torch.testing.assert_close(run(e, "b", t), a)
