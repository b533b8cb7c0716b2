"""HIP sequence-mixer kernels (csrc/seq_*.hip) against their plain PyTorch
fp32 forms (ops/seq_ref.py) on packed batches of unequal portions, in bf16
and fp32, with odd sizes that exercise every guard (rows per lane, columns
per wave, latent-row chunks, partial key blocks)."""
import math

import pytest
import torch

from polyrl_amd.ops import seq
from polyrl_amd.ops import seq_ref as R

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else \
        dict(rtol=2e-5, atol=2e-5)


def batch(lens, slots):
    cu = [0]
    sot = []
    for b, n in enumerate(lens):
        cu.append(cu[-1] + n)
        sot += [b] * n
    i32 = lambda x, d: torch.tensor(x, dtype=torch.int32, device=d)
    return {d: (i32(cu, d), i32(slots, d), i32(sot, d)) for d in ("cpu", DEV)}


def rnd(*s, dt=torch.float32, scale=1.0, seed=None):
    return (torch.randn(*s) * scale).to(dt)


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(1234)
    assert seq.seq_extension_loaded(), "polyrl_amd._hip_seq must be built"


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("D,wn", [(192, 1), (200, 200), (2048, 1)])
def test_add_rmsnorm_modes(dt, D, wn):
    N = 7
    res, y, w = rnd(N, D), rnd(N, D, dt=dt), rnd(wn).abs() + 0.5
    r0, r1 = res.clone(), res.clone().to(DEV)
    want = R.add_rmsnorm_f32res(r0, y, w, 1e-6, dt)
    got = seq.add_rmsnorm_f32res(r1, y.to(DEV), w.to(DEV), 1e-6, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-6, atol=1e-6)
    # no-add form leaves the residual alone
    got2 = seq.add_rmsnorm_f32res(r1, None, w.to(DEV), 1e-6, dt)
    torch.testing.assert_close(r1.cpu(), r0, rtol=0, atol=0)
    torch.testing.assert_close(
        got2.cpu().float(), R.add_rmsnorm_f32res(r0, None, w, 1e-6, dt).float(),
        **tol(dt))
    x = seq.residual_add_cast(r1, y.to(DEV), dt)
    xw = R.residual_add_cast(r0, y, dt)
    torch.testing.assert_close(x.cpu().float(), xw.float(), **tol(dt))
    wv = rnd(D).abs() + 0.5
    seq.add_scaled_unit_rms(r1, y.to(DEV), wv.to(DEV), 1e-6)
    R.add_scaled_unit_rms(r0, y, wv, 1e-6)
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("taps,lens", [(4, [5, 1, 2, 9]), (1, [3, 1]),
                                       (6, [2, 2, 1, 7])])
def test_causal_conv_state_portions(dt, taps, lens):
    C, slots = 300, [3, 0, 5, 1][:len(lens)]
    bt = batch(lens, slots)
    N = sum(lens)
    big = rnd(N, C + 40, dt=dt)
    w, bias = rnd(C, taps, scale=0.5), rnd(C)
    st0 = rnd(6, taps - 1, C)
    for add, silu, b in [(True, False, None), (False, True, bias)]:
        sc, sg = st0.clone(), st0.clone().to(DEV)
        want = R.causal_conv_state(big[:, 17:17 + C], w, b, sc, *bt["cpu"],
                                   add, silu, dt)
        got = seq.causal_conv_state(
            big.to(DEV)[:, 17:17 + C], w.to(DEV),
            None if b is None else b.to(DEV), sg, *bt[DEV], add, silu, dt)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
        torch.testing.assert_close(sg.cpu(), sc, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,Dk,lens", [(3, 32, [6, 1, 3]), (2, 24, [4, 1]),
                                       (2, 80, [1, 5]), (1, 128, [3])])
def test_delta_rule_scan(dt, H, Dk, lens):
    Dv = Dk
    slots = [2, 0, 3][:len(lens)]
    bt = batch(lens, slots)
    N, n = sum(lens), H * Dk
    big = rnd(N, 6 * n, dt=dt)
    col = lambda t, i: t[:, i * n:(i + 1) * n]
    w0, ab, nw = rnd(n), rnd(n), rnd(n).abs() + 0.5
    st0 = rnd(4, H, Dk, Dv, scale=0.3)
    sc, sg = st0.clone(), st0.clone().to(DEV)
    args = lambda t, d: [col(t, i) for i in range(6)]
    a = args(big, "cpu")
    want = R.delta_rule(*a, w0, ab, nw, sc, bt["cpu"][0], bt["cpu"][1],
                        math.exp(-0.5), 1e-6, 1e-6, dt)
    g = args(big.to(DEV), DEV)
    got = seq.delta_rule(*g, w0.to(DEV), ab.to(DEV), nw.to(DEV), sg,
                         bt[DEV][0], bt[DEV][1], math.exp(-0.5), 1e-6, 1e-6,
                         dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(sg.cpu(), sc, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,P,Ns,G,lens", [(6, 32, 48, 1, [5, 1, 2]),
                                           (4, 24, 16, 2, [1, 7]),
                                           (4, 80, 128, 4, [3])])
def test_ssm_scan(dt, H, P, Ns, G, lens):
    slots = [1, 3, 0][:len(lens)]
    bt = batch(lens, slots)
    N, inner = sum(lens), H * P
    ch = inner + 2 * G * Ns
    big = rnd(N, inner + ch + H, dt=dt)
    z, xbc, dtt = big[:, :inner], big[:, inner:inner + ch], big[:, inner + ch:]
    dtb, al, dk = rnd(H), rnd(H, scale=0.5), rnd(H)
    st0 = rnd(4, H, Ns, P, scale=0.3)
    sc, sg = st0.clone(), st0.clone().to(DEV)
    want = R.ssm_scan(xbc, dtt, z, dtb, al, dk, sc, bt["cpu"][0],
                      bt["cpu"][1], G)
    bg = big.to(DEV)
    got = seq.ssm_scan(bg[:, inner:inner + ch], bg[:, inner + ch:],
                       bg[:, :inner], dtb.to(DEV), al.to(DEV), dk.to(DEV), sg,
                       bt[DEV][0], bt[DEV][1], G)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(sg.cpu(), sc, rtol=1e-4, atol=1e-4)
    for groups in (1, H):
        nw = rnd(inner).abs() + 0.5
        torch.testing.assert_close(
            seq.group_rmsnorm(got, nw.to(DEV), groups, 1e-6, dt).cpu().float(),
            R.group_rmsnorm(want, nw, groups, 1e-6, dt).float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,R_,rd,dims,window", [(3, 64, 16, 16, 5),
                                                 (2, 40, 24, 16, 40),
                                                 (2, 200, 32, 32, 7)])
def test_latent_store_and_attention(dt, H, R_, rd, dims, window):
    ps, pages = 4, 40
    lens, starts = [9, 1, 3], [0, 21, 6]       # portions at these offsets
    # sequences hold start+len tokens; scatter their pages on purpose
    perm = torch.randperm(pages).tolist()
    ptab, used = [], 0
    for s, n in zip(starts, lens):
        need = -(-(s + n) // ps)
        ptab.append(perm[used:used + need] + [0] * (10 - need))
        used += need
    ptab_t = torch.tensor(ptab, dtype=torch.int32)
    inv = seq.rope_inv_freq(dims, 10000.0, "cpu")
    cache = rnd(pages, ps, R_ + rd, dt=dt)     # "history" = random rows
    pos, sot, slot = [], [], []
    for b, (s, n) in enumerate(zip(starts, lens)):
        for p in range(s, s + n):
            pos.append(p)
            sot.append(b)
            slot.append(ptab[b][p // ps] * ps + p % ps)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    N = len(pos)
    dkv, nw = rnd(N, R_ + rd + 8, dt=dt), rnd(R_).abs() + 0.5
    cc, cg = cache.clone(), cache.clone().to(DEV)
    R.latent_kv_store(dkv[:, 8:], R_, nw, 1e-6, i32(pos), inv, cc, i32(slot))
    seq.latent_kv_store(dkv.to(DEV)[:, 8:], R_, nw.to(DEV), 1e-6,
                        i32(pos).to(DEV), inv.to(DEV), cg, i32(slot).to(DEV))
    torch.testing.assert_close(cg.cpu().float(), cc.float(), **tol(dt))
    q = rnd(N, H, 20 + rd, dt=dt)
    qc, qg = q.clone(), q.clone().to(DEV)
    R.rope_partial_(qc, 20, inv, i32(pos))
    seq.rope_partial_(qg, 20, inv.to(DEV), i32(pos).to(DEV))
    torch.testing.assert_close(qg.cpu().float(), qc.float(), **tol(dt))
    q_lat, sink = rnd(N, H, R_, dt=dt, scale=0.3), rnd(H)
    want = R.latent_window_attention(q_lat, qc[:, :, 20:], cc, ptab_t,
                                     i32(sot), i32(pos), window, sink, 0.2,
                                     dt)
    got = seq.latent_window_attention(
        q_lat.to(DEV), qc.to(DEV)[:, :, 20:], cc.to(DEV), ptab_t.to(DEV),
        i32(sot).to(DEV), i32(pos).to(DEV), window, sink.to(DEV), 0.2, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_activations_and_combine(dt):
    N, C = 11, 72
    big = rnd(N, 2 * C + 5, dt=dt)
    a, b = big[:, 3:3 + C], big[:, 3 + C:3 + 2 * C]
    ag, bg = big.to(DEV)[:, 3:3 + C], big.to(DEV)[:, 3 + C:3 + 2 * C]
    for f, rf in [(seq.silu_mul_any, R.silu_mul_any),
                  (seq.sigmoid_mul, R.sigmoid_mul)]:
        torch.testing.assert_close(f(ag, bg).cpu().float(),
                                   rf(a, b).float(), **tol(dt))
    torch.testing.assert_close(seq.tanh_act(ag).cpu().float(),
                               R.tanh_act(a).float(), **tol(dt))
    table, tok = rnd(50, 3 * C, dt=dt), torch.randint(0, 50, (N,))
    torch.testing.assert_close(
        seq.gelu_tanh_mul_rows(ag, table.to(DEV), tok.to(DEV), C).cpu().float(),
        R.gelu_tanh_mul_rows(a, table, tok, C).float(), **tol(dt))
    top = 3
    y = rnd(N * top, C, dt=dt)
    inv = torch.randperm(N * top).view(N, top).int()
    r0 = rnd(N, C)
    r1 = r0.clone().to(DEV)
    R.moe_combine_(r0, y, inv, 1.0 / top)
    seq.moe_combine_(r1, y.to(DEV), inv.to(DEV), 1.0 / top)
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("N,top,E", [(1, 2, 4), (37, 3, 5), (64, 1, 2)])
def test_moe_table_ffn_bf16(N, top, E):
    W, ff, V = 96, 64, 50
    dt = torch.bfloat16
    h = rnd(N, W, dt=dt)
    tok = torch.randint(0, V, (N,))
    table = torch.stack([torch.randperm(E)[:top] for _ in range(V)]).int()
    if N > 20:
        table[:, 0] = 0                     # one crowded expert: > 16 rows
    w_gu, w_down = rnd(E, 2 * ff, W, dt=dt, scale=0.1), \
        rnd(E, W, ff, dt=dt, scale=0.1)
    assert seq.moe_table_ffn_supported(h.to(DEV), top, ff)
    got = seq.moe_table_ffn(h.to(DEV), tok.to(DEV), table.to(DEV),
                            w_gu.to(DEV), w_down.to(DEV))
    want = R.moe_table_ffn(h, tok, table, w_gu, w_down)
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=3e-2,
                               atol=3e-2)


@pytest.mark.parametrize("H,R_,rd,window,lens,starts", [
    (3, 64, 16, 5, [9, 1, 3], [0, 21, 6]),
    (6, 40, 24, 40, [70, 2], [3, 90]),
    (70, 256, 32, 33, [1, 1, 1], [0, 40, 131]),       # decode: heads as rows
    (2, 512, 64, 100, [130], [17]),
])
def test_latent_attention_matrix_cores(H, R_, rd, window, lens, starts):
    dt = torch.bfloat16
    ps, pages = 16, 64
    perm = torch.randperm(pages).tolist()
    ptab, used = [], 0
    for s, n in zip(starts, lens):
        need = -(-(s + n) // ps)
        ptab.append(perm[used:used + need] + [0] * (20 - need))
        used += need
    ptab_t = torch.tensor(ptab, dtype=torch.int32)
    cache = rnd(pages, ps, R_ + rd, dt=dt)
    pos, sot = [], []
    for b, (s, n) in enumerate(zip(starts, lens)):
        pos += list(range(s, s + n))
        sot += [b] * n
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    N = len(pos)
    q_lat, q_rot = rnd(N, H, R_, dt=dt, scale=0.3), rnd(N, H, rd, dt=dt)
    sink = rnd(H)
    sc = 1.0 / math.sqrt(R_ / 4 + rd)
    want = R.latent_window_attention(q_lat, q_rot, cache, ptab_t, i32(sot),
                                     i32(pos), window, sink, sc, dt)
    tiles = seq.attention_tiles(lens, DEV)
    assert tiles[2] == (1 if max(lens) == 1 else 0)
    got = seq.latent_window_attention(
        q_lat.to(DEV), q_rot.to(DEV), cache.to(DEV), ptab_t.to(DEV),
        i32(sot).to(DEV), i32(pos).to(DEV), window, sink.to(DEV), sc, dt,
        tiles=tiles)
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=3e-2,
                               atol=3e-2)


# --------------------------------- sandwich norms, GQA window attention, router
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("D", [48, 200, 2048])
def test_offset_norms_and_fused_joint(dt, D):
    N = 9
    res, y = rnd(N, D), rnd(N, D + 8, dt=dt)[:, 3:3 + D]
    wa, wb = rnd(D, scale=0.2), rnd(D, scale=0.2)
    r0, r1 = res.clone(), res.clone().to(DEV)
    want = R.add_unit_rms_then_norm(r0, y, wa, wb, 1e-5, dt, 1.0)
    got = seq.add_unit_rms_then_norm(r1, y.to(DEV), wa.to(DEV), wb.to(DEV),
                                     1e-5, dt, 1.0)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)
    seq.add_scaled_unit_rms(r1, y.to(DEV), wb.to(DEV), 1e-5, 1.0)
    R.add_scaled_unit_rms(r0, y, wb, 1e-5, 1.0)
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)
    got = seq.add_rmsnorm_f32res(r1, None, wa.to(DEV), 1e-5, dt, 1.0)
    want = R.add_rmsnorm_f32res(r0, None, wa, 1e-5, dt, 1.0)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


def _paged(lens, starts, page, row, dt):
    """Page tables for sequences of starts[b]+lens[b] tokens on shuffled
    pages, and the packed batch of each one's last lens[b] tokens."""
    total = [s + n for s, n in zip(starts, lens)]
    need = [-(-t // page) for t in total]
    perm = torch.randperm(sum(need) + 3).tolist()
    ptab = torch.zeros(len(lens), max(need), dtype=torch.int32)
    o = 0
    for b, k in enumerate(need):
        ptab[b, :k] = torch.tensor(perm[o:o + k], dtype=torch.int32)
        o += k
    cache = rnd(sum(need) + 3, page, row, dt=dt)
    pos, sot, slot = [], [], []
    for b, (s, n) in enumerate(zip(starts, lens)):
        for p in range(s, s + n):
            pos.append(p)
            sot.append(b)
            slot.append(int(ptab[b, p // page]) * page + p % page)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    return cache, ptab, i32(pos), i32(sot), i32(slot)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,half,norm,own_v", [
    (4, 2, 24, 24, 4, True, False), (6, 3, 64, 64, 32, True, False),
    (4, 1, 16, 40, 0, False, True), (2, 2, 128, 128, 16, True, False),
    (8, 2, 32, 32, 8, False, True)])
def test_gqa_prepare_store(dt, H, G, D, Dv, half, norm, own_v):
    lens, starts, page = [5, 1, 3], [0, 37, 6], 4
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, G * (D + Dv), dt)
    N = sum(lens)
    big = rnd(N, H * D + G * D + G * Dv + 5, dt=dt)
    q, k = big[:, :H * D], big[:, H * D:H * D + G * D]
    v = big[:, H * D + G * D:H * D + G * D + G * Dv] if own_v else None
    qn = (rnd(H * D, scale=0.2) + 1) if norm else None
    kn = (rnd(G * D, scale=0.2) + 1) if norm else None
    inv = torch.rand(half) if half else None
    c0, c1 = cache.clone(), cache.clone().to(DEV)
    want = R.gqa_prepare_store(q, k, v, qn, kn, 1e-5, inv, 1.07, pos, c0, slot,
                               H, G, D, Dv)
    g = lambda t: None if t is None else t.to(DEV)
    got = seq.gqa_prepare_store(g(big)[:, :H * D],
                                g(big)[:, H * D:H * D + G * D],
                                None if v is None else
                                g(big)[:, H * D + G * D:H * D + G * D + G * Dv],
                                g(qn), g(kn), 1e-5, g(inv), 1.07, g(pos), c1,
                                g(slot), H, G, D, Dv)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(c1.cpu().float(), c0.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,window,keep,bias,gate,lens,starts", [
    (4, 2, 24, 24, 7, 2, False, True, [5, 1, 3], [0, 37, 6]),
    (6, 3, 64, 64, 16, 5, False, True, [40, 1, 1, 2], [3, 70, 0, 15]),
    (4, 1, 16, 40, 9, 0, True, False, [5, 1, 30], [0, 37, 6]),
    (2, 2, 128, 128, 33, 4, False, False, [70, 1], [10, 200]),
    (8, 2, 32, 96, 20, 0, True, False, [64, 1, 9], [0, 19, 64]),
    (3, 3, 200, 72, 5, 1, False, True, [6, 2], [0, 9]),
    (4, 2, 64, 64, 16, 70, False, True, [100, 1, 40], [50, 300, 0]),
    (2, 1, 40, 24, 200, 0, True, False, [130, 1, 70], [170, 450, 0]),
    (4, 4, 96, 96, 40, 33, False, False, [1, 1, 1], [0, 31, 200]),
    (16, 8, 32, 32, 50, 3, False, True, [130, 1, 70], [20, 90, 0]),
    (8, 8, 24, 16, 1 << 30, 0, False, False, [200, 3], [0, 64]),
    (16, 16, 16, 8, 90, 0, False, True, [65, 64, 1], [0, 1, 5]),
])
def test_gqa_window_attention(dt, H, G, D, Dv, window, keep, bias, gate,
                              lens, starts):
    page = 4
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, G * (D + Dv), dt)
    N = sum(lens)
    # peaky softmax (score spread of several units): one key missing or one
    # too many moves the output far beyond the tolerance
    q = rnd(N, H * D, dt=dt, scale=2.5)
    rel = rnd(10, H) if bias else None
    dist = torch.randint(0, 10, (window,), dtype=torch.int32) if bias else None
    gfull = rnd(N, H + 3, dt=dt)
    gt = gfull[:, 1:1 + H] if gate else None
    gfull = gfull.to(DEV)
    scale = 1.0 / math.sqrt(D)
    want = R.gqa_window_attention(q, cache, ptab, sot, pos, H, G, D, Dv,
                                  window, keep, rel, dist, gt, scale, dt)
    g = lambda t: None if t is None else t.to(DEV)
    tiles = seq.attention_tiles(lens, DEV)
    for tl in (None, tiles):                 # one wave per row; matrix cores
        got = seq.gqa_window_attention(
            g(q), g(cache), g(ptab), g(sot), g(pos), H, G, D, Dv, window,
            keep, g(rel), g(dist),
            None if gt is None else gfull[:, 1:1 + H], scale, dt, tiles=tl)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


@pytest.mark.parametrize("N,top,E,n_id", [(1, 2, 4, 1), (37, 3, 5, 2),
                                          (64, 1, 2, 0), (200, 2, 6, 2)])
def test_routed_experts_bf16(N, top, E, n_id):
    dt = torch.bfloat16
    Wd, ff = 96, 64
    h = rnd(N, Wd, dt=dt)
    idx = torch.stack([torch.randperm(E + n_id)[:top] for _ in range(N)]).int()
    w = torch.rand(N, top)
    up, down = rnd(E, ff, Wd, dt=dt, scale=0.1), rnd(E, Wd, ff, dt=dt, scale=0.1)
    shared = rnd(N, Wd, dt=dt)
    ys0 = R.moe_routed_ffn(h, idx, up, down)
    want = R.moe_weighted_combine(ys0, idx, w, h, shared, E, 1e-20, dt)
    assert seq.moe_routed_ffn_supported(h.to(DEV), top, ff)
    ys1 = seq.moe_routed_ffn(h.to(DEV), idx.to(DEV), up.to(DEV), down.to(DEV))
    real = (idx < E).reshape(-1)
    torch.testing.assert_close(ys1.cpu().float()[real], ys0.float()[real],
                               **tol(dt))
    got = seq.moe_weighted_combine(ys1, idx.to(DEV), w.to(DEV), h.to(DEV),
                                   shared.to(DEV), E, 1e-20, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    got = seq.moe_weighted_combine(ys1.float(), idx.to(DEV), w.to(DEV),
                                   h.to(DEV).float(), None, E, 1e-20,
                                   torch.float32)
    want = R.moe_weighted_combine(ys0.float(), idx, w, h.float(), None, E,
                                  1e-20, torch.float32)
    torch.testing.assert_close(got.cpu()[:, :], want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dt", DTYPES)
def test_gelu_erf(dt):
    x = rnd(33, 70, dt=dt, scale=2.0)
    torch.testing.assert_close(seq.gelu_erf(x.to(DEV)[:, 3:60]).cpu().float(),
                               R.gelu_erf(x[:, 3:60]).float(), **tol(dt))


# ------------------ composed embedding, gated linear attention, causal
# attention with sink and query temperature, clamped gated unit, scaled joins
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("D,pair,pos", [(48, True, True), (37, True, False),
                                        (200, False, True), (16, False, False)])
def test_embed_compose(dt, D, pair, pos):
    V, buckets, N = 50, 23, 19
    table = rnd(V, D, dt=dt)
    ptab = rnd(buckets + 1, D, dt=dt) if pair else None
    tok = torch.randint(0, V, (N,))
    prev = torch.randint(0, V, (N,))
    prev[[0, 7, 8]] = -1                     # starts of sequences
    p = torch.randint(0, 3000, (N,), dtype=torch.int32)
    f = seq.sinusoid_inv_freq(D, 10000.0, "cpu") if pos else None
    want = R.embed_compose(table, tok, 3.25, ptab, prev, 29, 3, buckets, p, f)
    g = lambda t: None if t is None else t.to(DEV)
    got = seq.embed_compose(g(table), g(tok), 3.25, g(ptab), g(prev), 29, 3,
                            buckets, g(p), g(f))
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,Dk,Dv,lens", [
    (3, 32, 32, [6, 1, 3]), (2, 24, 40, [4, 1]), (2, 80, 16, [1, 5]),
    (1, 128, 70, [3]), (3, 5, 3, [2, 7, 1]), (2, 48, 32, [33, 1]),
    (2, 64, 128, [70, 1, 32]), (1, 200, 16, [40, 15]), (1, 256, 8, [29]),
    (1, 320, 24, [11, 2])])
def test_gla_scan(dt, H, Dk, Dv, lens):
    slots = [2, 0, 3][:len(lens)]
    bt = batch(lens, slots)
    N = sum(lens)
    nk, nv = H * Dk, H * Dv
    big = rnd(N, 3 * nk + nv + 5, dt=dt)     # operands are column slices
    cols = lambda t: (t[:, :nk], t[:, nk:2 * nk], t[:, 2 * nk:2 * nk + nv],
                      t[:, 2 * nk + nv:3 * nk + nv])
    zb = rnd(nk) + 2.0
    st0 = rnd(4, H, Dk, Dv, scale=0.3)
    sc, sg = st0.clone(), st0.clone().to(DEV)
    want = R.gla_scan(*cols(big), zb, sc, bt["cpu"][0], bt["cpu"][1],
                      Dk ** -0.5, 1.0 / 3.0)
    got = seq.gla_scan(*cols(big.to(DEV)), zb.to(DEV), sg, bt[DEV][0],
                       bt[DEV][1], Dk ** -0.5, 1.0 / 3.0)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(sg.cpu(), sc, rtol=1e-5, atol=1e-5)
    untouched = [s for s in range(4) if s not in slots]
    torch.testing.assert_close(sg.cpu()[untouched], st0[untouched], rtol=0,
                               atol=0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("groups,gs,shared,act", [
    (4, 32, True, "silu"), (3, 20, True, "sigmoid"), (6, 70, False, "silu"),
    (1, 600, True, "silu")])
def test_group_rmsnorm_gate_forms(dt, groups, gs, shared, act):
    N, D = 9, groups * gs
    y = rnd(N, D)
    w = rnd(gs if shared else D).abs() + 0.5
    gbig = rnd(N, D + 8, dt=dt)
    want = R.group_rmsnorm(y, w, groups, 1e-5, dt, gbig[:, 3:3 + D], act)
    got = seq.group_rmsnorm(y.to(DEV), w.to(DEV), groups, 1e-5, dt,
                            gbig.to(DEV)[:, 3:3 + D], act)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    want = R.group_rmsnorm(y, w, groups, 1e-5, dt)
    got = seq.group_rmsnorm(y.to(DEV), w.to(DEV), groups, 1e-5, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_clamped_glu_and_scaled_joins(dt):
    N, F = 11, 72
    gu = rnd(N, 2 * F + 4, dt=dt, scale=2.0)
    want = R.clamped_glu(gu[:, :F], gu[:, F:2 * F], 1.25, 1.702, 1.0)
    gd = gu.to(DEV)
    got = seq.clamped_glu(gd[:, :F], gd[:, F:2 * F], 1.25, 1.702, 1.0)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    D = 200
    res, y, w = rnd(N, D), rnd(N, D, dt=dt), rnd(D).abs() + 0.5
    ex, exv = rnd(N, D), rnd(D)
    r0, r1 = res.clone(), res.clone().to(DEV)
    want = R.add_rmsnorm_f32res(r0, y, w, 1e-6, dt, 0.0, 0.5, ex, exv)
    got = seq.add_rmsnorm_f32res(r1, y.to(DEV), w.to(DEV), 1e-6, dt, 0.0, 0.5,
                                 ex.to(DEV), exv.to(DEV))
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-6, atol=1e-6)
    got = seq.add_rmsnorm_f32res(r1, None, w.to(DEV), 1e-6, dt,
                                 extra_vec=exv.to(DEV))
    want = R.add_rmsnorm_f32res(r0, None, w, 1e-6, dt, extra_vec=exv)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-6, atol=1e-6)
    x = seq.residual_add_cast(r1, y.to(DEV), dt, scale=0.3)
    xw = R.residual_add_cast(r0, y, dt, scale=0.3)
    torch.testing.assert_close(x.cpu().float(), xw.float(), **tol(dt))
    seq.add_scaled_unit_rms(r1, y.to(DEV), w.to(DEV), 1e-6, scale=0.7)
    R.add_scaled_unit_rms(r0, y, w, 1e-6, scale=0.7)
    torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)
    w2 = rnd(D).abs() + 0.5
    for e1, e2 in ((ex, exv), (None, exv), (None, None)):
        gd = lambda t: None if t is None else t.to(DEV)
        got = seq.add_unit_rms_then_norm(r1, y.to(DEV), w.to(DEV), w2.to(DEV),
                                         1e-6, dt, 0.0, 0.4, gd(e1), gd(e2))
        want = R.add_unit_rms_then_norm(r0, y, w, w2, 1e-6, dt, 0.0, 0.4, e1,
                                        e2)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
        torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,coef,every,lens,starts", [
    (4, 2, 24, 24, 0.4, 7, [5, 1, 3], [0, 37, 6]),
    (6, 3, 64, 64, 0.0, 1, [40, 1, 1, 2], [3, 70, 0, 15]),
    (4, 1, 16, 40, 1.5, 1, [5, 1, 30], [0, 37, 6]),
    (6, 2, 96, 96, 0.3, 64, [70, 1, 130], [10, 300, 0]),
    (3, 3, 200, 72, 0.2, 3, [6, 2], [0, 9]),
    (4, 4, 32, 8, 0.5, 16, [1, 1, 1], [0, 31, 200]),
])
def test_causal_attention_with_sink_and_temperature(dt, H, G, D, Dv, coef,
                                                    every, lens, starts):
    from polyrl_amd.models.hybrid import UNBOUNDED
    page = 4
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, G * (D + Dv), dt)
    N = sum(lens)
    q = rnd(N, H * D, dt=dt, scale=2.5)
    sink = rnd(H, scale=3.0)
    scale = 1.0 / math.sqrt(D)
    want = R.gqa_window_attention(q, cache, ptab, sot, pos, H, G, D, Dv,
                                  UNBOUNDED, 0, None, None, None, scale, dt,
                                  sink, coef, every)
    plain = R.gqa_window_attention(q, cache, ptab, sot, pos, H, G, D, Dv,
                                   UNBOUNDED, 0, None, None, None, scale, dt)
    assert float((want.float() - plain.float()).abs().max()) > 0.05
    g = lambda t: t.to(DEV)
    tiles = seq.attention_tiles(lens, DEV)
    for tl in (None, tiles):                 # one wave per row; matrix cores
        got = seq.gqa_window_attention(
            g(q), g(cache), g(ptab), g(sot), g(pos), H, G, D, Dv, UNBOUNDED,
            0, None, None, None, scale, dt, tiles=tl, sink=g(sink),
            q_temp_coef=coef, q_temp_every=every)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


# ------------------------------------------- gated joints, recurrence, options
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("D", [48, 200, 2048])
def test_gated_add_layernorm(dt, D):
    N = 9
    res = rnd(N, D) + 0.7                    # a mean that matters
    big = rnd(N, 4 * D + 8, dt=dt)
    y1, g1 = big[:, 3:3 + D], big[:, 3 + D:3 + 2 * D]
    y2, g2 = big[:, 5 + 2 * D:5 + 3 * D], big[:, 5 + 3 * D:5 + 4 * D]
    w1, w2 = rnd(D) + 1, rnd(D) + 1
    g = lambda t: None if t is None else t.to(DEV)
    bg = big.to(DEV)
    dv = lambda t: None if t is None else \
        bg[:, t.storage_offset():t.storage_offset() + D]
    for a1, b1, a2, b2, wa, wb in [(y1, g1, y2, g2, w1, w2),
                                   (y1, g1, None, None, w1, None),
                                   (y1, None, y2, g2, w1, w2),
                                   (None, None, None, None, w1, w2),
                                   (y1, g1, y2, None, None, None)]:
        r0, r1 = res.clone(), res.clone().to(DEV)
        want = R.gated_add_layernorm(r0, a1, b1, a2, b2, wa, wb, 1e-5, dt)
        got = seq.gated_add_layernorm(r1, dv(a1), dv(b1), dv(a2), dv(b2),
                                      g(wa), g(wb), 1e-5, dt)
        torch.testing.assert_close(r1.cpu(), r0, rtol=1e-5, atol=1e-5)
        for x, y in zip(got, want):
            assert (x is None) == (y is None)
            if x is not None:
                torch.testing.assert_close(x.cpu().float(), y.float(),
                                           **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("B,bw,lens,max_rows", [
    (5, 8, [5, 1, 2, 9], 9), (1, 300, [3, 1], 0), (7, 1, [2, 2, 1, 7], 7),
    (3, 24, [300, 1, 70], 300), (2, 160, [257, 256], 0)])
def test_rglru_scan(dt, B, bw, lens, max_rows):
    C = B * bw
    slots = [3, 0, 5, 1][:len(lens)]
    bt = batch(lens, slots)
    N = sum(lens)
    big = rnd(N, 2 * C + 11, dt=dt)
    u, y = big[:, 4:4 + C], big[:, 9 + C:9 + 2 * C]
    gates, gb = rnd(B, N, 2 * bw), rnd(B, 2 * bw)
    lam = rnd(C) - 3.0
    st0 = rnd(6, C)
    s0, s1 = st0.clone(), st0.clone().to(DEV)
    cu, sl, _ = bt["cpu"]
    want = R.rglru_scan(u, gates, gb, lam, y, s0, cu, sl, 8.0, dt)
    cu, sl, _ = bt[DEV]
    bg = big.to(DEV)
    got = seq.rglru_scan(bg[:, 4:4 + C], gates.to(DEV), gb.to(DEV),
                         lam.to(DEV), bg[:, 9 + C:9 + 2 * C], s1, cu, sl, 8.0,
                         dt, max_rows=max_rows)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    torch.testing.assert_close(s1.cpu(), s0, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("inter", [False, True])
def test_rotation_pairs_and_amplitude(dt, inter):
    lens, starts, page = [5, 1, 3], [0, 37, 6], 4
    R_, rd, H, D = 24, 12, 3, 10
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, R_ + rd, dt)
    N = sum(lens)
    inv = torch.rand(4)
    q = rnd(N, H, D + rd, dt=dt)
    want = R.rope_partial_(q.clone(), D, inv, pos, 1.13, inter)
    got = seq.rope_partial_(q.clone().to(DEV), D, inv.to(DEV), pos.to(DEV),
                            1.13, inter)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    dkv, w = rnd(N, R_ + rd + 3, dt=dt), rnd(R_) + 1
    c0, c1 = cache.clone(), cache.clone().to(DEV)
    R.latent_kv_store(dkv[:, :R_ + rd], R_, w, 1e-5, pos, inv, c0, slot, 1.13,
                      inter)
    seq.latent_kv_store(dkv.to(DEV)[:, :R_ + rd], R_, w.to(DEV), 1e-5,
                        pos.to(DEV), inv.to(DEV), c1, slot.to(DEV), 1.13,
                        inter)
    torch.testing.assert_close(c1.cpu().float(), c0.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,half,cap,lens,starts", [
    (4, 2, 24, 24, 4, 5.0, [5, 1, 3], [0, 37, 6]),
    (6, 1, 96, 96, 48, 30.0, [70, 1, 1, 2], [3, 300, 0, 15]),
    (4, 4, 16, 40, 0, 0.0, [5, 1, 130], [0, 37, 6]),
    (2, 2, 128, 128, 16, 8.0, [64, 1, 65], [10, 200, 0]),
    (3, 3, 10, 6, 1, 2.0, [6, 2], [0, 9]),
    (8, 2, 32, 80, 16, 12.0, [1, 1, 1], [0, 31, 200]),
    (8, 8, 32, 32, 8, 6.0, [130, 2, 67], [0, 40, 64]),
])
def test_sigmoid_weight_attention_with_rotated_values(dt, H, G, D, Dv, half,
                                                      cap, lens, starts):
    """Writer: per-head unit norm after the rotation, values rotated by
    their positions.  Attention: capped scores, per-head bias, sigmoid
    weights without normalisation, head sums turned back; one wave per row
    and the matrix-core kernel."""
    page = 4
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, G * (D + Dv), dt)
    # every cached position of every sequence gets a proper row first
    all_lens = [s + n for s, n in zip(starts, lens)]
    pos2 = torch.tensor([p for n in all_lens for p in range(n)],
                        dtype=torch.int32)
    slot2 = torch.tensor([int(ptab[b, p // page]) * page + p % page
                          for b, n in enumerate(all_lens) for p in range(n)],
                         dtype=torch.int32)
    N2 = sum(all_lens)
    inv = torch.rand(half) if half else None
    vinv = seq.rope_inv_freq(Dv, 50.0, "cpu")
    kv = rnd(N2, G * D + G * Dv + H * D, dt=dt)
    c0, c1 = cache.clone(), cache.clone().to(DEV)
    g = lambda t: None if t is None else t.to(DEV)
    a, b = G * D, G * D + G * Dv
    q0 = R.gqa_prepare_store(kv[:, b:], kv[:, :a], kv[:, a:b], None, None,
                             1e-5, inv, 1.0, pos2, c0, slot2, H, G, D, Dv,
                             True, vinv)
    kd = kv.to(DEV)
    q1 = seq.gqa_prepare_store(kd[:, b:], kd[:, :a], kd[:, a:b], None, None,
                               1e-5, g(inv), 1.0, g(pos2), c1, g(slot2), H, G,
                               D, Dv, True, g(vinv))
    torch.testing.assert_close(q1.cpu().float(), q0.float(), **tol(dt))
    torch.testing.assert_close(c1.cpu().float(), c0.float(), **tol(dt))
    # the queries of this step's rows
    rows = torch.cat([torch.arange(s, s + n) + sum(all_lens[:i])
                      for i, (s, n) in enumerate(zip(starts, lens))])
    q = q0[rows].contiguous()
    pb = rnd(H) - 2.0
    gfull = rnd(len(rows), H + 3, dt=dt)
    scale = 4.0 / math.sqrt(D)
    for gate in (None, gfull[:, 1:1 + H]):
        want = R.gqa_window_attention(
            q, c0, ptab, sot, pos, H, G, D, Dv, 1 << 30, 0, None, None, gate,
            scale, dt, softcap=cap, head_bias=pb, sigmoid_weights=True,
            v_inv_freq=vinv)
        for tl in (None, seq.attention_tiles(lens, DEV)):
            got = seq.gqa_window_attention(
                g(q), g(c0), g(ptab), g(sot), g(pos), H, G, D, Dv, 1 << 30, 0,
                None, None,
                None if gate is None else gfull.to(DEV)[:, 1:1 + H], scale,
                dt, tiles=tl, softcap=cap, head_bias=g(pb),
                sigmoid_weights=True, v_inv_freq=g(vinv))
            ref = want.float()
            lim = dict(rtol=2e-2, atol=2e-2 * float(ref.abs().max())) \
                if dt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
            torch.testing.assert_close(got.cpu().float(), ref, **lim)


@pytest.mark.parametrize("dt", DTYPES)
def test_head_gate_and_causal_latent_attention_without_sink(dt):
    N, H, Dv = 11, 5, 12
    big, gate = rnd(N, H * Dv + 4, dt=dt), rnd(N, H + 2, dt=dt)
    want = R.sigmoid_mul_heads(big[:, 2:2 + H * Dv], gate[:, 1:1 + H])
    got = seq.sigmoid_mul_heads(big.to(DEV)[:, 2:2 + H * Dv],
                                gate.to(DEV)[:, 1:1 + H])
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    lens, starts, page = [70, 1, 3], [5, 300, 0], 4
    R_, rd, H = 32, 8, 4
    cache, ptab, pos, sot, slot = _paged(lens, starts, page, R_ + rd, dt)
    ql, qr = rnd(sum(lens), H, R_, dt=dt), rnd(sum(lens), H, rd, dt=dt)
    want = R.latent_window_attention(ql, qr, cache, ptab, sot, pos, 1 << 30,
                                     None, 0.3, dt)
    g = lambda t: t.to(DEV)
    for tl in (None, seq.attention_tiles(lens, DEV)):
        got = seq.latent_window_attention(g(ql), g(qr), g(cache), g(ptab),
                                          g(sot), g(pos), 1 << 30, None, 0.3,
                                          dt, tiles=tl)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))


@pytest.mark.parametrize("N,top,E", [(1, 2, 4), (37, 3, 5), (200, 4, 8)])
def test_gated_routed_experts_bf16(N, top, E):
    dt = torch.bfloat16
    Wd, ff = 96, 64
    h = rnd(N, Wd, dt=dt)
    idx = torch.stack([torch.randperm(E)[:top] for _ in range(N)]).int()
    w = torch.rand(N, top)
    gu, down = rnd(E, 2 * ff, Wd, dt=dt, scale=0.1), \
        rnd(E, Wd, ff, dt=dt, scale=0.1)
    ys0 = R.moe_routed_ffn(h, idx, gu, down, True)
    assert seq.moe_routed_ffn_supported(h.to(DEV), top, ff)
    ys1 = seq.moe_routed_ffn(h.to(DEV), idx.to(DEV), gu.to(DEV), down.to(DEV),
                             True)
    torch.testing.assert_close(ys1.cpu().float(), ys0.float(), **tol(dt))
    want = R.moe_weighted_combine(ys0, idx, w, h, None, E, 1e-20, dt, 1.75)
    got = seq.moe_weighted_combine(ys1, idx.to(DEV), w.to(DEV), h.to(DEV),
                                   None, E, 1e-20, dt, 1.75)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
