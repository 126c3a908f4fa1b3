"""Each mechanism that the Bogupel layers add to the layer-list worker alone, through its C-ABI op, against the float64 functions of
tests/bogupel_oracle.py: the Dynamic Tanh norm (store / behind a residual update), the start of a looped pass, the scaled pair embedding with
its second copy, the query / key / value writer with normed and turned values, attention over turned values with a window and learned sinks
and the turn back (tiled and single-row forms, portions, window edges), the gates and the scan of the generalized delta rule (register and
LDS forms, continued states, several sequences, reused slots), the router on sigmoid scores and the clamped gated experts in both forms."""
import ctypes as C

import numpy as np
import pytest
import torch

import inferflow_amd as ia
from tests import bogupel_oracle as orc
from tests.gelarax_oracle import bf16_round
from tests.gpu_util import capi, p, sync
from tests.test_gpu_layered_ops import Slots, dev32, devbf, devi, seq_tables

pytestmark = pytest.mark.gpu


def host_seqs(seqs):
    h, r = [], 0
    for n, pos0, slot in seqs:
        h += [r, n, pos0, slot]; r += n
    return (C.c_int * len(h))(*h)


def dev64(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float64)).cuda()


@pytest.mark.parametrize("rows,cols", [(1, 64), (5, 96), (33, 40), (3, 14), (2, 5000)])
def test_dynamic_tanh_store_after_an_update_and_the_start_of_a_pass(rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (3 * rng.standard_normal((rows, cols + 3))).astype(np.float32)
    m = rng.standard_normal((rows, cols + 2)).astype(np.float32)
    w, b, alpha = bf16_round(1 + 0.3 * rng.standard_normal(cols)), bf16_round(0.3 * rng.standard_normal(cols)), bf16_round(np.asarray([0.37]))
    L = capi()
    want = orc.dyt(orc.f64(x[:, :cols]), alpha, orc.f64(w), orc.f64(b))
    y = torch.full((rows, cols + 1), 7.0, dtype=torch.float32, device="cuda")
    ia.check(L.ifa_dyt_f32(p(dev32(x)), cols + 3, rows, cols, p(devbf(alpha)), p(devbf(w)), p(devbf(b)), p(y), cols + 1, None)); sync()
    got = y.cpu().numpy()
    assert np.abs(got[:, :cols] - want).max() < 2e-6 * max(1.0, np.abs(want).max()) and np.all(got[:, cols:] == 7.0)
    # x += m; h = dyt(x)
    xd, h = dev32(x), torch.full((rows, cols), 7.0, dtype=torch.float32, device="cuda")
    ia.check(L.ifa_add_dyt_f32(p(xd), cols + 3, rows, cols, p(dev32(m)), cols + 2, None, p(devbf(alpha)), p(devbf(w)), p(devbf(b)), p(h), cols, None)); sync()
    xs = x[:, :cols] + m[:, :cols]
    assert np.array_equal(xd.cpu().numpy()[:, :cols], xs) and np.array_equal(xd.cpu().numpy()[:, cols:], x[:, cols:])
    want2 = orc.dyt(orc.f64(xs), alpha, orc.f64(w), orc.f64(b))
    assert np.abs(h.cpu().numpy() - want2).max() < 2e-6 * max(1.0, np.abs(want2).max())
    # x += x0 + step; x += step alone
    step = bf16_round(rng.standard_normal(cols))
    for with_rows in (1, 0):
        xd = dev32(x)
        ia.check(L.ifa_add_rows_vec_f32(p(xd), cols + 3, rows, cols, p(dev32(m)) if with_rows else None, cols + 2, p(devbf(step)), None)); sync()
        ref = x[:, :cols] + (m[:, :cols] if with_rows else 0) + step
        assert np.abs(xd.cpu().numpy()[:, :cols] - ref).max() < 1e-6 * max(1.0, np.abs(ref).max()) and np.array_equal(xd.cpu().numpy()[:, cols:], x[:, cols:])


def test_scaled_pair_embedding_with_its_copy_in_portions():
    rng = np.random.default_rng(1)
    V, W, B, mp, mc, scale = 37, 20, 11, 29, 3, 2.5
    E, P = bf16_round(rng.standard_normal((V, W))), bf16_round(rng.standard_normal((B + 1, W)))
    cfg = {"embedding": {"scale": scale, "bigram": {"buckets": B, "mul_prev": mp, "mul_cur": mc}}}
    toks = [int(t) for t in rng.integers(0, V, 23)]
    want = orc.embed(cfg, {"embed": orc.f64(E), "bigram": orc.f64(P)}, toks)
    L = capi()
    slots = Slots(2, 8)
    at = 0
    for n in (1, 2, 9, 1, 10):
        sd, rs, rows = seq_tables([(n, at, 1)])
        x = torch.zeros((rows, W), dtype=torch.float32, device="cuda")
        x2 = torch.zeros((rows, W), dtype=torch.float32, device="cuda")
        ia.check(L.ifa_embed_pair_scaled_f32(p(devbf(E)), V, W, scale, p(devbf(P)), B, mp, mc, p(devi(toks[at:at + n])), p(sd), p(rs), rows, p(slots.table), 4, p(x),
                                             p(x2) if n != 9 else None, None)); sync()
        assert np.abs(x.cpu().numpy() - want[at:at + n]).max() < 1e-6 * np.abs(want).max(), (at, n)
        assert n == 9 or torch.equal(x, x2)
        at += n


def attention_case(heads, kv_heads, dim, vdim, L, rng):
    q = rng.standard_normal((L, heads * dim)).astype(np.float32)
    k = rng.standard_normal((L, kv_heads * dim)).astype(np.float32)
    v = (2 * rng.standard_normal((L, kv_heads * vdim))).astype(np.float32)
    qw, kw = bf16_round(1 + 0.3 * rng.standard_normal(dim)), bf16_round(1 + 0.3 * rng.standard_normal(dim))
    return q, k, v, qw, kw


def oracle_attention(q, k, v, qw, kw, sink, heads, kv_heads, dim, vdim, fr, fv, scale, window, eps):
    """the attention core from the oracle's pieces: normed and turned queries / keys, normed and turned values, windowed softmax with the sinks,
    the turn back"""
    T = q.shape[0]
    pos = np.arange(T)
    qq = orc.turn(orc.rms_unit(orc.f64(q).reshape(T, heads, dim), eps) * orc.f64(qw), pos, fr)
    kk = orc.turn(orc.rms_unit(orc.f64(k).reshape(T, kv_heads, dim), eps) * orc.f64(kw), pos, fr)
    vv = orc.turn(orc.rms_unit(orc.f64(v).reshape(T, kv_heads, vdim), eps), pos, fv)
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i) & (i - j < window)
    out = np.zeros((T, heads, vdim))
    for h in range(heads):
        g = h // (heads // kv_heads)
        sc = np.where(seen, (qq[:, h] @ kk[:, g].T) * scale, -np.inf)
        out[:, h] = orc.softmax_with_sink(sc, float(sink[h]) if sink is not None else -np.inf) @ vv[:, g]
    return orc.turn(out, pos, fv, sign=-1.0).reshape(T, heads * vdim)


@pytest.mark.parametrize("tile_min", [16, 1 << 30])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot_dims,window", [(4, 2, 24, 16, 24, 40), (2, 2, 8, 40, 4, 1000), (3, 1, 68, 36, 30, 33), (6, 3, 32, 32, 0, 64),
                                                                     (2, 1, 128, 128, 128, 65), (1, 1, 5, 2, 2, 1), (8, 2, 96, 8, 64, 31), (2, 1, 160, 20, 100, 77),
                                                                     (2, 1, 16, 200, 8, 50)])
def test_attention_over_turned_values_with_window_and_sinks_in_portions(heads, kv_heads, dim, vdim, rot_dims, window, tile_min):
    rng = np.random.default_rng(heads + dim + vdim)
    L, eps, scale, base, ctx = 150, 1e-5, 0.3, 300.0, 160
    q, k, v, qw, kw = attention_case(heads, kv_heads, dim, vdim, L, rng)
    sink = bf16_round(np.linspace(-2.0, 2.5, heads) + 0.2 * rng.standard_normal(heads)) if heads > 1 else bf16_round(np.asarray([1.25]))
    # the last row's query matches the key just inside the window and the key just outside it (directions count: the norm follows)
    for far in (window - 1, window):
        if 0 < far < L:
            k[L - 1 - far, :dim] = 5 * q[L - 1, :dim]
    scaling = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    fr, fv = orc.frequencies(base, rot_dims, scaling), orc.frequencies(base, vdim)
    want = oracle_attention(q, k, v, qw, kw, sink, heads, kv_heads, dim, vdim, fr, fv, scale, window, eps)
    frd, fvd = dev64(fr if len(fr) else [0.0]), dev64(fv)
    k_off, v_off = 4, 4 + ((ctx * kv_heads * dim + 3) // 4) * 4
    sl = Slots(2, v_off + ctx * kv_heads * vdim)
    ws = torch.full((2 * heads * 32 * (vdim + 2),), float('nan'), dtype=torch.float32, device='cuda')
    Lc = capi()
    at = 0
    for n in (1, 2, 60, 1, 1, 80, 3, 2):
        d, rs, T = seq_tables([(n, at, 1)])
        qd, kd, vd = dev32(q[at:at + n]), dev32(k[at:at + n]), dev32(v[at:at + n])
        ia.check(Lc.ifa_qkv_rope_store_f32(p(qd), heads * dim, heads, p(kd), kv_heads * dim, p(vd), kv_heads * vdim, kv_heads, dim, vdim, p(devbf(qw)), p(devbf(kw)), eps,
                                           rot_dims, p(frd), 1, p(fvd), p(d), p(rs), T, p(sl.table), k_off, v_off, None))
        out = torch.empty((T, heads * vdim + 1), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_sinks_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, scale, window, 0, p(devbf(sink)), p(d), p(rs), T, p(sl.table), k_off, v_off,
                                               p(out), heads * vdim + 1, host_seqs([(n, at, 1)]), 1, tile_min, ctx, p(ws) if n <= 2 else None, ws.numel() * 4, None))
        ia.check(Lc.ifa_rotate_heads_f32(p(out), heads * vdim + 1, heads, vdim, vdim, p(fvd), -1.0, p(d), p(rs), T, None))
        sync()
        assert np.abs(out.cpu().numpy()[:, :heads * vdim] - want[at:at + n]).max() < 3e-5 * max(1.0, np.abs(want).max()), (at, n)
        at += n
    assert at == L
    # the sinks are really counted, per query head: without them, and with them in another order, the last row differs
    d, rs, T = seq_tables([(1, L - 1, 1)])
    qd = dev32(q[L - 1:])
    ia.check(Lc.ifa_qkv_rope_store_f32(p(qd), heads * dim, heads, None, 0, None, 0, kv_heads, dim, vdim, p(devbf(qw)), None, eps, rot_dims, p(frd), 1, p(fvd), p(d), p(rs), T,
                                       p(sl.table), k_off, v_off, None))
    res = []
    for sk in (sink, None, sink[::-1].copy()):
        out = torch.empty((1, heads * vdim), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_sinks_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, 0.01, window, 0, p(devbf(sk)) if sk is not None else None, p(d), p(rs), T,
                                               p(sl.table), k_off, v_off, p(out), heads * vdim, None, 0, 0, ctx, None, 0, None))
        ia.check(Lc.ifa_rotate_heads_f32(p(out), heads * vdim, heads, vdim, vdim, p(fvd), -1.0, p(d), p(rs), T, None))
        sync(); res.append(out.cpu().numpy())
    flat = oracle_attention(q, k, v, qw, kw, sink, heads, kv_heads, dim, vdim, fr, fv, 0.01, window, eps)
    assert np.abs(res[0] - flat[L - 1:]).max() < 3e-5 * max(1.0, np.abs(flat).max())
    assert np.abs(res[1] - res[0]).max() > 1e-4
    assert heads == 1 or np.abs(res[2] - res[0]).max() > 1e-4


def test_values_as_projected_when_neither_normed_nor_turned():
    """the writer with both treatments off leaves the values as they are, with them on one at a time it matches the oracle's pieces"""
    rng = np.random.default_rng(5)
    heads, kv_heads, dim, vdim, T, eps = 2, 2, 8, 6, 5, 1e-5
    q, k, v, qw, kw = attention_case(heads, kv_heads, dim, vdim, T, rng)
    fv = orc.frequencies(100.0, vdim)
    Lc = capi()
    for norm, rot in ((0, 0), (1, 0), (0, 1)):
        sl = Slots(1, 2 * 16 * kv_heads * max(dim, vdim))
        d, rs, rows = seq_tables([(T, 3, 0)])
        v_off = 16 * kv_heads * dim
        ia.check(Lc.ifa_qkv_rope_store_f32(p(dev32(q)), heads * dim, heads, p(dev32(k)), kv_heads * dim, p(dev32(v)), kv_heads * vdim, kv_heads, dim, vdim, p(devbf(qw)),
                                           p(devbf(kw)), eps, 0, None, norm, p(dev64(fv)) if rot else None, p(d), p(rs), rows, p(sl.table), 0, v_off, None)); sync()
        got = sl.mem[0].cpu().numpy()[v_off + 3 * kv_heads * vdim: v_off + (3 + T) * kv_heads * vdim].reshape(T, kv_heads, vdim)
        want = orc.f64(v).reshape(T, kv_heads, vdim)
        if norm:
            want = orc.rms_unit(want, eps)
        if rot:
            want = orc.turn(want, np.arange(3, 3 + T), fv)
        assert np.abs(got - want).max() < 2e-6 * np.abs(want).max(), (norm, rot)


@pytest.mark.parametrize("H,D", [(3, 16), (2, 32), (5, 48), (2, 64), (1, 96), (2, 128), (2, 4), (3, 5), (1, 72), (2, 130)])
def test_generalized_delta_rule_gates_and_scan(H, D):
    """whole sequences, portions down to one and two tokens, several sequences in a launch, a continued state and a slot that is used again"""
    rng = np.random.default_rng(H * 100 + D)
    T, R, Wd = 61, 5, 24
    C_ = H * D
    names = ("r", "k", "v", "a", "lr")
    seqs = {s: {n: rng.standard_normal((T, R if n == "lr" else C_)).astype(np.float32) for n in names} for s in (0, 1, 2)}
    w2, w0 = bf16_round(rng.standard_normal((C_, R))), bf16_round(1.5 * rng.standard_normal(C_))
    if D >= 16:          # decays close to one and small removal rates in one head: its state remembers the first tokens
        w0[:D] = -7.0
        for s in seqs.values():
            s["a"][:, :D] -= 4.0

    def want_of(s):
        decay = np.exp(-np.exp(-0.5) * orc.logistic(np.tanh(orc.f64(s["lr"])) @ orc.f64(w2).T + orc.f64(w0))).reshape(T, H, D)
        rate = orc.logistic(orc.f64(s["a"])).reshape(T, H, D)
        r, k, v = (orc.f64(s[n]).reshape(T, H, D) for n in ("r", "k", "v"))
        return np.stack([orc.delta_scan(r[:, h], k[:, h], v[:, h], decay[:, h], rate[:, h])[0] for h in range(H)], 1).reshape(T, C_)
    want = {s: want_of(seqs[s]) for s in seqs}
    Lc = capi()
    off = 8
    sl = Slots(2, off + H * D * D)
    at = {0: 0, 1: 0, 2: 0}
    # sequence 2 starts on slot 1 after sequence 1 has ended there
    plan = [[(0, 1, 0)], [(0, 2, 0), (1, 30, 1)], [(0, 9, 0), (1, 31, 1)], [(2, 1, 1), (0, 17, 0)], [(2, 2, 1)], [(0, 32, 0), (2, 58, 1)]]
    for step in plan:
        d, rs, rows = seq_tables([(n, at[q], slot) for q, n, slot in step])
        cat = {n: np.concatenate([seqs[q][n][at[q]:at[q] + cnt] for q, cnt, _ in step], 0) for n in names}
        dec, unit, rem = (torch.empty((rows, C_), dtype=torch.float32, device="cuda") for _ in range(3))
        kd = dev32(cat["k"])
        ia.check(Lc.ifa_chan_delta_gates_f32(p(dev32(cat["lr"])), R, R, p(devbf(w2)), p(devbf(w0)), float(np.exp(-0.5)), p(dev32(cat["a"])), C_, p(kd), C_, H, D, 1e-6, rows,
                                             p(dec), p(unit), p(rem), None))
        out = torch.empty((rows, C_ + 1), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_state_scan_chan_f32(p(dev32(cat["r"])), C_, p(kd), C_, p(dev32(cat["v"])), C_, H, D, D, p(dec), p(unit), p(rem), C_, p(d), len(step), p(sl.table), off,
                                            p(out), C_ + 1, None))
        sync()
        got, r0 = out.cpu().numpy()[:, :C_], 0
        for q, cnt, _ in step:
            ref = want[q][at[q]:at[q] + cnt]
            assert np.abs(got[r0:r0 + cnt] - ref).max() < 1e-4 * max(1.0, np.abs(want[q]).max()), (q, at[q], cnt)
            r0 += cnt; at[q] += cnt
    assert at == {0: 61, 1: 61, 2: 61}
    # the gates themselves, on the last step's rows of sequence 0
    k0 = orc.f64(seqs[0]["k"][29:61]).reshape(32, H, D)
    u = k0 / np.sqrt((k0 * k0).sum(-1, keepdims=True) + 1e-6)
    assert np.abs(unit.cpu().numpy()[:32] - u.reshape(32, C_)).max() < 1e-6
    assert np.abs(rem.cpu().numpy()[:32] - (orc.logistic(orc.f64(seqs[0]["a"][29:61])).reshape(32, H, D) * u).reshape(32, C_)).max() < 1e-6


def test_the_slow_head_remembers_the_first_token():
    """with decays near one the first token's write still shows 60 tokens later in the oracle, so the scan's carried state is what is tested"""
    rng = np.random.default_rng(3)
    T, D = 61, 16
    r, k, v = (rng.standard_normal((T, D)) for _ in range(3))
    decay, rate = np.full((T, D), 0.999), np.full((T, D), 0.02)
    a, _ = orc.delta_scan(r, k, v, decay, rate)
    v2 = v.copy(); v2[0] += 1.0
    b, _ = orc.delta_scan(r, k, v2, decay, rate)
    assert np.abs(a[-1] - b[-1]).max() > 1e-2
    # carried state: two halves equal the whole
    h1, S = orc.delta_scan(r[:30], k[:30], v[:30], decay[:30], rate[:30])
    h2, _ = orc.delta_scan(r[30:], k[30:], v[30:], decay[30:], rate[30:], S)
    assert np.abs(np.concatenate([h1, h2]) - a).max() < 1e-12


@pytest.mark.parametrize("n_all,top", [(6, 2), (16, 1), (5, 5), (70, 8), (3, 2)])
def test_router_on_sigmoid_scores_with_correction_and_ties(n_all, top):
    rng = np.random.default_rng(n_all + top)
    T, W = 9, 40
    h = rng.standard_normal((T, W)).astype(np.float32)
    router = bf16_round(rng.standard_normal((n_all, W)) * 0.4)
    corr = bf16_round(0.3 * rng.standard_normal(n_all))
    if n_all >= 5:
        router[3] = router[1]; corr[3] = corr[1]          # a tie: the lower index wins
    idx_w, wgt_w = orc.route(orc.f64(h), orc.f64(router), orc.f64(corr), top)
    L = capi()
    logits = (orc.f64(h) @ orc.f64(router).T).astype(np.float32)
    for form in ("logits", "rows"):
        idx = torch.full((T, top), -1, dtype=torch.int32, device="cuda")
        wgt = torch.zeros((T, top), dtype=torch.float32, device="cuda")
        if form == "logits":
            ia.check(L.ifa_moe_route_scores_f32(1, p(dev32(logits)), n_all, T, n_all, top, p(devbf(corr)), p(idx), p(wgt), None))
        else:
            ia.check(L.ifa_moe_route_rows_scores_f32(1, p(dev32(h)), W, T, W, p(devbf(router)), n_all, top, p(devbf(corr)), p(idx), p(wgt), None))
        sync()
        assert np.array_equal(idx.cpu().numpy(), idx_w), form
        assert np.abs(wgt.cpu().numpy() - wgt_w).max() < 2e-6, form
    # the weights are the plain scores: they do not sum to one and do not contain the correction
    assert np.abs(wgt_w - orc.logistic(np.take_along_axis(orc.f64(logits), idx_w, -1))).max() < 1e-6


@pytest.mark.parametrize("T,W,F,E,top,limit", [(1, 64, 24, 6, 2, 1.0), (3, 40, 10, 3, 3, 0.3), (8, 128, 64, 16, 4, 7.0), (9, 64, 24, 6, 2, 1.0), (70, 48, 20, 5, 1, 0.5),
                                               (150, 64, 32, 20, 3, 2.0), (5, 14, 6, 4, 2, 1.5)])
def test_clamped_gated_experts_in_rows_and_grouped(T, W, F, E, top, limit):
    rng = np.random.default_rng(T + W + F)
    h = rng.standard_normal((T, W)).astype(np.float32)
    gate, up, down = (bf16_round(rng.standard_normal(s) * 0.3) for s in ((E, F, W), (E, F, W), (E, W, F)))
    idx = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    wgt = rng.uniform(0.1, 1.0, (T, top)).astype(np.float32)
    want = np.zeros((T, W))
    for t in range(T):
        for e, wv in zip(idx[t], wgt[t]):
            want[t] += wv * orc.clamped_expert(orc.f64(h[t:t + 1]), orc.f64(gate[e]), orc.f64(up[e]), orc.f64(down[e]), limit)[0]
    gu = np.concatenate([gate, up], 1)                     # per expert: its gate rows, then its up rows
    L = capi()
    nb = L.ifa_moe_workspace_bytes(T, top, W, 3 * F, E)
    ws = torch.empty((nb,), dtype=torch.uint8, device="cuda")
    y0 = rng.standard_normal((T, W + 2)).astype(np.float32)
    for ops32, tol in ((1, 2e-5), (0, 3e-2)):
        for acc in (0, 1):
            y = dev32(y0)
            ia.check(L.ifa_moe_experts_glu_f32(3, limit, p(dev32(h)), W, T, W, F, E, top, p(devbf(gu.reshape(E * 2 * F, W))), p(devbf(down.reshape(E * W, F))), p(devi(idx)),
                                               p(dev32(wgt)), ops32, p(ws), nb, p(y), W + 2, acc, None)); sync()
            got = y.cpu().numpy()
            ref = want + (y0[:, :W] if acc else 0)
            t_ = tol if T > 8 else 2e-5
            assert np.abs(got[:, :W] - ref).max() < t_ * max(1.0, np.abs(want).max()), (ops32, acc)
            assert np.array_equal(got[:, W:], y0[:, W:])
