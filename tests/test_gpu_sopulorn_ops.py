"""Each mechanism that the Sopulorn layers add to the layer-list worker alone, through its C-ABI op, against the float64 functions of
tests/sopulorn_oracle.py: the token-pair embedding with its carried previous token, the RMS norm with weight (1 + w) (store / accumulate /
both norms between two sub-layers in one launch), the clamped and the row-gated activations, the query / key norm + rotation + cache
writer, attention over rotated caches with values of their own size, a fixed sink and another layer's rows (tiled and single-row forms,
portions, several sequences, slots reused), the router on logits, and the gated experts in the row form and the grouped form."""
import ctypes as C

import numpy as np
import pytest
import torch

import inferflow_amd as ia
from tests import sopulorn_oracle as orc
from tests.gelarax_oracle import bf16_round
from tests.gpu_util import capi, p, sync
from tests.test_gpu_layered_ops import Slots, dev32, devbf, devi, seq_tables

pytestmark = pytest.mark.gpu


def t64(a):
    return orc.t64(a)


def host_seqs(seqs):
    h, r = [], 0
    for n, pos0, slot in seqs:
        h += [r, n, pos0, slot]; r += n
    return (C.c_int * len(h))(*h)


def test_pair_embedding_in_portions_batches_and_reused_slots():
    rng = np.random.default_rng(1)
    V, W, B, mp, mc = 37, 20, 11, 29, 3
    E, P = bf16_round(rng.standard_normal((V, W))), bf16_round(rng.standard_normal((B + 1, W)))
    L = capi()
    slots = Slots(2, 8)
    seqs = {0: [int(t) for t in rng.integers(0, V, 19)], 1: [int(t) for t in rng.integers(0, V, 7)], 2: [int(t) for t in rng.integers(0, V, 5)]}
    want = {k: (t64(E)[v] + t64(P)[orc.pair_rows(v, B, mp, mc)]).numpy() for k, v in seqs.items()}
    at = {0: 0, 1: 0, 2: 0}
    # sequence 2 starts on slot 1 after sequence 1 has ended there; portions of 1, 2 and more tokens; two sequences in a step
    for step in ([(0, 1, 0)], [(0, 2, 0), (1, 4, 1)], [(0, 1, 0), (1, 3, 1)], [(0, 9, 0), (2, 1, 1)], [(2, 4, 1), (0, 6, 0)]):
        sd, rs, rows = seq_tables([(n, at[q], slot) for q, n, slot in step])
        toks = devi(sum([seqs[q][at[q]:at[q] + n] for q, n, _ in step], []))
        x = torch.zeros((rows, W), dtype=torch.float32, device="cuda")
        ia.check(L.ifa_embed_pair_f32(p(devbf(E)), V, W, p(devbf(P)), B, mp, mc, p(toks), p(sd), p(rs), rows, p(slots.table), 4, p(x), None)); sync()
        got, r = x.cpu().numpy(), 0
        for q, n, _ in step:
            assert np.abs(got[r:r + n] - want[q][at[q]:at[q] + n]).max() < 1e-6, (q, at[q], n)
            r += n; at[q] += n
    # without the table: plain embedding rows
    sd, rs, rows = seq_tables([(3, 0, 0)])
    x = torch.zeros((3, W), dtype=torch.float32, device="cuda")
    ia.check(L.ifa_embed_pair_f32(p(devbf(E)), V, W, None, 0, 0, 0, p(devi(seqs[0][:3])), p(sd), p(rs), 3, p(slots.table), 4, p(x), None)); sync()
    assert np.array_equal(x.cpu().numpy(), E[seqs[0][:3]])


@pytest.mark.parametrize("rows,cols", [(1, 64), (5, 96), (33, 40), (3, 14), (2, 1030)])
def test_norm_with_one_plus_weight_store_accumulate_and_both_in_one_launch(rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols + 3)).astype(np.float32)
    w, w2 = bf16_round(0.3 * rng.standard_normal(cols)), bf16_round(0.3 * rng.standard_normal(cols))
    y0 = rng.standard_normal((rows, cols + 1)).astype(np.float32)
    want = orc.norm_one_plus(t64(x[:, :cols]), t64(w), 1e-5).numpy()
    L = capi()
    for acc in (0, 1):
        xd, yd = dev32(x), dev32(y0)
        ia.check(L.ifa_rmsnorm_offset_f32(p(xd), cols + 3, rows, cols, p(devbf(w)), 1.0, 1e-5, acc, p(yd), cols + 1, None)); sync()
        got = yd.cpu().numpy()
        ref = want + (y0[:, :cols] if acc else 0)
        assert np.abs(got[:, :cols] - ref).max() < 1e-5 * max(1.0, np.abs(ref).max())
        assert np.array_equal(got[:, cols:], y0[:, cols:])
    # x += norm(m) (1 + w); h = norm(x) (1 + w2)
    for with_h in (1, 0):
        xd, md, hd = dev32(y0), dev32(x), torch.full((rows, cols), 7.0, dtype=torch.float32, device="cuda")
        ia.check(L.ifa_norm_add_norm_f32(p(xd), cols + 1, rows, cols, p(md), cols + 3, p(devbf(w)), p(devbf(w2)) if with_h else None, 1.0, 1e-5, p(hd), cols, None)); sync()
        xs = y0[:, :cols] + want
        assert np.abs(xd.cpu().numpy()[:, :cols] - xs).max() < 1e-5 * max(1.0, np.abs(xs).max())
        if with_h:
            hs = orc.norm_one_plus(t64(xs), t64(w2), 1e-5).numpy()
            assert np.abs(hd.cpu().numpy() - hs).max() < 1e-5 * max(1.0, np.abs(hs).max())
        else:
            assert float(hd.min()) == 7.0


def test_clamped_activation_and_row_gate():
    rng = np.random.default_rng(3)
    T, F = 5, 70
    gu = (3.0 * rng.standard_normal((T, 2 * F + 2))).astype(np.float32)
    gate = rng.standard_normal((T, 3)).astype(np.float32)
    L = capi()
    out = torch.zeros((T, F), dtype=torch.float32, device="cuda")
    ia.check(L.ifa_glu_ex_f32(3, 1.25, p(dev32(gu)), 2 * F + 2, T, F, None, 0, p(out), F, None)); sync()
    g, u = t64(gu[:, :F]).clamp(max=1.25), t64(gu[:, F:2 * F]).clamp(-1.25, 1.25)
    assert np.abs(out.cpu().numpy() - (g * torch.sigmoid(1.702 * g) * (u + 1)).numpy()).max() < 1e-5
    assert (np.abs(gu[:, :F]) > 1.25).any() and (gu[:, F:2 * F] < -1.25).any()          # (the clamps are at work)
    ia.check(L.ifa_glu_ex_f32(0, 0.0, p(dev32(gu)), 2 * F + 2, T, F, p(dev32(gate)), 3, p(out), F, None)); sync()
    g, u = t64(gu[:, :F]), t64(gu[:, F:2 * F])
    want = g * torch.sigmoid(g) * u * torch.sigmoid(t64(gate[:, :1]))
    assert np.abs(out.cpu().numpy() - want.numpy()).max() < 1e-5 * float(want.abs().max())


def attention_case(heads, kv_heads, dim, vdim, rot_dims, L, rng, base=300.0):
    q = rng.standard_normal((L, heads * dim)).astype(np.float32)
    k = rng.standard_normal((L, kv_heads * dim)).astype(np.float32)
    v = rng.standard_normal((L, kv_heads * vdim)).astype(np.float32)
    qw, kw = bf16_round(1 + 0.3 * rng.standard_normal(dim)), bf16_round(1 + 0.3 * rng.standard_normal(dim))
    return q, k, v, qw, kw


def oracle_attention(q, k, v, qw, kw, heads, kv_heads, dim, vdim, rot_dims, base, scale, eps):
    T = q.shape[0]
    pos = list(range(T))
    qq = orc.rotate_half_layout(orc.rms_unit(t64(q).reshape(T, heads, dim), eps) * t64(qw), pos, rot_dims, base)
    kk = orc.rotate_half_layout(orc.rms_unit(t64(k).reshape(T, kv_heads, dim), eps) * t64(kw), pos, rot_dims, base)
    return orc.attention_core(qq, kk, t64(v).reshape(T, kv_heads, vdim), scale).numpy()


def freq_table(rot_dims, base):
    return torch.from_numpy(np.asarray([base ** (-2.0 * i / max(rot_dims, 1)) for i in range(max(rot_dims // 2, 1))], np.float64)).cuda()


@pytest.mark.parametrize("tile_min", [16, 1 << 30])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot_dims", [(4, 2, 24, 16, 24), (2, 2, 8, 40, 4), (3, 1, 68, 36, 30), (6, 3, 32, 32, 0), (2, 1, 128, 128, 128),
                                                              (4, 1, 40, 72, 40), (1, 1, 5, 3, 2), (8, 2, 96, 8, 64), (2, 1, 160, 20, 100), (2, 1, 320, 24, 200)])
def test_rotated_attention_in_portions_and_single_rows(heads, kv_heads, dim, vdim, rot_dims, tile_min):
    rng = np.random.default_rng(heads + dim + vdim)
    L, eps, scale, base, ctx = 150, 1e-5, 0.3, 300.0, 160
    q, k, v, qw, kw = attention_case(heads, kv_heads, dim, vdim, rot_dims, L, rng)
    # one key far back and the very first one get large matching queries at the last rows (before the norm: directions count)
    k[1, :dim] = 5 * rng.standard_normal(dim); q[-1, :dim] = k[1, :dim]
    want = oracle_attention(q, k, v, qw, kw, heads, kv_heads, dim, vdim, rot_dims, base, scale, eps)
    fr = freq_table(rot_dims, base)
    k_off, v_off = 4, 4 + ((ctx * kv_heads * dim + 3) // 4) * 4
    sl = Slots(2, v_off + ctx * kv_heads * vdim)
    ws = torch.full((2 * heads * 32 * (vdim + 2),), float('nan'), dtype=torch.float32, device='cuda')
    Lc = capi()
    at = 0
    for n in (1, 2, 60, 1, 1, 80, 5):
        d, rs, T = seq_tables([(n, at, 1)])
        qd, kd, vd = dev32(q[at:at + n]), dev32(k[at:at + n]), dev32(v[at:at + n])
        ia.check(Lc.ifa_qk_rope_store_f32(p(qd), heads * dim, heads, p(kd), kv_heads * dim, p(vd), kv_heads * vdim, kv_heads, dim, vdim, p(devbf(qw)), p(devbf(kw)), eps,
                                          rot_dims, p(fr), p(d), p(rs), T, p(sl.table), k_off, v_off, None))
        out = torch.empty((T, heads * vdim + 1), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, scale, 0, 0, 1, 0.0, p(d), p(rs), T, p(sl.table), k_off, v_off, p(out),
                                         heads * vdim + 1, host_seqs([(n, at, 1)]), 1, tile_min, ctx, p(ws) if n <= 2 else None, ws.numel() * 4, None))
        sync()
        assert np.abs(out.cpu().numpy()[:, :heads * vdim] - want[at:at + n]).max() < 2e-5 * max(1.0, np.abs(want).max()), (at, n)
        at += n
    assert at == L
    # without the one in the denominator the weights sum to one: a different result, so it is really counted; another score counts as exp(score)
    d, rs, T = seq_tables([(1, L - 1, 1)])
    qd = dev32(q[L - 1:])
    ia.check(Lc.ifa_qk_rope_store_f32(p(qd), heads * dim, heads, None, 0, None, 0, kv_heads, dim, vdim, p(devbf(qw)), None, eps, rot_dims, p(fr), p(d), p(rs), T,
                                      p(sl.table), k_off, v_off, None))
    res, flat = [], 0.1 / dim          # (scores so small that no key drowns the sink)
    for sink, score in ((0, 0.0), (1, 0.0), (1, 1.5)):
        out = torch.empty((1, heads * vdim), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, flat, 0, 0, sink, score, p(d), p(rs), T, p(sl.table), k_off, v_off, p(out),
                                         heads * vdim, None, 0, 0, ctx, None, 0, None))
        sync(); res.append(out.cpu().numpy())
    want_flat = oracle_attention(q, k, v, qw, kw, heads, kv_heads, dim, vdim, rot_dims, base, flat, eps)
    assert np.abs(res[1] - want_flat[L - 1:]).max() < 2e-5 * max(1.0, np.abs(want_flat).max())
    assert np.abs(res[0] - res[1]).max() > 1e-4 and np.abs(res[2] - res[1]).max() > 1e-4


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot_dims", [(2, 2, 40, 72, 40), (4, 1, 100, 100, 50), (2, 1, 16, 200, 8)])
def test_single_rows_over_a_long_context_with_value_heads_that_end_inside_a_group_of_64_columns(heads, kv_heads, dim, vdim, rot_dims):
    """1300 keys: the keys of a (row, head) are shared out to twenty workgroups, and the merge of their partial results walks value
    columns 64 .. vdim - 1 with only some lanes holding a column"""
    rng = np.random.default_rng(dim + vdim)
    L, eps, scale, base, ctx = 1300, 1e-5, 0.3, 10000.0, 2001
    q, k, v, qw, kw = attention_case(heads, kv_heads, dim, vdim, rot_dims, L, rng)
    want = oracle_attention(q, k, v, qw, kw, heads, kv_heads, dim, vdim, rot_dims, base, scale, eps)
    fr = freq_table(rot_dims, base)
    k_off, v_off = 0, ctx * kv_heads * dim
    sl = Slots(1, v_off + ctx * kv_heads * vdim)
    ws = torch.full((heads * 32 * (vdim + 2),), float('nan'), dtype=torch.float32, device='cuda')
    Lc = capi()
    at = 0
    for n in [1290] + [1] * 10:
        d, rs, T = seq_tables([(n, at, 0)])
        qd, kd, vd = dev32(q[at:at + n]), dev32(k[at:at + n]), dev32(v[at:at + n])
        ia.check(Lc.ifa_qk_rope_store_f32(p(qd), heads * dim, heads, p(kd), kv_heads * dim, p(vd), kv_heads * vdim, kv_heads, dim, vdim, p(devbf(qw)), p(devbf(kw)), eps,
                                          rot_dims, p(fr), p(d), p(rs), T, p(sl.table), k_off, v_off, None))
        out = torch.empty((T, heads * vdim), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, scale, 0, 0, 1, 0.0, p(d), p(rs), T, p(sl.table), k_off, v_off, p(out),
                                         heads * vdim, host_seqs([(n, at, 0)]), 1, 16, ctx, p(ws), ws.numel() * 4, None))
        sync()
        assert np.abs(out.cpu().numpy() - want[at:at + n]).max() < 2e-5 * max(1.0, np.abs(want).max()), (at, n)
        at += n


def test_rotated_attention_tiles_over_several_sequences():
    """one step holds a 150-token prompt, a single continued token and a 40-token continued portion: tiles must not cross sequences"""
    rng = np.random.default_rng(78)
    heads, kv_heads, dim, vdim, rot_dims, eps, scale, base = 4, 2, 40, 24, 16, 1e-5, 0.4, 1000.0
    L, ctx = 200, 208
    seq = {s_: attention_case(heads, kv_heads, dim, vdim, rot_dims, L, rng) for s_ in (0, 1, 2)}
    fr = freq_table(rot_dims, base)
    k_off, v_off = 0, ctx * kv_heads * dim
    sl = Slots(3, v_off + ctx * kv_heads * vdim)
    Lc = capi()
    at = {0: 0, 1: 0, 2: 0}
    for step in ([(1, 30), (2, 100)], [(0, 150), (1, 1), (2, 40)], [(2, 60), (0, 50), (1, 129)]):
        seqs = [(n, at[s_], s_) for s_, n in step]
        d, rs, T = seq_tables(seqs)
        qd, kd, vd = (dev32(np.concatenate([seq[s_][i][at[s_]:at[s_] + n] for s_, n in step], 0)) for i in range(3))
        qw, kw = seq[0][3], seq[0][4]          # (every sequence shares the norm weights of sequence 0: they are the layer's)
        ia.check(Lc.ifa_qk_rope_store_f32(p(qd), heads * dim, heads, p(kd), kv_heads * dim, p(vd), kv_heads * vdim, kv_heads, dim, vdim, p(devbf(qw)), p(devbf(kw)), eps,
                                          rot_dims, p(fr), p(d), p(rs), T, p(sl.table), k_off, v_off, None))
        out = torch.empty((T, heads * vdim), dtype=torch.float32, device="cuda")
        ia.check(Lc.ifa_attention_kv_f32(p(qd), heads * dim, heads, kv_heads, dim, vdim, scale, 0, 0, 1, 0.0, p(d), p(rs), T, p(sl.table), k_off, v_off, p(out),
                                         heads * vdim, host_seqs(seqs), len(seqs), 16, ctx, None, 0, None))
        sync()
        got, r = out.cpu().numpy(), 0
        for s_, n in step:
            w_ = oracle_attention(seq[s_][0], seq[s_][1], seq[s_][2], qw, kw, heads, kv_heads, dim, vdim, rot_dims, base, scale, eps)
            assert np.abs(got[r:r + n] - w_[at[s_]:at[s_] + n]).max() < 2e-5 * max(1.0, np.abs(w_).max()), (s_, at[s_], n)
            r += n; at[s_] += n


@pytest.mark.parametrize("n_all,top", [(6, 2), (16, 1), (5, 5), (70, 8), (3, 2)])
def test_router_on_logits_with_ties_and_softmax_over_the_chosen(n_all, top):
    rng = np.random.default_rng(n_all + top)
    T = 9
    z = rng.standard_normal((T, n_all + 2)).astype(np.float32)
    z[1, :n_all] = 0.5                      # all equal: the lowest indices win
    if n_all > 2:
        z[2, 2] = z[2, 0] = 3.0             # a tie at the top
    bias = bf16_round(rng.standard_normal(n_all))
    for use_bias in (0, 1):
        zz = t64(z[:, :n_all]) + (t64(bias) if use_bias else 0)
        idx_w = torch.argsort(-zz, dim=-1, stable=True)[:, :top]
        wgt_w = torch.softmax(torch.gather(zz, 1, idx_w), -1).numpy()
        idx = torch.zeros((T, top), dtype=torch.int32, device="cuda"); wgt = torch.zeros((T, top), dtype=torch.float32, device="cuda")
        ia.check(capi().ifa_moe_route_top_f32(p(dev32(z)), n_all + 2, T, n_all, top, p(devbf(bias)) if use_bias else None, p(idx), p(wgt), None)); sync()
        assert np.array_equal(idx.cpu().numpy(), idx_w.numpy())
        assert np.abs(wgt.cpu().numpy() - wgt_w).max() < 1e-6


@pytest.mark.parametrize("T,W,F,E,top", [(1, 64, 24, 6, 2), (3, 40, 10, 3, 3), (8, 128, 64, 16, 4), (9, 64, 24, 6, 2), (70, 48, 20, 5, 1), (150, 64, 32, 20, 3), (5, 14, 6, 4, 2)])
def test_gated_experts_in_rows_and_grouped(T, W, F, E, top):
    rng = np.random.default_rng(T + W + F)
    h = rng.standard_normal((T, W + 4)).astype(np.float32)
    gu = bf16_round(rng.standard_normal((E, 2 * F, W)) / np.sqrt(W)); dn = bf16_round(rng.standard_normal((E, W, F)) / np.sqrt(F))
    idx = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    wgt = rng.uniform(0.1, 1.0, (T, top)).astype(np.float32)
    want = np.zeros((T, W))
    for t in range(T):
        for e, a in zip(idx[t], wgt[t]):
            want[t] += a * orc.gated_expert(t64(h[t:t + 1, :W]), t64(gu[e, :F]), t64(gu[e, F:]), t64(dn[e])).numpy()[0]
    L = capi()
    nb = L.ifa_moe_workspace_bytes(T, top, W, 3 * F, E)
    ws = torch.zeros((nb + 15) // 4, dtype=torch.float32, device="cuda")
    y0 = rng.standard_normal((T, W + 1)).astype(np.float32)
    for ops32, tol in ((1, 2e-5), (0, 3e-2)):
        for acc in (0, 1):
            y = dev32(y0)
            ia.check(L.ifa_moe_experts_gated_f32(p(dev32(h)), W + 4, T, W, F, E, top, p(devbf(gu.reshape(E * 2 * F, W))), p(devbf(dn.reshape(E * W, F))), p(devi(idx)),
                                                 p(dev32(wgt)), ops32, p(ws), nb, p(y), W + 1, acc, None)); sync()
            ref = want + (y0[:, :W] if acc else 0)
            t_ = tol if T > 8 else 2e-5          # (steps of at most 8 rows keep fp32 activations in both modes)
            assert np.abs(y.cpu().numpy()[:, :W] - ref).max() < t_ * max(1.0, np.abs(want).max()), (ops32, acc)
