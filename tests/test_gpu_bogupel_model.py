"""The layer-list worker serving Bogupel models through the InferenceEngine (registry, expert stacking, slots, scheduler, sampling entry
points) against the float64 oracle of tests/bogupel_oracle.py: whole prompts, the residual after every layer run (the looped group counts
once per pass), token-by-token decoding, portions, mixed batches with slots reused, a marked key far back and just inside / outside the
window in prompts and in decoding, sinks that matter, states that decay slowly, the first tokens of a sequence, long decoding past the
window, other sizes, greedy generation, the trace tool."""
import json
import os
import subprocess

import numpy as np
import pytest

from tests import bogupel_fixtures as fx
from tests import bogupel_oracle as orc
from tests.gelarax_oracle import bf16_round

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL32 = 3e-5        # fp32 operands: rounding of fp32 sums only
TOL16 = 4e-2        # operands of the matrix products rounded to bfloat16


def assert_close(err, dtype, tol, what=None):
    """fp32: every row within tol.  bfloat16 operands: a router's close call may fall the other way for a row (its experts change, a
    discrete step), and the states and windows of the layers behind carry that row's change to later rows: the typical row must be within
    tol and no row far off.  (test_whole_prompt_in_bfloat16_without_close_calls bounds every row.)"""
    if dtype == "float32":
        assert err.max() < tol, (what, err.max())
    else:
        assert np.median(err) < tol and err.max() < 1.0, (what, np.median(err), err.max())


def engine_for(tmp_path, cfg, weights, dtype="float32", ctx=512, queries=6):
    from inferflow_amd.engine import InferenceEngine
    d = fx.write_model_dir(str(tmp_path / ("m%d" % len(os.listdir(tmp_path)))), fx.clean(cfg), weights)
    return InferenceEngine.from_model_dir(d, dtype, ctx, queries, True)


def tokens_for(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


def oracle_logits(cfg, weights, tokens, taps=None):
    return orc.forward(cfg, fx.oracle_weights(weights), tokens, taps)


def run_whole(eng, tokens):
    q = eng.add_query(tokens)
    assert q > 0
    out = eng.infer()
    assert [i for i, _ in out] == [q]
    lg = eng.last_logits_f32(q)
    eng.remove_query(q)
    return lg, out[0][1]


def run_portions(eng, tokens, sizes):
    """the prompt in portions of the given sizes (the last size repeats); logits of every token"""
    q = eng.add_query(tokens[:sizes[0]])
    rows, at, k = [], sizes[0], 0
    eng.infer(); rows.append(eng.last_logits_f32(q))
    while at < len(tokens):
        k = min(k + 1, len(sizes) - 1)
        n = min(sizes[k], len(tokens) - at)
        for t in tokens[at:at + n]:
            assert eng.commit({q: t})
        eng.infer(); rows.append(eng.last_logits_f32(q))
        at += n
    eng.remove_query(q)
    return np.concatenate(rows, 0)


# an attention layer in front, a looped group of a delta layer, an attention layer without feed-forward and an attention layer with one
# (three passes, so the group's attention layers keep three caches each and the delta layer three states), a delta layer behind the group;
# grouped queries (2 and 3 per key head), part of the head rotated, value heads smaller and larger than key heads, windows 20 / 9 / 33
MIXED = fx.config([fx.attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, rot_dims=16, window=20),
                   fx.delta_layer(heads=3, dim=16, rank=6),
                   fx.attention_layer(heads=6, kv_heads=2, dim=16, vdim=40, rot_dims=8, base=500.0, window=9, mlp=None),
                   fx.attention_layer(heads=2, kv_heads=2, dim=32, vdim=24, rot_dims=32, window=33, scaling=None, mlp=fx.moe(experts=5, top=3, ff=12, limit=0.6)),
                   fx.delta_layer(heads=2, dim=24, rank=3, mlp=fx.moe(experts=3, top=1, ff=40, limit=4.0))],
                  width=64, vocab=97, loop=(1, 4, 3))


@pytest.mark.parametrize("dtype,tol", [("float32", TOL32), ("bfloat16", TOL16)])
def test_whole_prompt_matches_the_oracle(tmp_path, dtype, tol):
    w = fx.random_weights(MIXED, 1)
    toks = tokens_for(MIXED, 71, 2)
    eng = engine_for(tmp_path, MIXED, w, dtype)
    lg, nxt = run_whole(eng, toks)
    want = oracle_logits(MIXED, w, toks)
    assert lg.shape == want.shape
    assert_close(fx.rel_err(lg, want), dtype, tol)
    if dtype == "float32":
        assert nxt == int(want[-1].argmax())
    eng.close()


def test_whole_prompt_in_bfloat16_without_close_calls(tmp_path):
    """every expert chosen, so no choice can fall the other way: every row within the rounding of bfloat16 operands"""
    layers = [dict(L) for L in MIXED["layers"]]
    for L in layers:
        if L.get("mlp"):
            L["mlp"] = fx.moe(experts=L["mlp"]["router"]["experts"], top=L["mlp"]["router"]["experts"], ff=L["mlp"]["expert"]["ff"], limit=L["mlp"]["expert"]["limit"])
    cfg = dict(MIXED); cfg["layers"] = layers
    w = fx.random_weights(cfg, 1)
    toks = tokens_for(cfg, 71, 2)
    want = oracle_logits(cfg, w, toks)
    eng = engine_for(tmp_path, cfg, w, "bfloat16")
    for got in (run_whole(eng, toks)[0], run_portions(eng, toks, [40, 9, 1])):
        err = fx.rel_err(got, want)          # (eleven layer runs deep: the bound of a single row is wider than the typical row's)
        assert np.median(err) < 0.5 * TOL16 and err.max() < 1.5 * TOL16, (np.median(err), err.max())
    eng.close()


def test_residual_after_every_layer_run_matches_the_oracle(tmp_path):
    import ctypes as C
    import inferflow_amd as ia
    w = fx.random_weights(MIXED, 3)
    eng = engine_for(tmp_path, MIXED, w)
    L = ia.lib()
    ia.check(L.ifa_model_set_option(eng.worker(), b"tap_layers", 1))
    for n in (40, 5):          # the tiled and the single-row attention, the grouped and the row form of the experts
        toks = tokens_for(MIXED, n, 4)
        run_whole(eng, toks)
        res = []
        oracle_logits(MIXED, w, toks, res)
        assert len(res) == 1 + 3 * 3 + 1
        for ri, want in enumerate(res):
            p, b = C.c_void_p(), C.c_size_t()
            ia.check(L.ifa_model_get_buffer(eng.worker(), b"layer_taps", ri, C.byref(p), C.byref(b)))
            got = np.zeros((len(toks), MIXED["width"]), np.float32)
            ia.check(L.ifa_memcpy_d2h(got.ctypes.data_as(C.c_void_p), p, got.nbytes, None)); ia.check(L.ifa_stream_sync(None))
            assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max()), (n, ri)
    eng.close()


@pytest.mark.parametrize("sizes", [[1], [2], [5, 3], [30, 1], [7, 2, 1], [64, 4], [17, 16, 2]])
def test_portions_and_token_by_token_equal_the_whole_prompt(tmp_path, sizes):
    w = fx.random_weights(MIXED, 5)
    toks = tokens_for(MIXED, 83, 6)
    eng = engine_for(tmp_path, MIXED, w)
    whole, _ = run_whole(eng, toks)
    parts = run_portions(eng, toks, sizes)
    assert parts.shape == whole.shape
    assert fx.rel_err(parts, whole).max() < TOL32
    assert fx.rel_err(parts, oracle_logits(MIXED, w, toks)).max() < TOL32
    eng.close()


def test_folded_launches_and_separate_ops_agree(tmp_path):
    """the start of a pass inside the norm's launch and the norm inside the router's launch against the same steps as launches of their own"""
    import inferflow_amd as ia
    w = fx.random_weights(MIXED, 25)
    toks = tokens_for(MIXED, 60, 26)
    want = oracle_logits(MIXED, w, toks)
    eng = engine_for(tmp_path, MIXED, w)
    for fuse in (1, 0, 1):
        ia.check(ia.lib().ifa_model_set_option(eng.worker(), b"fuse_post", fuse))
        for sizes in ([33, 1], [3, 2], [8, 7, 1]):
            assert fx.rel_err(run_portions(eng, toks, sizes), want).max() < TOL32, (fuse, sizes)
    eng.close()


@pytest.mark.parametrize("n", [1, 2, 3])
def test_first_tokens_of_a_sequence(tmp_path, n):
    """the shortest prompts, whole and token by token, on a slot that held a longer sequence before (cache rows, states, last token)"""
    w = fx.random_weights(MIXED, 21)
    eng = engine_for(tmp_path, MIXED, w, queries=1)
    run_whole(eng, tokens_for(MIXED, 50, 22))
    toks = tokens_for(MIXED, n, 23 + n)
    want = oracle_logits(MIXED, w, toks)
    assert fx.rel_err(run_whole(eng, toks)[0], want).max() < TOL32
    assert fx.rel_err(run_portions(eng, toks, [1]), want).max() < TOL32
    eng.close()


def test_batches_of_unequal_requests_equal_each_alone_and_slots_are_reused(tmp_path):
    w = fx.random_weights(MIXED, 7)
    eng = engine_for(tmp_path, MIXED, w, queries=3)
    prompts = [tokens_for(MIXED, n, 10 + n) for n in (1, 37, 64, 5, 90, 2)]
    tails = [tokens_for(MIXED, 12, 50 + i) for i in range(len(prompts))]
    alone = [oracle_logits(MIXED, w, p + t) for p, t in zip(prompts, tails)]
    # three queries on three slots, twice: the second time reuses the slots of the first
    for rnd in range(2):
        qs = [eng.add_query(p) for p in prompts[3 * rnd:3 * rnd + 3]]
        assert all(q > 0 for q in qs) and eng.add_query([1, 2]) == 0          # busy: every slot is taken
        got = {q: [] for q in qs}
        assert sorted(i for i, _ in eng.infer()) == sorted(qs)                 # ONE step for the three prompts
        for q in qs:
            got[q].append(eng.last_logits_f32(q))
        for step in range(12):
            live = [q for k, q in enumerate(qs) if not (k == 0 and step >= 6)]  # the first query ends earlier
            if step == 6:
                eng.remove_query(qs[0])
            eng.commit({q: tails[3 * rnd + qs.index(q)][step] for q in live})
            assert sorted(i for i, _ in eng.infer()) == sorted(live)
            for q in live:
                got[q].append(eng.last_logits_f32(q))
        for k, q in enumerate(qs):
            g = np.concatenate(got[q], 0)
            assert fx.rel_err(g, alone[3 * rnd + k][:len(g)]).max() < TOL32, (rnd, k)
            if not (k == 0):
                eng.remove_query(q)
    eng.close()


def test_ten_requests_start_together_and_are_decoded_together(tmp_path):
    """a step of ten prompts of unequal lengths, then steps of ten, later six, single tokens: more rows than the few-row forms of the products, the
    router and the experts take, every row a sequence of its own"""
    w = fx.random_weights(MIXED, 41)
    eng = engine_for(tmp_path, MIXED, w, queries=10)
    prompts = [tokens_for(MIXED, n, 60 + n) for n in (3, 18, 1, 40, 7, 25, 2, 33, 12, 5)]
    tails = [tokens_for(MIXED, 9, 80 + i) for i in range(10)]
    alone = [oracle_logits(MIXED, w, p + t) for p, t in zip(prompts, tails)]
    qs = [eng.add_query(p) for p in prompts]
    got = {q: [] for q in qs}
    assert sorted(i for i, _ in eng.infer()) == sorted(qs)
    for q in qs:
        got[q].append(eng.last_logits_f32(q))
    live = list(qs)
    for step in range(9):
        if step == 5:
            for q in qs[6:]:
                eng.remove_query(q); live.remove(q)
        eng.commit({q: tails[qs.index(q)][step] for q in live})
        assert sorted(i for i, _ in eng.infer()) == sorted(live)
        for q in live:
            got[q].append(eng.last_logits_f32(q))
    for k, q in enumerate(qs):
        g = np.concatenate(got[q], 0)
        assert fx.rel_err(g, alone[k][:len(g)]).max() < TOL32, k
    eng.close()


def marked_model(window, passes):
    """One attention layer, run `passes` times as a looped group, whose weights make one key stand out: residual feature 0 is set only by the
    token `mark`, feature 1 only by the token `probe`; the last dimension of every query head reads feature 1 alone, the last dimension of the
    key head feature 0 alone, and that dimension does not rotate, so the probe's query matches the mark's key at any distance.  The last
    row's logits then depend strongly on whether the mark's cache row is read."""
    D = 16
    cfg = fx.config([fx.attention_layer(heads=2, kv_heads=1, dim=D, vdim=24, rot_dims=8, scale=1.0, window=window, mlp=None)], width=32, vocab=50,
                    embed_scale=2.0, loop=(0, 1, passes))
    w = fx.random_weights(cfg, 9)
    mark, probe = 7, 9
    w["embed"][:, :2] = 0; w["bigram"][:, :2] = 0; w["loop.step"][:, :2] = 0
    w["embed"][mark, 0] = 4.0; w["embed"][probe, 1] = 4.0
    p = "l0."
    w[p + "norm1"][:2] = 1.0; w[p + "norm1.b"][:2] = 0
    q, k = w[p + "mix.q"], w[p + "mix.k"]
    q[:, :2] = 0; k[:, :2] = 0
    for h in range(2):
        q[h * D + D - 1, :] = 0; q[h * D + D - 1, 1] = 6.0
    k[D - 1, :] = 0; k[D - 1, 0] = 6.0
    w[p + "mix.q.b"][:] *= 0.2; w[p + "mix.k.b"][:] *= 0.2
    for b in (w[p + "mix.q.b"], w[p + "mix.k.b"]):
        b[D - 1::D] = 0
    w[p + "mix.q.norm"][D - 1] = 3.0; w[p + "mix.k.norm"][D - 1] = 3.0
    w[p + "mix.o"][:2, :] = 0                               # the layer leaves features 0 and 1 as they were
    w[p + "mix.sink"][:] = 0.5
    return cfg, {k_: bf16_round(v) for k_, v in w.items()}, mark, probe


def marked_tokens(n, mark_at, mark, probe):
    filler = [t for t in range(10, 50)]
    toks = [filler[(3 * i + mark_at + n) % len(filler)] for i in range(n)]
    toks[mark_at] = mark; toks[-1] = probe
    return toks, filler


def test_far_keys_at_block_and_share_edges_in_prompts_and_decoding(tmp_path):
    """a window wider than every sequence; the marked key at the borders of the tiled kernel's key blocks (32) and query tiles (128) and of
    the single-row kernel's key shares, hundreds of tokens back"""
    cfg, w, mark, probe = marked_model(window=1000, passes=2)
    eng = engine_for(tmp_path, cfg, w, ctx=700)
    for mark_at, n in ((0, 2), (0, 33), (31, 300), (32, 300), (63, 129), (64, 129), (127, 128), (128, 130), (15, 600), (16, 600), (255, 257), (256, 258), (5, 640)):
        toks, filler = marked_tokens(n, mark_at, mark, probe)
        want = oracle_logits(cfg, w, toks)
        whole, _ = run_whole(eng, toks)
        assert fx.rel_err(whole, want).max() < TOL32, ("prompt", mark_at, n)
        dec = run_portions(eng, toks, [max(1, n - 3), 1])
        assert fx.rel_err(dec, want).max() < TOL32, ("decoded", mark_at, n)
        # the oracle itself must see the key: without the mark the last row differs clearly
        blind = list(toks); blind[mark_at] = filler[0]
        assert fx.rel_err(oracle_logits(cfg, w, blind)[-1:], want[-1:]).max() > 1e-3, (mark_at, n)
    eng.close()


@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 64, 70, 129])
def test_keys_just_inside_and_just_outside_the_window(tmp_path, window):
    """the marked key at distance window - 1 (seen) and window (not seen) from the probe, in a whole prompt, in portions of two tokens and
    decoded token by token; a window of 1 sees the token itself only"""
    cfg, w, mark, probe = marked_model(window=window, passes=2)
    eng = engine_for(tmp_path, cfg, w, ctx=400)
    n = window + 150
    for dist in (window - 1, window):
        if dist == 0:
            continue
        toks, filler = marked_tokens(n, n - 1 - dist, mark, probe)
        want = oracle_logits(cfg, w, toks)
        for sizes in ([n], [n - 40, 2], [n - 40, 1], [max(1, n - 200), 37, 1]):
            got = run_portions(eng, toks, sizes)
            assert fx.rel_err(got, want).max() < TOL32, (window, dist, sizes)
        if dist < window:       # inside: the oracle's last row knows the mark (outside it may still hear of it through the rows between, a pass later)
            blind = list(toks); blind[n - 1 - dist] = filler[0]
            assert fx.rel_err(oracle_logits(cfg, w, blind)[-1:], want[-1:]).max() > 1e-3, (window, dist)
    eng.close()


def test_sinks_that_matter(tmp_path):
    """large sinks take most of the weight: leaving them out, or counting them per key head, changes the logits clearly"""
    cfg = fx.config([fx.attention_layer(heads=4, kv_heads=2, window=12), fx.attention_layer(heads=4, kv_heads=1, window=50, mlp=None)], width=48, vocab=41)
    w = fx.random_weights(cfg, 27)
    w["l0.mix.sink"][:] = [6.0, -3.0, 2.0, 9.0]; w["l1.mix.sink"][:] = [4.0, 5.0, -6.0, 0.0]
    w = {k: bf16_round(v) for k, v in w.items()}
    toks = tokens_for(cfg, 70, 28)
    want = oracle_logits(cfg, w, toks)
    eng = engine_for(tmp_path, cfg, w)
    assert fx.rel_err(run_whole(eng, toks)[0], want).max() < TOL32
    assert fx.rel_err(run_portions(eng, toks, [50, 1]), want).max() < TOL32
    none = dict(w); none["l0.mix.sink"] = np.full(4, -60.0, np.float32); none["l1.mix.sink"] = np.full(4, -60.0, np.float32)
    assert fx.rel_err(oracle_logits(cfg, none, toks), want).max() > 1e-2
    eng.close()


def test_states_that_decay_slowly_are_carried_through_portions_and_decoding(tmp_path):
    """decays close to one and small removal rates: what the first tokens wrote into the state still shows hundreds of tokens later, so a
    state that is lost, restarted or taken from another pass shows"""
    cfg = fx.config([fx.delta_layer(heads=2, dim=16, rank=4, mlp=None), fx.delta_layer(heads=3, dim=48, rank=5), fx.delta_layer(heads=1, dim=20, rank=2, mlp=None)],
                    width=48, vocab=61, loop=(0, 2, 2))
    w = fx.random_weights(cfg, 33)
    for li in range(3):
        w["l%d.mix.w0" % li][:] = -7.0
        w["l%d.mix.a.b" % li][:] = -4.0
    w = {k: bf16_round(v) for k, v in w.items()}
    toks = tokens_for(cfg, 300, 34)
    want = oracle_logits(cfg, w, toks)
    other = list(toks); other[0] = (toks[0] + 1) % cfg["vocab"]
    assert fx.rel_err(oracle_logits(cfg, w, other)[-1:], want[-1:]).max() > 1e-4       # the first token still matters at the end
    eng = engine_for(tmp_path, cfg, w, ctx=400)
    for sizes in ([300], [150, 1], [9, 8, 7, 2], [100, 64, 3]):
        assert fx.rel_err(run_portions(eng, toks, sizes), want).max() < 1e-4, sizes
    eng.close()


def test_long_decoding_past_the_window(tmp_path):
    cfg = fx.config([fx.attention_layer(heads=2, kv_heads=1, dim=16, vdim=8, rot_dims=16, base=200.0, window=40, mlp=fx.moe(experts=4, top=2, ff=16)),
                     fx.delta_layer(heads=2, dim=32, rank=4, mlp=None),
                     fx.attention_layer(heads=2, kv_heads=2, dim=16, vdim=12, rot_dims=4, window=100)], width=32, vocab=61, loop=(0, 2, 2))
    w = fx.random_weights(cfg, 11)
    toks = tokens_for(cfg, 330, 12)
    want = oracle_logits(cfg, w, toks)
    eng = engine_for(tmp_path, cfg, w, ctx=400)
    got = run_portions(eng, toks, [200, 1])        # 130 tokens decoded one by one: both windows pass over decoded tokens
    assert fx.rel_err(got, want).max() < 5e-5
    eng.close()


CASES = {
    # one head, one expert of which one is chosen, a pair table of one bucket, two rotated dimensions, value heads of two numbers, a window of
    # one token, a bottleneck of one, scales of one, one pass of the group
    "ones": lambda: fx.config([fx.attention_layer(heads=1, kv_heads=1, dim=2, vdim=2, rot_dims=2, window=1, mlp=fx.moe(experts=1, top=1, ff=4, limit=1.0)),
                               fx.delta_layer(heads=1, dim=4, rank=1, mlp=fx.moe(experts=2, top=1, ff=3))], width=16, vocab=11, bigram=(1, 1, 1), embed_scale=1.0,
                              logit_scale=1.0, loop=(1, 2, 1)),
    # no pair table, no rotation of queries and keys, no feed-forward, every expert chosen, no group
    "plain": lambda: fx.config([fx.attention_layer(rot_dims=0, mlp=None), fx.delta_layer(mlp=None), fx.attention_layer(rot_dims=0, mlp=fx.moe(experts=3, top=3, ff=12))],
                               width=48, vocab=33, bigram=None),
    # sizes that keep every 16-byte path off: odd head sizes of the keys, width 14, odd bottleneck, delta heads of 5 and 7 channels
    "unaligned": lambda: fx.config([fx.attention_layer(heads=3, kv_heads=1, dim=5, vdim=6, rot_dims=4, window=7, mlp=fx.moe(experts=3, top=2, ff=10)),
                                    fx.delta_layer(heads=3, dim=5, rank=3, mlp=fx.moe(experts=2, top=2, ff=9, limit=0.5)),
                                    fx.delta_layer(heads=2, dim=7, rank=5, mlp=None)], width=14, vocab=9, bigram=(7, 3, 2), loop=(0, 3, 2)),
    # the widest heads the tiled kernel takes, all of them rotated; delta heads of 128 and 64 channels (states in registers)
    "wide_heads": lambda: fx.config([fx.attention_layer(heads=2, kv_heads=1, dim=128, vdim=128, rot_dims=128, window=64, mlp=fx.moe(experts=4, top=2, ff=64)),
                                     fx.delta_layer(heads=1, dim=128, rank=8, mlp=None), fx.delta_layer(heads=2, dim=64, rank=8, mlp=None)], width=128, vocab=50,
                                    loop=(1, 3, 2)),
    # heads beyond the tiled kernel (prompts take the single-row form too), delta heads beyond the register kernels, the group first
    "beyond_the_tile": lambda: fx.config([fx.attention_layer(heads=2, kv_heads=2, dim=160, vdim=136, rot_dims=96, window=30, mlp=fx.moe(experts=2, top=1, ff=32, limit=2.0)),
                                          fx.delta_layer(heads=2, dim=72, rank=4, mlp=None)], width=64, vocab=23, loop=(0, 1, 2)),
    # many experts, eight chosen; delta heads of 32 and 96 channels
    "many_experts": lambda: fx.config([fx.delta_layer(heads=2, dim=32, rank=16, mlp=fx.moe(experts=70, top=8, ff=16)), fx.delta_layer(heads=1, dim=96, rank=2, mlp=None)],
                                      width=32, vocab=29),
    # the group at the end, four passes, as many key heads as query heads, a limit that clamps nearly everything, a large hash
    "group_last": lambda: fx.config([fx.delta_layer(heads=2, dim=16, mlp=None)]
                                    + [fx.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, window=25, mlp=fx.moe(experts=3, top=2, ff=40, limit=0.05)) for _ in range(2)],
                                    width=32, vocab=40, bigram=(2039, 40009, 65537), loop=(1, 3, 4)),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_other_sizes(tmp_path, case):
    cfg = CASES[case]()
    w = fx.random_weights(cfg, 13)
    toks = tokens_for(cfg, 45, 14)
    want = oracle_logits(cfg, w, toks)
    for dtype, tol in (("float32", TOL32), ("bfloat16", TOL16)):
        eng = engine_for(tmp_path, cfg, w, dtype)
        whole, _ = run_whole(eng, toks)
        assert_close(fx.rel_err(whole, want), dtype, tol, (case, dtype))
        assert_close(fx.rel_err(run_portions(eng, toks, [20, 9, 1]), want), dtype, tol, (case, dtype, "portions"))
        eng.close()


def test_correction_decides_the_choice_and_not_the_weights(tmp_path):
    """a large correction moves the choice to experts whose scores are small; the weights stay the plain sigmoid scores"""
    cfg = fx.config([fx.delta_layer(mlp=fx.moe(experts=5, top=2, ff=16))], width=32, vocab=31)
    w = fx.random_weights(cfg, 31)
    c = w["l0.mlp.correction"]
    c[:] = 0; c[4] = 30.0; c[1] = 29.0
    w = {k: bf16_round(v) for k, v in w.items()}
    toks = tokens_for(cfg, 40, 32)
    eng = engine_for(tmp_path, cfg, w)
    want = oracle_logits(cfg, w, toks)
    assert fx.rel_err(run_whole(eng, toks)[0], want).max() < TOL32
    assert fx.rel_err(run_portions(eng, toks, [1]), want).max() < TOL32
    plain = dict(w); plain["l0.mlp.correction"] = np.zeros_like(c)
    assert fx.rel_err(oracle_logits(cfg, plain, toks), want).max() > 1e-3
    eng.close()


def test_greedy_generation_through_the_engine(tmp_path):
    w = fx.random_weights(MIXED, 15)
    prompt = tokens_for(MIXED, 19, 16)
    eng = engine_for(tmp_path, MIXED, w)
    # Generate(): prompt step + decode steps replayed from a captured graph with the token fed back on the device
    q = eng.add_query(prompt)
    gen, _ = eng.generate(q, 24)
    eng.remove_query(q)
    # the serving loop: Infer -> Commit of the greedy token
    q = eng.add_query(prompt)
    loop = []
    for _ in range(24):
        (qq, tok), = eng.infer()
        loop.append(tok); eng.commit({q: tok})
    eng.remove_query(q)
    assert gen == loop
    # the oracle follows the same tokens and agrees wherever its two best logits are clearly apart
    want = oracle_logits(MIXED, w, prompt + gen)
    for i, tok in enumerate(gen):
        row = want[len(prompt) - 1 + i]
        top2 = np.sort(row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
            assert tok == int(row.argmax()), i
    # a second generation on the same slot replays the captured step against a new sequence (and its own previous token and states)
    q = eng.add_query(prompt[:7])
    gen2, _ = eng.generate(q, 10)
    eng.remove_query(q)
    want2 = oracle_logits(MIXED, w, prompt[:7] + gen2)
    for i, tok in enumerate(gen2):
        row = want2[6 + i]
        top2 = np.sort(row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
            assert tok == int(row.argmax()), i
    # sampled queries draw from the same logits (top-k with a seed: reproducible)
    a = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    b = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    out = dict(eng.infer())
    assert out[a] == out[b] and 0 <= out[a] < MIXED["vocab"]
    eng.close()


def test_ini_route_and_trace_replay_tool(tmp_path):
    from inferflow_amd.engine import InferenceEngine
    w = fx.random_weights(MIXED, 17)
    d = fx.write_model_dir(str(tmp_path / "model"), fx.clean(MIXED), w)
    ini = tmp_path / "serve.ini"
    ini.write_text("[transformer_engine]\nmodels = m\ndevices = 0\nmax_concurrent_queries = 2\nreturn_output_tensors_f32 = true\n\n"
                   "[model.m]\nmodel_dir = %s/\ncompute_dtype = float32\nmax_context_len = 100\n" % d)
    eng = InferenceEngine.from_ini(str(ini))
    toks = tokens_for(MIXED, 30, 18)
    lg, _ = run_whole(eng, toks)
    want = oracle_logits(MIXED, w, toks)
    assert fx.rel_err(lg, want).max() < TOL32
    assert eng.model_info("vocab_size") == MIXED["vocab"] and eng.model_info("decoder_layers") == len(MIXED["layers"])
    eng.close()
    # the trace tool: two requests start together, go on token by token, one ends earlier
    a, b = tokens_for(MIXED, 26, 19), tokens_for(MIXED, 9, 20)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [0, 19]}, {"id": "b", "tokens": b[:6], "want": [5]}], "end": []}]
    for s in range(1, 7):
        ent = [{"id": "a", "tokens": [a[19 + s]], "want": [0]}]
        if s <= 3:
            ent.append({"id": "b", "tokens": [b[5 + s]], "want": [0] if s != 2 else []})
        steps.append({"step": s, "entries": ent, "end": (["b"] if s == 3 else []) + (["a"] if s == 6 else [])})
    out = tmp_path / "out"; out.mkdir()
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                       input="".join(json.dumps(s) + "\n" for s in steps).encode(), stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=900)
    assert r.returncode == 0, r.stderr.decode()[-2000:]
    assert [l for l in r.stdout.decode().split() if l != "done"] == [str(s) for s in range(7)]
    wa, wb = oracle_logits(MIXED, w, a), oracle_logits(MIXED, w, b)
    V = MIXED["vocab"]
    g0 = np.fromfile(out / "0.f32", np.float32).reshape(-1, V)
    assert fx.rel_err(g0, np.stack([wa[0], wa[19], wb[5]])).max() < TOL32
    for s in range(1, 7):
        g = np.fromfile(out / ("%d.f32" % s), np.float32).reshape(-1, V)
        exp = [wa[19 + s]] + ([wb[5 + s]] if s <= 3 and s != 2 else [])
        assert fx.rel_err(g, np.stack(exp)).max() < TOL32, s
