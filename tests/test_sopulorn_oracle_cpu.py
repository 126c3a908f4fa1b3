"""The float64 oracle of the Sopulorn tests checked against properties of its own equations (no GPU): the tests of the product rest on it."""
import numpy as np
import torch

from tests import sopulorn_fixtures as fx
from tests import sopulorn_oracle as orc

CFG = fx.config([fx.attention_layer(mlp=fx.dense()), fx.attention_layer(rot_dims=8), fx.attention_layer(kv_from=1, mlp=None)], width=32, vocab=41)


def logits(cfg, w, toks, res=None):
    with torch.no_grad():
        return orc.forward(cfg, fx.oracle_weights(w), toks, res).numpy()


def test_causal_and_first_token_row():
    w = fx.random_weights(CFG, 1)
    a = [3, 9, 27, 40, 1, 8, 8, 30]
    b = a[:5] + [11, 2, 5]
    la, lb = logits(CFG, w, a), logits(CFG, w, b)
    assert np.allclose(la[:5], lb[:5], atol=1e-12) and not np.allclose(la[5], lb[5], atol=1e-6)
    # the pair table: the last row for the first token, the hash of (previous, current) afterwards
    assert orc.pair_rows([4, 7, 7], 53, 31, 5) == [53, (4 * 31 + 7 * 5) % 53, (7 * 31 + 7 * 5) % 53]
    # the same token after another previous token reads another row
    assert not np.allclose(logits(CFG, w, [5, 6])[1], logits(CFG, w, [7, 6])[1], atol=1e-6)


def test_one_in_the_denominator():
    s = torch.tensor([[0.3, -1.0, 2.0], [float("-inf"), 0.0, float("-inf")]], dtype=orc.F64)
    p = orc.softmax_plus_one(s)
    e = np.exp([0.3, -1.0, 2.0])
    assert np.allclose(p[0].numpy(), e / (1 + e.sum())) and np.allclose(p[1].numpy(), [0, 0.5, 0])
    big = orc.softmax_plus_one(torch.tensor([[800.0, 799.0]], dtype=orc.F64))          # no overflow, the one vanishes
    assert np.allclose(big.numpy(), [[1 / (1 + np.exp(-1)), np.exp(-1) / (1 + np.exp(-1))]])


def test_rotation_pairs_dimension_i_with_i_plus_half_and_keeps_the_rest():
    z = torch.arange(2 * 1 * 10, dtype=orc.F64).reshape(2, 1, 10) + 1
    r = orc.rotate_half_layout(z, [0, 3], 6, 100.0)
    assert torch.equal(r[0], z[0]) and torch.equal(r[1, 0, 6:], z[1, 0, 6:])
    for i in range(3):
        a = 3 * 100.0 ** (-2 * i / 6)
        u, v = z[1, 0, i].item(), z[1, 0, i + 3].item()
        assert np.isclose(r[1, 0, i].item(), u * np.cos(a) - v * np.sin(a)) and np.isclose(r[1, 0, i + 3].item(), v * np.cos(a) + u * np.sin(a))
    # scores depend on the distance only
    q, k = torch.randn(1, 1, 6, dtype=orc.F64), torch.randn(1, 1, 6, dtype=orc.F64)
    s1 = (orc.rotate_half_layout(q, [7], 6, 50.0) * orc.rotate_half_layout(k, [4], 6, 50.0)).sum()
    s2 = (orc.rotate_half_layout(q, [103], 6, 50.0) * orc.rotate_half_layout(k, [100], 6, 50.0)).sum()
    assert np.isclose(s1.item(), s2.item())


def test_router_ties_weights_and_shared_expert():
    W = {"p.mlp.router": orc.t64(np.zeros((4, 3))), "p.mlp.router.b": orc.t64([0.5, 2.0, 2.0, -1.0])}
    idx, wgt = orc.route(orc.t64(np.ones((2, 3))), W, "p.", 3)
    assert idx.tolist() == [[1, 2, 0], [1, 2, 0]]
    e = np.exp([2.0, 2.0, 0.5])
    assert np.allclose(wgt[0].numpy(), e / e.sum())
    # clamps of the dense form: the gate from above only, the other factor on both sides
    Wd = {"p.mlp.gate": orc.t64([[1.0]]), "p.mlp.up": orc.t64([[1.0]]), "p.mlp.down": orc.t64([[1.0]])}
    for x, g, u in ((5.0, 2.0, 2.0), (-5.0, -5.0, -2.0), (0.5, 0.5, 0.5)):
        want = g / (1 + np.exp(-1.702 * g)) * (u + 1)
        assert np.isclose(orc.dense_ffn(orc.t64([[x]]), Wd, "p.", 2.0).item(), want)


def test_shared_keys_and_values_are_the_other_layers_cache_rows():
    # layer 2 reads layer 1's rows: changing layer 1's key projection changes layer 2's output even with layer 1's own output cut off
    w = fx.random_weights(CFG, 2)
    w["l1.mix.o"][:] = 0; w["l1.mlp.shared.down"][:] = 0
    for e in range(6):
        w["l1.mlp.e%d.down" % e][:] = 0
    toks = [1, 2, 3, 4, 5, 6, 7]
    r1 = []; logits(CFG, w, toks, r1)
    w2 = dict(w); w2["l1.mix.k"] = -w["l1.mix.k"]
    r2 = []; logits(CFG, w2, toks, r2)
    assert np.allclose(r1[1].numpy(), r2[1].numpy()) and not np.allclose(r1[2].numpy(), r2[2].numpy(), atol=1e-6)


def test_the_layer_list_library_profile_exports_the_ops_of_this_design():
    import os
    import shutil
    import subprocess
    import sys
    import pytest
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("needs hipcc")
    from inferflow_amd import build
    path = build.build_layered_library()
    names = ("ifa_attention_kv_f32", "ifa_qk_rope_store_f32", "ifa_embed_pair_f32", "ifa_rmsnorm_offset_f32", "ifa_norm_add_norm_f32", "ifa_glu_ex_f32",
             "ifa_moe_route_top_f32", "ifa_moe_experts_gated_f32")
    code = "import ctypes as C, sys\nL = C.CDLL(sys.argv[1])\nprint([n for n in sys.argv[2].split(',') if not hasattr(L, n)])\n"
    r = subprocess.run([sys.executable, "-c", code, path, ",".join(names)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "[]", (r.stdout, r.stderr[-1000:])
