"""The float64 oracle of the Bogupel tests against properties of the equations themselves (no GPU): what the element-wise norm does at its
ends, where the scaled frequencies change, that rotation depends on distance only and that turned values come back unturned, what the sink
does in its limits, that the generalized delta rule replaces what a key held, the tie rule and the weights of the router, the clamps, the
run order of a looped group, causality of the whole model."""
import math

import numpy as np

from tests import bogupel_fixtures as fx
from tests import bogupel_oracle as orc


def test_dynamic_tanh_at_its_ends():
    x = np.array([[-50.0, -0.1, 0.0, 0.1, 50.0]])
    w, b = np.array([2.0, 2.0, 2.0, 2.0, 2.0]), np.array([0.5, 0.5, 0.5, 0.5, 0.5])
    y = orc.dyt(x, 0.5, w, b)
    assert np.allclose(y[0, [0, 2, 4]], [-1.5, 0.5, 2.5]) and abs(y[0, 3] - (0.5 + 2 * math.tanh(0.05))) < 1e-15
    assert np.allclose(orc.dyt(x, 0.0, w, b), b)


def test_scaled_frequencies_keep_short_waves_and_slow_long_ones():
    sc = {"factor": 6.0, "low": 1.5, "high": 5.0, "original": 64}
    plain, scaled = orc.frequencies(10000.0, 32), orc.frequencies(10000.0, 32, sc)
    wl = 2 * math.pi / plain
    short, long_ = wl < 64 / 5.0, wl > 64 / 1.5
    assert short.any() and long_.any() and (~short & ~long_).any()
    assert np.array_equal(scaled[short], plain[short]) and np.allclose(scaled[long_], plain[long_] / 6.0)
    mid = ~short & ~long_
    assert np.all(scaled[mid] < plain[mid]) and np.all(scaled[mid] > plain[mid] / 6.0)
    # continuous at both ends of the blend: a frequency just on either side of an edge is scaled alike (dims 4, i = 1: f = base^(-1/2))
    for edge in (64 / 5.0, 64 / 1.5):
        f = 2 * math.pi / edge
        ratios = []
        for eps_ in (-1e-9, 1e-9):
            base = (f * (1 + eps_)) ** -2.0
            ratios.append(orc.frequencies(base, 4, sc)[1] / orc.frequencies(base, 4)[1])
        assert abs(ratios[0] - ratios[1]) < 1e-6 and (abs(ratios[0] - 1.0) < 1e-6 or abs(ratios[0] - 1 / 6.0) < 1e-6)


def test_rotation_depends_on_distance_only_and_turned_values_come_back():
    rng = np.random.default_rng(0)
    fr = orc.frequencies(100.0, 8)
    q, k = rng.standard_normal((1, 1, 12)), rng.standard_normal((1, 1, 12))
    dots = [float((orc.turn(q, [p + 5], fr) * orc.turn(k, [p], fr)).sum()) for p in (0, 3, 40)]
    assert max(dots) - min(dots) < 1e-12
    assert np.array_equal(orc.turn(q, [7], fr)[..., 8:], q[..., 8:])          # dimensions beyond the rotated ones pass
    v = rng.standard_normal((5, 2, 6))
    fv = orc.frequencies(100.0, 6)
    back = orc.turn(orc.turn(v, np.arange(5), fv), np.arange(5), fv, sign=-1.0)
    assert np.abs(back - v).max() < 1e-14
    # a value at position j read at position i comes out turned by j - i
    one = orc.turn(orc.turn(v[:1], [9], fv), [11], fv, sign=-1.0)
    assert np.abs(one - orc.turn(v[:1], [-2], fv)).max() < 1e-14


def test_sink_in_its_limits():
    sc = np.array([[0.3, -1.0, 2.0]])
    assert np.allclose(orc.softmax_with_sink(sc, -np.inf).sum(), 1.0)
    p = orc.softmax_with_sink(sc, 0.7)
    assert abs(p.sum() - np.exp(sc).sum() / (np.exp(sc).sum() + math.exp(0.7))) < 1e-15
    assert orc.softmax_with_sink(sc, 60.0).sum() < 1e-20
    masked = np.array([[0.3, -np.inf, -np.inf]])
    assert np.allclose(orc.softmax_with_sink(masked, 0.3), [[0.5, 0.0, 0.0]])


def test_generalized_delta_rule_replaces_what_a_key_held():
    rng = np.random.default_rng(1)
    d = 6
    k = np.zeros((3, d)); k[0, 2] = 1.0; k[1, 2] = 1.0; k[2, 4] = 1.0
    v = rng.standard_normal((3, d))
    ones = np.ones((3, d))
    o, S = orc.delta_scan(k, k, v, ones, ones)
    # no decay, full removal: the second write to the same unit key replaces the first; another key is left alone
    assert np.abs(o[1] - v[1]).max() < 1e-5 and np.abs(S[2] - v[1]).max() < 1e-5 and np.abs(S[4] - v[2]).max() < 1e-5
    # no removal: writes add up, weighted by the decay of their rows
    o2, S2 = orc.delta_scan(k, k, v, 0.5 * ones, 0.0 * ones)
    assert np.abs(S2[2] - (0.25 * v[0] + 0.5 * v[1])).max() < 1e-12
    # both terms read the OLD state: decay and removal do not compound
    o3, S3 = orc.delta_scan(k[:2], k[:2], v[:2], 0.5 * ones[:2], ones[:2])
    assert np.abs(S3[2] - (0.5 * v[0] - v[0] * (1 - 5e-7) + v[1])).max() < 1e-5


def test_router_ties_weights_and_clamps():
    h = np.array([[1.0, 0.0], [0.0, 1.0]])
    router = np.array([[0.2, 0.0], [0.2, 0.0], [-1.0, 3.0]])
    idx, wgt = orc.route(h, router, np.array([0.0, 0.0, 0.0]), 2)
    assert idx[0].tolist() == [0, 1] and idx[1].tolist() == [2, 0]
    idx2, wgt2 = orc.route(h, router, np.array([0.0, 0.0, 5.0]), 1)
    assert idx2[:, 0].tolist() == [2, 2] and abs(wgt2[0, 0] - orc.logistic(-1.0)) < 1e-15          # chosen by the correction, weighted without it
    g, u, dn = np.array([[3.0], [-3.0]]), np.array([[-4.0], [0.5]]), np.eye(2)
    y = orc.clamped_expert(np.array([[1.0]]), g, u, dn, 1.5)
    assert np.allclose(y, [[1.5 * orc.logistic(1.702 * 1.5) * (-1.5 + 1), -3.0 * orc.logistic(-3.0 * 1.702) * 1.5]])


def test_run_order_of_a_looped_group():
    cfg = {"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}
    assert orc.run_order(cfg) == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, None), (4, None)]
    assert orc.run_order({"layers": [0] * 2}) == [(0, None), (1, None)]
    assert orc.run_order({"layers": [0] * 2, "loop": {"start": 0, "stop": 2, "times": 1}}) == [(0, 0), (1, 0)]


def test_whole_model_is_causal_and_the_first_token_takes_the_last_pair_row():
    cfg = fx.config([fx.attention_layer(window=5), fx.delta_layer(), fx.attention_layer(heads=2, kv_heads=1, window=3, mlp=None)], width=32, vocab=23, loop=(1, 3, 2))
    w = fx.oracle_weights(fx.random_weights(cfg, 2))
    toks = [int(t) for t in np.random.default_rng(3).integers(0, 23, 20)]
    taps = []
    a = orc.forward(cfg, w, toks, taps)
    assert len(taps) == 5 and a.shape == (20, 23)
    other = list(toks); other[12] = (toks[12] + 1) % 23
    b = orc.forward(cfg, w, other)
    assert np.array_equal(a[:12], b[:12]) and np.abs(a[12:] - b[12:]).max() > 1e-6
    assert orc.pair_rows(toks, 53, 31, 5)[0] == 53 and orc.pair_rows(toks, 53, 31, 5)[1] == (toks[0] * 31 + toks[1] * 5) % 53
    # the group's passes differ: the second starts from x + x_0 + step[1]
    one = dict(cfg); one["loop"] = {"start": 1, "stop": 3, "times": 1}
    w1 = dict(w); w1["loop.step"] = w["loop.step"][:1]
    assert np.abs(orc.forward(one, w1, toks) - a).max() > 1e-6
