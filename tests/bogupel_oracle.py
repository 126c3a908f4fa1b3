"""Plain float64 implementation of the Bogupel decoder in numpy, one function per mechanism, whole sequences only (no cache, no state
carried between calls, no batching).  It is what the tests compare the layer-list worker with; it shares no code with the product path.

A model: x_t = s_e E[tok_t] + B[pair_t]; the layers in their run order; logits = s_l head(dyt(x)).  A layer, with dyt(y) = tanh(alpha y) w + b:
    x <- x + mixer(dyt_1(x));   x <- x + experts(dyt_2(x))        (the second line only if the layer has a feed-forward)
Layers [start, stop) form a group that runs `times` times; pass t starts from x + (t > 0 ? x_0 : 0) + step[t], x_0 the embedding output.
"""
import math

import numpy as np


def f64(a):
    return np.asarray(a, dtype=np.float64)


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def dyt(y, alpha, w, b):
    """the element-wise norm of this design: no mean, no variance"""
    return np.tanh(float(np.asarray(alpha).reshape(-1)[0]) * y) * w + b


def rms_unit(y, eps):
    return y / np.sqrt((y * y).mean(-1, keepdims=True) + eps)


def pair_rows(tokens, buckets, mul_prev, mul_cur):
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((int(a) * mul_prev + int(b) * mul_cur) % buckets)
    return rows


def embed(cfg, W, tokens):
    em = cfg.get("embedding") or {}
    x = W["embed"][list(tokens)] * float(em.get("scale", 1.0))
    bg = em.get("bigram")
    if bg:
        x = x + W["bigram"][pair_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


def frequencies(base, dims, scaling=None):
    """f_i = base^(-2 i / dims); with scaling: short wavelengths keep f, long ones get f / factor, a linear blend in between"""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            wavelength = 2.0 * math.pi / f
            if wavelength > scaling["original"] / scaling["low"]:
                f = f / scaling["factor"]
            elif wavelength >= scaling["original"] / scaling["high"]:
                t = (scaling["original"] / wavelength - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - t) * f / scaling["factor"] + t * f
        out.append(f)
    return np.array(out, dtype=np.float64)


def turn(z, positions, freqs, sign=1.0):
    """z [T, heads, d]: with n = len(freqs), dimension i < n turns together with dimension i + n by sign * p * freqs[i]; the rest pass"""
    n = len(freqs)
    if n == 0:
        return z.copy()
    ang = sign * f64(positions)[:, None, None] * freqs[None, None, :]
    c, s = np.cos(ang), np.sin(ang)
    lo, hi = z[..., :n], z[..., n:2 * n]
    return np.concatenate([lo * c - hi * s, hi * c + lo * s, z[..., 2 * n:]], -1)


def queries_and_keys(h, W, p, mx, eps, positions):
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, mx["heads"], mx["dim"])
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, mx["kv_heads"], mx["dim"])
    q = rms_unit(q, eps) * W[p + "q.norm"]
    k = rms_unit(k, eps) * W[p + "k.norm"]
    rot = mx["rot"]
    fr = frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    return turn(q, positions, fr), turn(k, positions, fr)


def cached_values(h, W, p, mx, eps, positions):
    """values as they are kept: divided by their root mean square, then turned by their own position over the whole head"""
    T = h.shape[0]
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, mx["kv_heads"], mx["vdim"])
    return turn(rms_unit(v, eps), positions, frequencies(mx["rot"]["base"], mx["vdim"]))


def softmax_with_sink(scores, sink):
    """rows of scores (-inf where masked); exp(sink) is one more term of the denominator"""
    m = np.maximum(scores.max(-1, keepdims=True), sink)
    e = np.exp(scores - m)
    return e / (e.sum(-1, keepdims=True) + np.exp(sink - m))


def attention_mixer(h, W, p, mx, eps):
    T = h.shape[0]
    H, G, dv = mx["heads"], mx["kv_heads"], mx["vdim"]
    positions = np.arange(T)
    q, k = queries_and_keys(h, W, p, mx, eps, positions)
    v = cached_values(h, W, p, mx, eps, positions)
    i, j = positions[:, None], positions[None, :]
    seen = (j <= i)
    window = (mx.get("mask") or {}).get("size")
    if window:
        seen = seen & (i - j < window)
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // (H // G)
        sc = np.where(seen, (q[:, hd] @ k[:, g].T) * mx["scale"], -np.inf)
        out[:, hd] = softmax_with_sink(sc, float(W[p + "sink"][hd])) @ v[:, g]
    out = turn(out, positions, frequencies(mx["rot"]["base"], dv), sign=-1.0)
    return out.reshape(T, H * dv) @ W[p + "o"].T


def delta_gates(h, W, p, H, d):
    """decay per key channel (through the two-matrix bottleneck), removal rate per key channel"""
    T = h.shape[0]
    decay = np.exp(-math.exp(-0.5) * logistic(np.tanh(h @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"]))
    rate = logistic(h @ W[p + "a"].T + W[p + "a.b"])
    return decay.reshape(T, H, d), rate.reshape(T, H, d)


def delta_scan(r, k, v, decay, rate, state=None):
    """one head: r, k, v, decay, rate [T, d].  S_t = diag(decay_t) S_(t-1) - (rate_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t"""
    T, d = k.shape
    S = np.zeros((d, v.shape[1])) if state is None else state.copy()
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        u = k[t] / math.sqrt(float((k[t] * k[t]).sum()) + 1e-6)
        S = decay[t][:, None] * S - np.outer(rate[t] * u, u @ S) + np.outer(k[t], v[t])
        o[t] = S.T @ r[t]
    return o, S


def general_delta_mixer(h, W, p, mx, eps):
    T = h.shape[0]
    H, d = mx["heads"], mx["dim"]
    r = (h @ W[p + "r"].T).reshape(T, H, d)
    k = (h @ W[p + "k"].T).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, d)
    decay, rate = delta_gates(h, W, p, H, d)
    o = np.stack([delta_scan(r[:, hd], k[:, hd], v[:, hd], decay[:, hd], rate[:, hd])[0] for hd in range(H)], 1)
    o = rms_unit(o, eps).reshape(T, H * d) * W[p + "norm"] * logistic(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def route(h, router, correction, top):
    """sigmoid scores; the `top` largest of score + correction (lowest index on ties); weights = the plain scores"""
    s = logistic(h @ router.T)
    idx = np.argsort(-(s + correction), axis=-1, kind="stable")[:, :top]
    return idx, np.take_along_axis(s, idx, -1)


def clamped_expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ down.T


def mixture(h, W, p, mlp):
    idx, wgt = route(h, W[p + "router"], W[p + "correction"], mlp["router"]["top"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t], wgt[t]):
            q = p + "e%d." % e
            out[t] += w * clamped_expert(h[t:t + 1], W[q + "gate"], W[q + "up"], W[q + "down"], mlp["expert"]["limit"])[0]
    return out


def run_order(cfg):
    """(layer, pass or None) in the order the stack is walked"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["start"] >= loop["stop"] or loop["times"] < 1:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def layer(cfg, W, li, x):
    L, eps, p = cfg["layers"][li], cfg["norm"]["eps"], "l%d." % li
    h = dyt(x, W[p + "norm1.alpha"], W[p + "norm1"], W[p + "norm1.b"])
    mixer = attention_mixer if L["type"] == "attention" else general_delta_mixer
    x = x + mixer(h, W, p + "mix.", L["mixer"], eps)
    if L.get("mlp"):
        x = x + mixture(dyt(x, W[p + "norm2.alpha"], W[p + "norm2"], W[p + "norm2.b"]), W, p + "mlp.", L["mlp"])
    return x


def forward(cfg, W, tokens, taps=None):
    """logits [T, vocab] of one whole sequence; taps: a list that receives the residual after every layer run"""
    x0 = embed(cfg, W, tokens)
    x = x0.copy()
    for li, t in run_order(cfg):
        if t is not None and li == cfg["loop"]["start"]:
            x = x + (x0 if t > 0 else 0.0) + W["loop.step"][t]
        x = layer(cfg, W, li, x)
        if taps is not None:
            taps.append(x.copy())
    y = dyt(x, W["final.norm.alpha"], W["final.norm"], W["final.norm.b"])
    return (y @ W["head"].T) * float(cfg.get("logit_scale", 1.0))
