"""Plain float64 implementation of the Sopulorn decoder, one function per mechanism, whole sequences only (no cache, no batching, no
portions).  It is what the tests compare the layer-list worker with; it shares no code with the product path.

A model: x_t = E[tok_t] + B[pair_t]; layers; logits = head(norm(x)).  A layer, with x the residual and norm_w(y) = y / rms(y) * (1 + w):
    x <- x + norm_1b(attention(norm_1(x)));   x <- x + norm_2b(ffn(norm_2(x)))        (the second line only if the layer has a feed-forward)
"""
import numpy as np
import torch

F64 = torch.float64


def t64(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float64))


def rms_unit(y, eps):
    """y over its root mean square (eps inside the root), along the last axis"""
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def norm_one_plus(y, w, eps):
    """the norm of this design: the stored weight is what is added to one"""
    return rms_unit(y, eps) * (1.0 + w)


def pair_rows(tokens, buckets, mul_prev, mul_cur):
    """row of the token-pair table per position: the last row for a sequence's first token, else the hash of (previous, current)"""
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((int(a) * mul_prev + int(b) * mul_cur) % buckets)
    return rows


def embed(cfg, W, tokens):
    x = W["embed"][list(tokens)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + W["bigram"][pair_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


def rotate_half_layout(z, positions, dims, base):
    """z [T, heads, dim]: dimension i < dims / 2 turns together with dimension i + dims / 2 by the angle p * base^(-2 i / dims);
    dimensions from `dims` on pass unchanged"""
    if not dims:
        return z
    half = dims // 2
    f = float(base) ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    ang = torch.as_tensor(positions, dtype=F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    lo, hi = z[..., :half], z[..., half:dims]
    return torch.cat([lo * c - hi * s, hi * c + lo * s, z[..., dims:]], -1)


def queries(h, W, p, mx, eps, positions):
    T = h.shape[0]
    rot = mx.get("rot") or {}
    q = (h @ W[p + "mix.q"].T + W[p + "mix.q.b"]).reshape(T, mx["heads"], mx["dim"])
    q = rms_unit(q, eps) * W[p + "mix.q.norm"]
    return rotate_half_layout(q, positions, rot.get("dims", 0), rot.get("base", 1.0))


def keys_values(h, W, p, mx, eps, positions):
    """what a layer with projections of its own leaves in its cache: keys normed and rotated, values as projected"""
    T = h.shape[0]
    rot = mx.get("rot") or {}
    k = (h @ W[p + "mix.k"].T + W[p + "mix.k.b"]).reshape(T, mx["kv_heads"], mx["dim"])
    k = rotate_half_layout(rms_unit(k, eps) * W[p + "mix.k.norm"], positions, rot.get("dims", 0), rot.get("base", 1.0))
    v = (h @ W[p + "mix.v"].T + W[p + "mix.v.b"]).reshape(T, mx["kv_heads"], mx["vdim"])
    return k, v


def softmax_plus_one(s):
    """weights exp(s_j) / (1 + sum_j exp(s_j)) along the last axis (entries of -inf are masked out)"""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention_core(q, k, v, scale):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; causal; query head h reads key / value head h // (H / G)"""
    T, H, _ = q.shape
    G = k.shape[1]
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~causal, float("-inf"))
        out.append(softmax_plus_one(s) @ v[:, g])
    return torch.stack(out, 1).reshape(T, -1)


def dense_ffn(h, W, p, limit):
    g = torch.clamp(h @ W[p + "mlp.gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "mlp.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "mlp.down"].T


def gated_expert(h, w_gate, w_up, w_down):
    g = h @ w_gate.T
    return (g * torch.sigmoid(g) * (h @ w_up.T)) @ w_down.T


def route(h, W, p, top):
    """indices [T, top] of the largest router logits (lowest index first on ties) and the softmax over those logits only"""
    z = h @ W[p + "mlp.router"].T + W[p + "mlp.router.b"]
    idx = torch.argsort(-z, dim=-1, stable=True)[:, :top]
    return idx, torch.softmax(torch.gather(z, 1, idx), -1)


def moe_ffn(h, W, p, mlp):
    idx, wgt = route(h, W, p, mlp["router"]["top"])
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wgt[t]):
            pe = p + "mlp.e%d." % e
            y[t] = y[t] + a * gated_expert(h[t:t + 1], W[pe + "gate"], W[pe + "up"], W[pe + "down"])[0]
    if mlp.get("shared"):
        ps = p + "mlp.shared."
        y = y + gated_expert(h, W[ps + "gate"], W[ps + "up"], W[ps + "down"]) * torch.sigmoid(h @ W[ps + "sg"].reshape(1, -1).T)
    return y


def forward(cfg, W, tokens, residuals=None):
    """logits [T, vocab]; residuals (a list) receives the residual stream after every layer"""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    pos = list(range(T))
    x = embed(cfg, W, tokens)
    cache = {}
    for li, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % li, L["mixer"]
        h = norm_one_plus(x, W[p + "norm1"], eps)
        q = queries(h, W, p, mx, eps, pos)
        if mx.get("kv_from") is not None:
            k, v = cache[mx["kv_from"]]
        else:
            k, v = cache[li] = keys_values(h, W, p, mx, eps, pos)
        a = attention_core(q, k, v, mx["scale"]) @ W[p + "mix.o"].T
        x = x + norm_one_plus(a, W[p + "norm1b"], eps)
        mlp = L.get("mlp")
        if mlp:
            h = norm_one_plus(x, W[p + "norm2"], eps)
            y = dense_ffn(h, W, p, mlp["limit"]) if mlp["kind"] == "dense" else moe_ffn(h, W, p, mlp)
            x = x + norm_one_plus(y, W[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return norm_one_plus(x, W["final.norm"], eps) @ W["head"].T
