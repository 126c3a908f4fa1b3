"""Synthetic models for measurement and parity tests:
fp16 source tensors N(0, 0.02) from seed = 1000 + layer*16 + tensor_id, norm
weights = 1, quantised on the device with the reference rule; tensors below
tensor_quant_threshold stay F16 (src/transformer/network_builder.cc:1557-1562),
lm_head stays F16 (network_builder.cc:825-846)."""
import torch

from . import dtypes as dt
from . import worker as W

SHAPES = {
    # data/models/llama2_7b_chat_hf/model_spec.json + config: d=4096 L=32 H=32 ffn=11008 vocab=32000
    "llama2_7b": dict(dim=4096, layers=32, heads=32, kv_heads=32, head_dim=128, ffn=11008, vocab=32000),
    # bin/llm_inference.tiny.ini shape (stories15M)
    "tiny15m": dict(dim=288, layers=6, heads=6, kv_heads=6, head_dim=48, ffn=768, vocab=32000),
    "test_tiny": dict(dim=288, layers=2, heads=6, kv_heads=6, head_dim=48, ffn=768, vocab=1000),   # stories15M layers, small vocabulary
    # small GQA shapes for parity tests
    "test_gqa": dict(dim=256, layers=2, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=1000),
    "test_mha": dict(dim=256, layers=3, heads=8, kv_heads=8, head_dim=32, ffn=640, vocab=777),
    # w2 rows longer than one 4096-column chunk of the rows GEMM (chunk loop / whole-row staging)
    "test_longffn": dict(dim=256, layers=2, heads=4, kv_heads=4, head_dim=64, ffn=4352, vocab=500),
    # data/models/yi_34b_chat (configs[3]) and a Llama-2-70B-shaped model: w2 rows of 20480 / 28672 columns
    "yi_34b": dict(dim=7168, layers=60, heads=56, kv_heads=8, head_dim=128, ffn=20480, vocab=64000),
    "llama2_70b": dict(dim=8192, layers=80, heads=64, kv_heads=8, head_dim=128, ffn=28672, vocab=32000),
    # data/models/falcon_40b_instruct (configs[3]): LayerNorm, GELU, plain (non-gated) MLP, attention and MLP both read
    # the layer input through their own norm (mlp_attn_share_input), 128 heads of 64 over 8 KV heads
    "falcon_40b": dict(dim=8192, layers=60, heads=128, kv_heads=8, head_dim=64, ffn=32768, vocab=65024,
                       norm_kind=1, act_kind=1, is_glu=0, share_input=1, rope_order=2),
    # Mixtral-8x7B (data/models/mixtral_8x7b_instruct_v0.1) and a small MoE shape for parity tests
    "mixtral_8x7b": dict(dim=4096, layers=32, heads=32, kv_heads=8, head_dim=128, ffn=14336, vocab=32000, experts=8, moe_top_k=2),
    "test_moe": dict(dim=256, layers=2, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=1000, experts=4, moe_top_k=2),
    "test_moe_longffn": dict(dim=256, layers=2, heads=4, kv_heads=2, head_dim=64, ffn=4352, vocab=600, experts=4, moe_top_k=2),
    # a small Falcon-40B-like wiring (LayerNorm, GELU, plain MLP, shared MLP / attention input, grouped KV heads)
    "test_falcon": dict(dim=256, layers=2, heads=8, kv_heads=2, head_dim=32, ffn=512, vocab=1000,
                        norm_kind=1, act_kind=1, is_glu=0, share_input=1, rope_order=2),
}

MATRICES = [(W.T_WQ, "q"), (W.T_WK, "kv"), (W.T_WV, "kv"), (W.T_WO, "o"), (W.T_W1, "up"), (W.T_W3, "up"), (W.T_W2, "down")]
TENSOR_QUANT_THRESHOLD = 4000000   # ModelSpec::tensor_quant_threshold (src/transformer/model.h:137)


def _shape(kind, s):
    qd, kvd = s["heads"] * s["head_dim"], s["kv_heads"] * s["head_dim"]
    return {"q": (qd, s["dim"]), "kv": (kvd, s["dim"]), "o": (s["dim"], qd),
            "up": (s["ffn"], s["dim"]), "down": (s["dim"], s["ffn"])}[kind]


def gen_f16(shape, seed, std=0.02, device="cuda"):
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return (torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std).half()


def build(shape_name, wdtype=dt.Q4_B32T1A, kv_dtype=dt.F16, max_ctx=1024, quant_threshold=TENSOR_QUANT_THRESHOLD,
          std=0.02, keep_host=False, device=0, embd_std=None, tied_lm_head=None, **overrides):
    """Returns (worker, host_tensors or None).  host_tensors: {(layer, tid): (dtype, np array, rows, cols)}.
    embd_std / tied_lm_head = (permutation seed, scale): the "peaky" model of the free-running parity test -- embedding rows of std
    embd_std (the token's own row then carries through the residual stream) and lm_head[v] = scale * embedding[perm[v]]: the logit
    of the one row aligned with the current token's embedding stands several logit-std above the rest, so greedy ids are well
    separated although every layer is random (next token = perm^-1(current): a walk along a cycle of the permutation)."""
    s = dict(SHAPES[shape_name])
    s.update({k: v for k, v in overrides.items() if k in s})
    extra = {k: v for k, v in overrides.items() if k not in s}
    wk = W.DecodeWorker(max_ctx=max_ctx, kv_dtype=kv_dtype, device=device, **s, **extra)
    host = {} if keep_host else None
    dev = "cuda:%d" % device

    def put(layer, tid, target, t16, expert=-1):
        rows, cols = (1, t16.numel()) if t16.dim() == 1 else t16.shape
        wk.set_tensor_f16(layer, tid, target, t16, rows, cols, expert=expert)
        if keep_host:
            key = (layer, tid) if expert < 0 else (layer, tid, expert)
            host[key] = (target, t16.cpu().view(torch.int16).numpy().view("float16").copy(), rows, cols)

    embd = gen_f16((s["vocab"], s["dim"]), 999, std if embd_std is None else embd_std, dev)
    put(-1, W.T_EMBD, dt.F16, embd)
    put(-1, W.T_OUT_NORM, dt.F16, torch.ones(s["dim"], dtype=torch.float16, device=dev))
    if tied_lm_head is None:
        put(-1, W.T_LM_HEAD, dt.F16, gen_f16((s["vocab"], s["dim"]), 998, std, dev))
    else:
        pg = torch.Generator(device="cpu"); pg.manual_seed(int(tied_lm_head[0]))
        perm = torch.randperm(s["vocab"], generator=pg).to(dev)
        put(-1, W.T_LM_HEAD, dt.F16, (embd[perm].float() * float(tied_lm_head[1])).half())
    del embd
    for layer in range(s["layers"]):
        put(layer, W.T_ATTN_NORM, dt.F16, torch.ones(s["dim"], dtype=torch.float16, device=dev))
        put(layer, W.T_FFN_NORM, dt.F16, torch.ones(s["dim"], dtype=torch.float16, device=dev))
        n_exp = s.get("experts", 0)
        for tid, kind in MATRICES:
            if tid == W.T_W3 and not s.get("is_glu", 1):
                continue
            rows, cols = _shape(kind, s)
            target = wdtype if rows * cols >= quant_threshold else dt.F16
            if n_exp and tid in (W.T_W1, W.T_W2, W.T_W3):       # one FFN per expert (ProcessGpuLayer_Moe)
                for e in range(n_exp):
                    put(layer, tid, target, gen_f16((rows, cols), 100000 + (layer * 64 + e) * 16 + tid, std, dev), expert=e)
                continue
            t16 = gen_f16((rows, cols), 1000 + layer * 16 + tid, std, dev)
            put(layer, tid, target, t16)
        if n_exp:   # router: always F16 (far below tensor_quant_threshold)
            put(layer, W.T_MOE_GATE, dt.F16, gen_f16((n_exp, s["dim"]), 1000 + layer * 16 + W.T_MOE_GATE, std, dev))
    wk.finalize()
    return wk, host, s


def weight_bytes(shape_name, wdtype=dt.Q4_B32T1A, quant_threshold=TENSOR_QUANT_THRESHOLD, streamed=False):
    """Algorithmic weight bytes per decoded token, excluding KV.  streamed=True: the bytes of the layout
    the decode kernels read (differs from the reference block bytes for Q3H_B64T1 only: 36 vs 32 per 64 weights)."""
    s = SHAPES[shape_name]
    per_layer = 0
    for tid, kind in MATRICES:
        if tid == W.T_W3 and not s.get("is_glu", 1):
            continue
        rows, cols = _shape(kind, s)
        d = wdtype if rows * cols >= quant_threshold else dt.F16
        n = rows * (dt.streamed_row_bytes(d, cols) if streamed else dt.row_bytes(d, cols))
        if s.get("experts", 0) and tid in (W.T_W1, W.T_W2, W.T_W3):
            n *= s["moe_top_k"]                  # a token streams its top-k experts only
        per_layer += n
    if s.get("experts", 0):
        per_layer += s["experts"] * s["dim"] * 2     # F16 router
    lm_head = s["vocab"] * s["dim"] * 2
    return per_layer * s["layers"] + lm_head


def kv_bytes_per_ctx_row(shape_name, kv_dtype=dt.F16):
    s = SHAPES[shape_name]
    return s["layers"] * 2 * dt.row_bytes(kv_dtype, s["kv_heads"] * s["head_dim"])


# ---------------------------------------------------------------- layer-list models (Gelarax) with random weights
def gelarax_config(width=2048, ff=5632, blocks=2, vocab=32000, heads=16, kv_heads=4, dim=128, window=1024, keep_first=4, lin_heads=16, lin_dim=64,
                   lin_vdim=128, delta_heads=16, delta_kv_heads=8, delta_dim=128, delta_vdim=128, conv=4):
    """`blocks` x (three windowed + linear attention layers, one gated delta rule layer), each with a gated feed-forward"""
    par = {"type": "parallel",
           "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5 * 8, "softcap": 30.0, "bias_max": 4 * window,
                              "mask": {"size": window, "keep_first": keep_first}},
                     "right": {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "decay": [1.0 - 2.0 ** (-3 - 7 * i / max(1, lin_heads - 1)) for i in range(lin_heads)]},
                     "left_scale": 1.0, "right_scale": 1.0},
           "mlp": {"kind": "dense", "ff": ff}}
    dl = {"type": "delta", "mixer": {"heads": delta_heads, "kv_heads": delta_kv_heads, "dim": delta_dim, "vdim": delta_vdim, "conv": conv},
          "mlp": {"kind": "dense", "ff": ff}}
    return {"architecture": "Gelarax", "width": width, "vocab": vocab, "norm": {"eps": 1e-6}, "layers": [par, par, par, dl] * blocks}


def gelarax_tensor_shapes(cfg, buckets=32):
    W_, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W_), "final.norm": (W_,), "head": (V, W_)}
    for li, L in enumerate(cfg["layers"]):
        p = "l%d." % li
        s[p + "norm1"] = (W_,); s[p + "ls1"] = (W_,)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            s.update({p + "ls2": (W_,), p + "mlp.gate": (F, W_), p + "mlp.gate.b": (F,), p + "mlp.up": (F, W_), p + "mlp.up.b": (F,), p + "mlp.down": (W_, F),
                      p + "mlp.down.b": (W_,)})
        m = L["mixer"]
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            s.update({p + "mix.left.q": (a["heads"] * a["dim"], W_), p + "mix.left.k": (a["kv_heads"] * a["dim"], W_), p + "mix.left.rel": (buckets, a["heads"]),
                      p + "mix.left.sink": (a["heads"],), p + "mix.left.o": (W_, a["heads"] * a["dim"]),
                      p + "mix.right.q": (r["heads"] * r["dim"], W_), p + "mix.right.k": (r["heads"] * r["dim"], W_), p + "mix.right.v": (r["heads"] * r["vdim"], W_),
                      p + "mix.right.g": (r["heads"] * r["vdim"], W_), p + "mix.right.o": (W_, r["heads"] * r["vdim"]), p + "mix.right.norm": (r["heads"] * r["vdim"],)})
        else:
            qk, dv = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            s.update({p + "mix.q": (qk, W_), p + "mix.k": (qk, W_), p + "mix.v": (dv, W_), p + "mix.q.conv": (qk, m["conv"]), p + "mix.k.conv": (qk, m["conv"]),
                      p + "mix.v.conv": (dv, m["conv"]), p + "mix.b": (m["heads"], W_), p + "mix.a": (m["heads"], W_), p + "mix.A_log": (m["heads"],),
                      p + "mix.dt_bias": (m["heads"],), p + "mix.g": (dv, W_), p + "mix.norm": (m["vdim"],), p + "mix.o": (W_, dv)})
    return s


def muzopel_config(width=2048, blocks=2, vocab=32000, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=768, experts=32, identity=2, top=6, ff=1408,
                   taps=4, groups=8):
    """`blocks` x (three latent-attention layers with direct queries, one with latent queries, YaRN rotation and head gates), each with a
    mixture of experts behind it"""
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    scale = float((dim + rot_dim) ** -0.5)
    two = {"type": "latent_attention_2", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                                                   "rot": {"base": 10000.0, "dims": rot_dim}}, "mlp": mlp}
    one = {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                                                 "rot": {"base": 10000.0, "dims": rot_dim, "scaling": {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}}},
           "mlp": mlp}
    return {"architecture": "Muzopel", "width": width, "vocab": vocab, "norm": {"eps": 1e-6, "groups": groups}, "canon": {"taps": taps}, "logit_softcap": 30.0,
            "layers": [two, two, two, one] * blocks}


def muzopel_tensor_shapes(cfg):
    W_, V = cfg["width"], cfg["vocab"]
    taps = cfg.get("canon", {}).get("taps", 0)
    s = {"embed": (V, W_), "embed.norm": (W_,), "final.norm": (W_,), "head": (V, W_)}
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        s[p + "norm1"] = (W_,); s[p + "dwa"] = (li + 2,)
        if taps:
            s[p + "canon1"] = (W_, taps)
        if L["type"] == "latent_attention":
            s.update({p + "mix.dq": (m["q_rank"], W_), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (H * (dn + dr), m["q_rank"]), p + "mix.g": (H, W_)})
        else:
            s[p + "mix.q"] = (H * (dn + dr), W_)
        s.update({p + "mix.dkv": (R + dr, W_), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * dn, R), p + "mix.uv": (H * dv, R), p + "mix.o": (W_, H * dv)})
        if L.get("mlp"):
            r, F = L["mlp"]["router"], L["mlp"]["expert"]["ff"]
            s[p + "norm2"] = (W_,)
            if taps:
                s[p + "canon2"] = (W_, taps)
            s[p + "mlp.router"] = (r["experts"] + r.get("identity", 0), W_); s[p + "mlp.correction"] = (r["experts"] + r.get("identity", 0),)
            for e in range(r["experts"]):
                s[p + "mlp.e%d.up" % e] = (F, W_); s[p + "mlp.e%d.down" % e] = (W_, F)
    return s


def sopulorn_config(width=2048, blocks=2, vocab=32000, heads=16, kv_heads=4, dim=128, vdim=128, rot_dims=64, dense_ff=5632, experts=32, top=6, ff=1408, shared_ff=2816):
    """`blocks` x (one layer with the clamped dense feed-forward, three with a mixture of gated experts + a shared expert; the last two of each
    block read the keys and values of the block's second layer)"""
    def layer(mlp, kv_from=None):
        mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(dim ** -0.5), "rot": {"base": 10000.0, "dims": rot_dims}}
        if kv_from is not None:
            mx["kv_from"] = kv_from
        return {"type": "attention", "mixer": mx, "mlp": mlp}
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}, "shared": {"ff": shared_ff}}
    layers = []
    for b in range(blocks):
        layers += [layer({"kind": "dense", "ff": dense_ff, "limit": 7.0}), layer(moe), layer(moe, 4 * b + 1), layer(moe, 4 * b + 1)]
    return {"architecture": "Sopulorn", "width": width, "vocab": vocab, "norm": {"eps": 1e-6}, "embedding": {"bigram": {"buckets": 65521, "mul_prev": 31337, "mul_cur": 7919}},
            "layers": layers}


def sopulorn_tensor_shapes(cfg):
    W_, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W_), "final.norm": (W_,), "head": (V, W_)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        s["bigram"] = (bg["buckets"] + 1, W_)
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        s.update({p + "norm1": (W_,), p + "norm1b": (W_,), p + "mix.q": (H * D, W_), p + "mix.q.b": (H * D,), p + "mix.q.norm": (D,), p + "mix.o": (W_, H * DV)})
        if m.get("kv_from") is None:
            s.update({p + "mix.k": (G * D, W_), p + "mix.k.b": (G * D,), p + "mix.k.norm": (D,), p + "mix.v": (G * DV, W_), p + "mix.v.b": (G * DV,)})
        mlp = L.get("mlp")
        if not mlp:
            continue
        s.update({p + "norm2": (W_,), p + "norm2b": (W_,)})
        if mlp["kind"] == "dense":
            s.update({p + "mlp.gate": (mlp["ff"], W_), p + "mlp.up": (mlp["ff"], W_), p + "mlp.down": (W_, mlp["ff"])})
            continue
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({p + "mlp.router": (E, W_), p + "mlp.router.b": (E,)})
        for e in range(E):
            s.update({p + "mlp.e%d.gate" % e: (F, W_), p + "mlp.e%d.up" % e: (F, W_), p + "mlp.e%d.down" % e: (W_, F)})
        if mlp.get("shared"):
            S = mlp["shared"]["ff"]
            s.update({p + "mlp.shared.gate": (S, W_), p + "mlp.shared.up": (S, W_), p + "mlp.shared.down": (W_, S), p + "mlp.shared.sg": (1, W_)})
    return s


def bogupel_config(width=2048, vocab=32000, heads=16, kv_heads=4, dim=128, vdim=128, rot_dims=64, window=1024, delta_heads=16, delta_dim=128, rank=64, experts=32, top=6,
                   ff=1408):
    """six layers, eight layer runs: attention, delta rule, a looped group of (attention, delta rule) that runs twice, attention, attention; a mixture of clamped
    gated experts in every layer"""
    moe = {"kind": "moe", "expert": {"ff": ff, "limit": 7.0}, "router": {"experts": experts, "top": top}}
    att = {"type": "attention", "mlp": moe,
           "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(dim ** -0.5), "mask": {"size": window},
                     "rot": {"base": 10000.0, "dims": rot_dims, "scaling": {"factor": 32.0, "low": 1.0, "high": 4.0, "original": 8192}}}}
    dlt = {"type": "general_delta", "mlp": moe, "mixer": {"heads": delta_heads, "dim": delta_dim}, "_rank": rank}
    return {"architecture": "Bogupel", "width": width, "vocab": vocab, "norm": {"eps": 1e-6}, "logit_scale": 0.25, "loop": {"start": 2, "stop": 4, "times": 2},
            "embedding": {"scale": 4.0, "bigram": {"buckets": 65521, "mul_prev": 31337, "mul_cur": 7919}}, "layers": [att, dlt, att, dlt, att, att]}


def bogupel_tensor_shapes(cfg):
    W_, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W_), "final.norm": (W_,), "final.norm.b": (W_,), "final.norm.alpha": (), "head": (V, W_)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        s["bigram"] = (bg["buckets"] + 1, W_)
    if cfg.get("loop"):
        s["loop.step"] = (cfg["loop"]["times"], W_)
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        s.update({p + "norm1": (W_,), p + "norm1.b": (W_,), p + "norm1.alpha": ()})
        if L["type"] == "attention":
            H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            s.update({p + "mix.q": (H * D, W_), p + "mix.q.b": (H * D,), p + "mix.q.norm": (D,), p + "mix.k": (G * D, W_), p + "mix.k.b": (G * D,), p + "mix.k.norm": (D,),
                      p + "mix.v": (G * DV, W_), p + "mix.v.b": (G * DV,), p + "mix.sink": (H,), p + "mix.o": (W_, H * DV)})
        else:
            C, R = m["heads"] * m["dim"], L.get("_rank", 64)
            s.update({p + "mix.r": (C, W_), p + "mix.k": (C, W_), p + "mix.v": (C, W_), p + "mix.g": (C, W_), p + "mix.a": (C, W_), p + "mix.a.b": (C,), p + "mix.w1": (R, W_),
                      p + "mix.w2": (C, R), p + "mix.w0": (C,), p + "mix.norm": (C,), p + "mix.o": (W_, C)})
        mlp = L.get("mlp")
        if not mlp:
            continue
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({p + "norm2": (W_,), p + "norm2.b": (W_,), p + "norm2.alpha": (), p + "mlp.router": (E, W_), p + "mlp.correction": (E,)})
        for e in range(E):
            s.update({p + "mlp.e%d.gate" % e: (F, W_), p + "mlp.e%d.up" % e: (F, W_), p + "mlp.e%d.down" % e: (W_, F)})
    return s


def write_bogupel_dir(path, cfg, seed=0):
    clean = dict(cfg)
    clean["layers"] = [{k: v for k, v in L.items() if not k.startswith("_")} for L in cfg["layers"]]
    return write_gelarax_dir(path, clean, seed, bogupel_tensor_shapes(cfg))


def write_sopulorn_dir(path, cfg, seed=0):
    return write_gelarax_dir(path, cfg, seed, sopulorn_tensor_shapes(cfg))


def write_muzopel_dir(path, cfg, seed=0):
    return write_gelarax_dir(path, cfg, seed, muzopel_tensor_shapes(cfg))


def write_gelarax_dir(path, cfg, seed=0, shapes=None):
    """config.json + model.safetensors (bfloat16, N(0, 1/fan_in) matrices, norm weights and layer scales near 1) for measurements"""
    import json
    import os
    import struct
    import numpy as np
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    rng = np.random.default_rng(seed)
    if shapes is None:
        shapes = gelarax_tensor_shapes(cfg)
    header, off = {}, 0
    for name, shape in shapes.items():
        n = int(np.prod(shape)) * 2
        header[name] = {"dtype": "BF16", "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj))); f.write(hj)
        for name, shape in shapes.items():
            leaf = name.split(".")[-1]
            if cfg.get("architecture") == "Sopulorn" and len(shape) == 1 and (leaf in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm"):
                a = 0.05 * rng.standard_normal(shape, dtype=np.float32)          # (this design's norms multiply by one plus the stored weight)
            elif len(shape) == 1 and leaf in ("norm1", "norm2", "norm", "ls1", "ls2"):
                a = 1.0 + 0.05 * rng.standard_normal(shape, dtype=np.float32)
            elif leaf == "alpha":
                a = np.full(shape, 0.5, np.float32)          # (the scalar of an element-wise tanh norm)
            elif leaf == "dwa":
                a = np.full(shape, 1.0 / shape[0], np.float32)
            elif leaf == "correction":
                a = 0.01 * rng.standard_normal(shape, dtype=np.float32)
            elif leaf in ("canon1", "canon2"):
                a = 0.2 * rng.standard_normal(shape, dtype=np.float32)
            elif leaf == "A_log":
                a = rng.uniform(-3.0, 0.0, shape).astype(np.float32)
            elif len(shape) == 1 or leaf in ("rel", "conv"):
                a = 0.3 * rng.standard_normal(shape, dtype=np.float32)
            else:
                a = rng.standard_normal(shape, dtype=np.float32) * np.float32(1.0 / np.sqrt(shape[-1]))
            f.write((np.ascontiguousarray(a).view(np.uint32) >> 16).astype(np.uint16).tobytes())
    return path
