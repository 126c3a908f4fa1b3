"""Small Bogupel configurations with random bfloat16 weights: config.json + model.safetensors in a directory for the engine, and the same
weights as float64 arrays for the oracle (tests/bogupel_oracle.py)."""
import numpy as np

from tests import bogupel_oracle as orc
from tests.gelarax_oracle import bf16_round
from tests.layered_fixtures import rel_err, write_model_dir      # noqa: F401  (the directory writer and the error measure are shared test helpers)


def moe(experts=6, top=2, ff=24, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, rot_dims=None, base=10000.0, scale=None, window=20, scaling="default", mlp="default"):
    rot = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if scaling == "default":
        scaling = {"factor": 4.0, "low": 1.5, "high": 3.0, "original": 96}
    if scaling:
        rot["scaling"] = scaling
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": float(scale if scale is not None else 1.3 * dim ** -0.5),
          "mask": {"size": window}}
    return {"type": "attention", "mixer": mx, "mlp": moe() if mlp == "default" else mlp}


def delta_layer(heads=3, dim=16, rank=6, mlp="default"):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}, "mlp": moe() if mlp == "default" else mlp, "_rank": rank}


def config(layers, width=64, vocab=97, eps=1e-5, bigram=(53, 31, 5), embed_scale=3.0, logit_scale=0.7, loop=None):
    cfg = {"architecture": "Bogupel", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers, "logit_scale": logit_scale,
           "embedding": {"scale": embed_scale}}
    if bigram:
        cfg["embedding"]["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "final.norm.alpha": (), "head": (V, W)}
    bg = cfg["embedding"].get("bigram")
    if bg:
        s["bigram"] = (bg["buckets"] + 1, W)
    if cfg.get("loop"):
        s["loop.step"] = (cfg["loop"]["times"], W)
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        s.update({p + "norm1": (W,), p + "norm1.b": (W,), p + "norm1.alpha": ()})
        if L["type"] == "attention":
            H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            s.update({p + "mix.q": (H * D, W), p + "mix.q.b": (H * D,), p + "mix.q.norm": (D,), p + "mix.k": (G * D, W), p + "mix.k.b": (G * D,),
                      p + "mix.k.norm": (D,), p + "mix.v": (G * DV, W), p + "mix.v.b": (G * DV,), p + "mix.sink": (H,), p + "mix.o": (W, H * DV)})
        else:
            C, R = m["heads"] * m["dim"], L.get("_rank", 6)
            s.update({p + "mix.r": (C, W), p + "mix.k": (C, W), p + "mix.v": (C, W), p + "mix.g": (C, W), p + "mix.a": (C, W), p + "mix.a.b": (C,),
                      p + "mix.w1": (R, W), p + "mix.w2": (C, R), p + "mix.w0": (C,), p + "mix.norm": (C,), p + "mix.o": (W, C)})
        mlp = L.get("mlp")
        if not mlp:
            continue
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({p + "norm2": (W,), p + "norm2.b": (W,), p + "norm2.alpha": (), p + "mlp.router": (E, W), p + "mlp.correction": (E,)})
        for e in range(E):
            s.update({p + "mlp.e%d.gate" % e: (F, W), p + "mlp.e%d.up" % e: (F, W), p + "mlp.e%d.down" % e: (W, F)})
    return s


def random_weights(cfg, seed=0):
    """name -> float32 array of bfloat16-representable values"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf == "alpha":
            a = np.asarray(rng.uniform(0.4, 0.9))
        elif leaf in ("norm1", "norm2") or name == "final.norm" or leaf == "norm":
            a = 1.0 + 0.3 * rng.standard_normal(shape)
        elif leaf == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "sink":
            a = rng.standard_normal(shape)
        elif leaf == "correction":
            a = 0.2 * rng.standard_normal(shape)
        elif leaf == "w0":
            a = rng.standard_normal(shape) * 1.5
        elif leaf == "router":
            a = rng.standard_normal(shape) * (3.0 / np.sqrt(shape[-1]))
        elif leaf == "step":
            a = 0.5 * rng.standard_normal(shape)
        elif name in ("embed", "bigram"):
            a = rng.standard_normal(shape) * (0.4 if name == "embed" else 0.7)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = bf16_round(np.asarray(a, dtype=np.float32))
    return out


def clean(cfg):
    """the configuration as it goes into config.json (the fixtures' own notes taken out)"""
    c = dict(cfg)
    c["layers"] = [{k: v for k, v in L.items() if not k.startswith("_")} for L in cfg["layers"]]
    return c


def oracle_weights(weights):
    return {k: orc.f64(v) for k, v in weights.items()}
