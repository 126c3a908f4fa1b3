"""Small Sopulorn configurations with random bfloat16 weights: config.json + model.safetensors in a directory for the engine, and the same
weights as float64 tensors for the oracle (tests/sopulorn_oracle.py)."""
import numpy as np

from tests import sopulorn_oracle as orc
from tests.gelarax_oracle import bf16_round
from tests.layered_fixtures import rel_err, write_model_dir      # noqa: F401  (the directory writer and the error measure are shared test helpers)


def dense(ff=80, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=6, top=2, ff=24, shared=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, rot_dims=None, base=10000.0, scale=None, kv_from=None, mlp="default"):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims},
          "scale": float(scale if scale is not None else dim ** -0.5)}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx, "mlp": moe() if mlp == "default" else mlp}


def config(layers, width=64, vocab=97, eps=1e-5, bigram=(53, 31, 5)):
    cfg = {"architecture": "Sopulorn", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return cfg


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        s["bigram"] = (bg["buckets"] + 1, W)
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        s.update({p + "norm1": (W,), p + "norm1b": (W,), p + "mix.q": (H * D, W), p + "mix.q.b": (H * D,), p + "mix.q.norm": (D,), p + "mix.o": (W, H * DV)})
        if m.get("kv_from") is None:
            s.update({p + "mix.k": (G * D, W), p + "mix.k.b": (G * D,), p + "mix.k.norm": (D,), p + "mix.v": (G * DV, W), p + "mix.v.b": (G * DV,)})
        mlp = L.get("mlp")
        if not mlp:
            continue
        s.update({p + "norm2": (W,), p + "norm2b": (W,)})
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            s.update({p + "mlp.gate": (F, W), p + "mlp.up": (F, W), p + "mlp.down": (W, F)})
        else:
            E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
            s.update({p + "mlp.router": (E, W), p + "mlp.router.b": (E,)})
            for e in range(E):
                s.update({p + "mlp.e%d.gate" % e: (F, W), p + "mlp.e%d.up" % e: (F, W), p + "mlp.e%d.down" % e: (W, F)})
            if mlp.get("shared"):
                S = mlp["shared"]["ff"]
                s.update({p + "mlp.shared.gate": (S, W), p + "mlp.shared.up": (S, W), p + "mlp.shared.down": (W, S), p + "mlp.shared.sg": (1, W)})
    return s


def random_weights(cfg, seed=0):
    """name -> float32 array of bfloat16-representable values"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
            a = 0.3 * rng.standard_normal(shape)                    # (the norm multiplies by one plus this)
            if leaf in ("norm1b", "norm2b"):
                a -= 0.5
        elif leaf == "norm":
            a = 1.0 + 0.3 * rng.standard_normal(shape)              # q / k norms: a plain weight
        elif leaf == "b":
            a = 0.5 * rng.standard_normal(shape)
        elif leaf == "router":
            a = rng.standard_normal(shape) * (3.0 / np.sqrt(shape[-1]))
        elif name in ("embed", "bigram"):
            a = rng.standard_normal(shape) * (1.0 if name == "embed" else 0.7)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = bf16_round(a.astype(np.float32))
    return out


def oracle_weights(weights):
    return {k: orc.t64(v) for k, v in weights.items()}
