"""Small Muzopel configurations with random bfloat16 weights: config.json + model.safetensors in a directory for the engine, and the same
weights as float64 tensors for the oracle (tests/muzopel_oracle.py)."""
import numpy as np

from tests import muzopel_oracle as orc
from tests.gelarax_oracle import bf16_round
from tests.layered_fixtures import rel_err, write_model_dir      # noqa: F401  (the directory writer and the error measure are shared test helpers)


def moe(experts=6, identity=2, top=3, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}


def latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=32, q_rank=20, rot_dims=None, base=10000.0, scale=None, scaling="default", mlp="default"):
    """type latent_attention: queries through a latent, YaRN scaling (None: plain rotation), gate per head"""
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot,
                      "scale": scale if scale is not None else 1.0 / np.sqrt(dim + rot_dim)},
            "mlp": moe() if mlp == "default" else mlp}


def latent2_layer(heads=4, dim=16, rot_dim=16, vdim=40, kv_rank=24, base=50000.0, scale=None, mlp="default"):
    """type latent_attention_2: direct queries, plain rotation, no gate"""
    return {"type": "latent_attention_2",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": {"base": base, "dims": rot_dim},
                      "scale": scale if scale is not None else 1.0 / np.sqrt(dim + rot_dim)},
            "mlp": moe() if mlp == "default" else mlp}


def config(layers, width=64, vocab=97, eps=1e-6, groups=2, taps=4, softcap=12.0):
    return {"architecture": "Muzopel", "width": width, "vocab": vocab, "norm": {"eps": eps, "groups": groups}, "canon": {"taps": taps},
            "logit_softcap": softcap, "layers": layers}


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    taps = cfg.get("canon", {}).get("taps", 0)
    s = {"embed": (V, W), "embed.norm": (W,), "final.norm": (W,), "head": (V, W)}
    for li, L in enumerate(cfg["layers"]):
        p, m = "l%d." % li, L["mixer"]
        H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        s[p + "norm1"] = (W,); s[p + "dwa"] = (li + 2,)
        if taps:
            s[p + "canon1"] = (W, taps)
        if L["type"] == "latent_attention":
            s.update({p + "mix.dq": (m["q_rank"], W), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (H * (dn + dr), m["q_rank"]), p + "mix.g": (H, W)})
        else:
            s[p + "mix.q"] = (H * (dn + dr), W)
        s.update({p + "mix.dkv": (R + dr, W), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * dn, R), p + "mix.uv": (H * dv, R), p + "mix.o": (W, H * dv)})
        if L.get("mlp"):
            r, F = L["mlp"]["router"], L["mlp"]["expert"]["ff"]
            n_all = r["experts"] + r.get("identity", 0)
            s[p + "norm2"] = (W,)
            if taps:
                s[p + "canon2"] = (W, taps)
            s[p + "mlp.router"] = (n_all, W); s[p + "mlp.correction"] = (n_all,)
            for e in range(r["experts"]):
                s[p + "mlp.e%d.up" % e] = (F, W); s[p + "mlp.e%d.down" % e] = (W, F)
    return s


def random_weights(cfg, seed=0):
    """name -> float32 array of bfloat16-representable values"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm", "norm1", "norm2"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
            if leaf in ("norm1", "norm2"):
                a *= 0.5
        elif leaf in ("canon1", "canon2"):
            a = 0.4 * rng.standard_normal(shape)
        elif leaf == "dwa":
            a = np.full(shape, 0.3 / shape[0]) + 0.1 * rng.standard_normal(shape)
            a[-1] += 0.7
        elif leaf == "correction":
            a = 0.05 * rng.standard_normal(shape)
        elif leaf == "router":
            a = rng.standard_normal(shape) * (3.0 / np.sqrt(shape[-1]))
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = bf16_round(a.astype(np.float32))
    return out


def oracle_weights(weights):
    return {k: orc.t64(v) for k, v in weights.items()}
