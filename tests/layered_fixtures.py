"""Small Gelarax configurations with random bfloat16 weights for the tests of the layer-list worker: builds config.json +
model.safetensors in a directory, and the same weights as float64 tensors for the oracle (tests/gelarax_oracle.py)."""
import json
import os
import struct

import numpy as np

from tests import gelarax_oracle as orc


def parallel_layer(heads=4, kv_heads=2, dim=32, window=24, keep_first=3, scale=0.2, softcap=15.0, bias_max=40, lin_heads=2, lin_dim=16, lin_vdim=32,
                   decay=None, left_scale=0.9, right_scale=1.3, ff=96):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "softcap": softcap, "bias_max": bias_max,
                               "mask": {"size": window, "keep_first": keep_first}},
                      "right": {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "decay": decay or [0.5 + 0.49 * i / max(1, lin_heads - 1) for i in range(lin_heads)]},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, ff=96):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=64, vocab=97, eps=1e-5):
    return {"architecture": "Gelarax", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}


def tensor_shapes(cfg, buckets=12):
    W, V = cfg["width"], cfg["vocab"]
    s = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    for li, L in enumerate(cfg["layers"]):
        p = "l%d." % li
        s[p + "norm1"] = (W,); s[p + "ls1"] = (W,)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            s.update({p + "ls2": (W,), p + "mlp.gate": (F, W), p + "mlp.gate.b": (F,), p + "mlp.up": (F, W), p + "mlp.up.b": (F,), p + "mlp.down": (W, F),
                      p + "mlp.down.b": (W,)})
        m = L["mixer"]
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            nb = buckets[li] if isinstance(buckets, (list, tuple)) else buckets
            s.update({p + "mix.left.q": (a["heads"] * a["dim"], W), p + "mix.left.k": (a["kv_heads"] * a["dim"], W), p + "mix.left.rel": (nb, a["heads"]),
                      p + "mix.left.sink": (a["heads"],), p + "mix.left.o": (W, a["heads"] * a["dim"]),
                      p + "mix.right.q": (r["heads"] * r["dim"], W), p + "mix.right.k": (r["heads"] * r["dim"], W), p + "mix.right.v": (r["heads"] * r["vdim"], W),
                      p + "mix.right.g": (r["heads"] * r["vdim"], W), p + "mix.right.o": (W, r["heads"] * r["vdim"]), p + "mix.right.norm": (r["heads"] * r["vdim"],)})
        else:
            qk, dv = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            s.update({p + "mix.q": (qk, W), p + "mix.k": (qk, W), p + "mix.v": (dv, W), p + "mix.q.conv": (qk, m["conv"]), p + "mix.k.conv": (qk, m["conv"]),
                      p + "mix.v.conv": (dv, m["conv"]), p + "mix.b": (m["heads"], W), p + "mix.a": (m["heads"], W), p + "mix.A_log": (m["heads"],),
                      p + "mix.dt_bias": (m["heads"],), p + "mix.g": (dv, W), p + "mix.norm": (m["vdim"],), p + "mix.o": (W, dv)})
    return s


def random_weights(cfg, seed=0, buckets=12):
    """name -> float32 array of bfloat16-representable values"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, buckets).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm") and len(shape) == 1:
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf in ("ls1", "ls2"):
            a = 0.6 + 0.2 * rng.standard_normal(shape)
        elif leaf == "conv":
            a = 0.5 * rng.standard_normal(shape)
        elif leaf in ("rel", "sink", "b") and len(shape) <= 2 and (leaf != "b" or len(shape) == 1):
            a = 0.8 * rng.standard_normal(shape)
        elif leaf == "A_log":
            a = rng.uniform(-2.0, 0.5, shape)
        elif leaf == "dt_bias":
            a = rng.uniform(-1.0, 1.0, shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) * (1.5 / np.sqrt(shape[-1]))
        out[name] = orc.bf16_round(a.astype(np.float32))
    return out


def write_model_dir(path, cfg, weights):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name, a in weights.items():
        b = orc.bf16_bits(a).tobytes()
        header[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [off, off + len(b)]}
        blobs.append(b); off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj))); f.write(hj)
        for b in blobs:
            f.write(b)
    return path


def oracle_weights(weights):
    return {k: orc.t64(v) for k, v in weights.items()}


def rel_err(got, want):
    """rms over the vocabulary of the difference with its mean taken off, relative to the rms of the wanted logits"""
    d = np.asarray(got, np.float64) - np.asarray(want, np.float64)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, np.float64)
    w = w - w.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt((w * w).mean() + 1e-30)
