"""Plain float64 implementation of the Muzopel decoder, one function per mechanism, whole sequences only (no cache, no batching,
no portions).  It is what the tests compare the layer-list worker with; it shares no code with the product path.

A model: embedding -> grouped RMS norm -> layers -> grouped RMS norm -> head -> soft cap.  A layer, with x the residual:
    x <- x + gnorm1(mixer(x + conv1(x)));  x <- x + gnorm2(moe(x + conv2(x)));  X_(i+1) = x;  x <- sum_j dwa[j] X_j  (j <= i + 1)
"""
import math

import numpy as np
import torch

F64 = torch.float64


def t64(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float64))


def group_rms_norm(x, w, groups, eps):
    """the row in `groups` equal consecutive parts, each over its own root mean square, then the weight"""
    T, W = x.shape
    g = x.reshape(T, groups, W // groups)
    g = g / torch.sqrt((g * g).mean(-1, keepdim=True) + eps)
    return g.reshape(T, W) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def input_conv(h, w):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the sequence (w [width, taps]: the last tap is the current token)"""
    T, W = h.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, W, dtype=F64), h], 0)
    out = h.clone()
    for j in range(taps):
        out = out + w[:, j] * padded[j:j + T]
    return out


def rotation_tables(rot, T):
    """cos / sin [T, dims / 2] of angle p * f_i, f_i = base^(-2i / dims); with rot['scaling'] the YaRN blend and factor on cos / sin"""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        def dim_of(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / sc["factor"] * ramp + f * (1.0 - ramp)
        mult = 0.1 * math.log(sc["factor"]) + 1.0
    ang = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    return torch.cos(ang) * mult, torch.sin(ang) * mult


def rotate(x, cos, sin, dims):
    """x [T, ..., n]: pairs (2i, 2i + 1) of the first `dims` dimensions turn by the position's angle, the rest pass"""
    y = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    while cos.dim() < u.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    y[..., 0:dims:2] = u * cos - v * sin
    y[..., 1:dims:2] = v * cos + u * sin
    return y


def latent_attention_core(q, kv, P, pre, mx, first, eps, gate=None):
    """q [T, heads * (dim + rot_dim)] and kv [T, kv_rank + rot_dim] as projected: latent norm, key / value maps, rotation, causal
    softmax, gate (sigmoid of gate [T, heads]) -> [T, heads * vdim]"""
    T = q.shape[0]
    H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    q = q.reshape(T, H, dn + dr)
    c = rms_norm(kv[:, :R], P[pre + "dkv.norm"], eps)
    k_u = (c @ P[pre + "uk"].T).reshape(T, H, dn)
    v = (c @ P[pre + "uv"].T).reshape(T, H, dv)
    rot = dict(mx["rot"])
    if not first:
        rot.pop("scaling", None)
    cos, sin = rotation_tables(rot, T)
    q_r = rotate(q[..., dn:], cos, sin, rot["dims"])
    k_r = rotate(kv[:, R:], cos, sin, rot["dims"])
    s = (torch.einsum("thd,shd->hts", q[..., :dn], k_u) + torch.einsum("thd,sd->hts", q_r, k_r)) * mx["scale"]
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), -float("inf"))
    o = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v)
    if gate is not None:
        o = o * torch.sigmoid(gate)[:, :, None]
    return o.reshape(T, H * dv)


def latent_attention(h, P, pre, mx, kind, eps):
    """kind 'latent_attention': queries through a normed latent, gate per head; 'latent_attention_2': direct queries, no gate"""
    first = kind == "latent_attention"
    if first:
        q = rms_norm(h @ P[pre + "dq"].T, P[pre + "dq.norm"], eps) @ P[pre + "uq"].T
    else:
        q = h @ P[pre + "q"].T
    o = latent_attention_core(q, h @ P[pre + "dkv"].T, P, pre, mx, first, eps, h @ P[pre + "g"].T if first else None)
    return o @ P[pre + "o"].T


def route(z, correction, top):
    """scores = softmax(z); the `top` largest of scores + correction (lowest index on ties) with the plain scores as weights"""
    s = torch.softmax(z, -1)
    choice = (s + correction).clone()
    idx = []
    for _ in range(top):
        mx = choice.max(-1).values
        first = torch.stack([torch.nonzero(choice[t] == mx[t])[0, 0] for t in range(z.shape[0])])
        idx.append(first)
        choice[torch.arange(z.shape[0]), first] = -float("inf")
    idx = torch.stack(idx, -1)
    return idx, torch.gather(s, -1, idx)


def gelu_erf(a):
    return 0.5 * a * (1.0 + torch.erf(a / math.sqrt(2.0)))


def mixture(h, P, pre, mlp):
    E, I, top = mlp["router"]["experts"], mlp["router"].get("identity", 0), mlp["router"]["top"]
    idx, wgt = route(h @ P[pre + "router"].T, P[pre + "correction"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(idx[t, k])
            if e >= E:
                out[t] += wgt[t, k] * h[t]
            else:
                out[t] += wgt[t, k] * (P[pre + "e%d.down" % e] @ gelu_erf(P[pre + "e%d.up" % e] @ h[t]))
    return out


def forward(cfg, P, tokens, layers_out=None):
    """logits [T, vocab]; layers_out (a list) receives what every layer hands on (after its depth average)"""
    eps, G = cfg["norm"]["eps"], cfg["norm"]["groups"]
    taps = cfg.get("canon", {}).get("taps", 0)
    x = group_rms_norm(P["embed"][torch.as_tensor(tokens)], P["embed.norm"], G, eps)
    X = [x]
    for li, L in enumerate(cfg["layers"]):
        p = "l%d." % li
        h = input_conv(x, P[p + "canon1"]) if taps else x
        x = x + group_rms_norm(latent_attention(h, P, p + "mix.", L["mixer"], L["type"], eps), P[p + "norm1"], G, eps)
        if L.get("mlp"):
            h = input_conv(x, P[p + "canon2"]) if taps else x
            x = x + group_rms_norm(mixture(h, P, p + "mlp.", L["mlp"]), P[p + "norm2"], G, eps)
        X.append(x)
        x = sum(P[p + "dwa"][j] * X[j] for j in range(li + 2))
        if layers_out is not None:
            layers_out.append(x.clone())
    lg = group_rms_norm(x, P["final.norm"], G, eps) @ P["head"].T
    cap = cfg.get("logit_softcap", 0.0)
    return cap * torch.tanh(lg / cap) if cap else lg
