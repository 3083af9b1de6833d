"""Plain, slow float64 implementation of the Gelarax design, one function per mechanism, for the tests of the
layer-list worker.  It shares no code with the product path: whole sequences only, python loops over time for
every recurrence, dense [T, T] masks for the attention.

Notation: x [T, W] residual, h = norm(x), weights W_* as [out, in] matrices applied as h @ W.T.
"""
import math

import numpy as np
import torch

F64 = torch.float64


def bf16_round(a):
    """float array -> nearest bfloat16 values (round to nearest even), as float32."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return (u & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(a.shape)


def bf16_bits(a):
    return (np.ascontiguousarray(bf16_round(a)).view(np.uint32) >> 16).astype(np.uint16)


def t64(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float64))


def sinusoid(positions, width, base=10000.0):
    """pe[p, 2i] = sin(p * base^(-2i/width)), pe[p, 2i+1] = cos(same)."""
    p = torch.as_tensor(positions, dtype=F64)[:, None]
    even = torch.arange(0, width, 2, dtype=F64)
    ang = p * base ** (-even / width)
    pe = torch.zeros(len(positions), width, dtype=F64)
    pe[:, 0::2] = torch.sin(ang)[:, :pe[:, 0::2].shape[1]]
    pe[:, 1::2] = torch.cos(ang)[:, :pe[:, 1::2].shape[1]]
    return pe


def layer_norm_nobias(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * w


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gated_ffn(h, w_gate, b_gate, w_up, b_up, w_down, b_down):
    return (gelu_tanh(h @ w_gate.T + b_gate) * (h @ w_up.T + b_up)) @ w_down.T + b_down


def distance_bucket(n, n_rows, d_max):
    half = n_rows // 2
    if n < half:
        return n
    return min(n_rows - 1, half + int(math.floor(math.log(n / half) / math.log(d_max / half) * (n_rows - half))))


def visible(T, window, keep_first):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def windowed_attention(q, k, heads, kv_heads, dim, scale, softcap, window, keep_first, rel, d_max, sink, eps):
    """q [T, heads*dim], k [T, kv_heads*dim] as projected; the values are k as projected.  Returns [T, heads*dim]."""
    T = q.shape[0]
    q = q.reshape(T, heads, dim)
    k = k.reshape(T, kv_heads, dim)
    qn, kn = rms_unit(q, eps), rms_unit(k, eps)
    n_rows = rel.shape[0]
    bk = torch.tensor([[distance_bucket(i - j, n_rows, d_max) if j <= i else 0 for j in range(T)] for i in range(T)])
    vis = visible(T, window, keep_first)
    out = torch.zeros(T, heads, dim, dtype=F64)
    group = heads // kv_heads
    for hh in range(heads):
        g = hh // group
        s = qn[:, hh] @ kn[:, g].T * scale
        s = softcap * torch.tanh(s / softcap)
        s = s + rel[bk, hh]
        e = torch.where(vis, torch.exp(s), torch.zeros_like(s))
        den = e.sum(-1, keepdim=True) + torch.exp(sink[hh])
        out[:, hh] = (e / den) @ k[:, g]
    return out.reshape(T, heads * dim)


def decayed_linear_attention(q, k, v, heads, dk, dv, decay):
    """q, k [T, heads*dk], v [T, heads*dv] after their activations.  S_t = d S_{t-1} + k_t v_t^T; o_t = S_t^T q_t."""
    T = q.shape[0]
    q, k, v = q.reshape(T, heads, dk), k.reshape(T, heads, dk), v.reshape(T, heads, dv)
    o = torch.zeros(T, heads, dv, dtype=F64)
    for hh in range(heads):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = decay[hh] * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    return o.reshape(T, heads * dv)


def short_conv(x, w):
    """x [T, C]; w [C, taps], last column multiplies the current token; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return y


def unit_vectors(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def delta_gates(b, a, a_log, dt_bias):
    beta = torch.sigmoid(b)
    g = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(a + dt_bias))
    return beta, g


def gated_delta_rule(q, k, v, beta, g, heads, kv_heads, dk, dv):
    """q, k [T, kv_heads*dk] (unit vectors, q scaled), v [T, heads*dv], beta, g [T, heads]."""
    T = q.shape[0]
    q, k, v = q.reshape(T, kv_heads, dk), k.reshape(T, kv_heads, dk), v.reshape(T, heads, dv)
    o = torch.zeros(T, heads, dv, dtype=F64)
    group = heads // kv_heads
    for hh in range(heads):
        kh = hh // group
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hh] = S.T @ q[t, kh]
    return o.reshape(T, heads * dv)


def mixer_parallel(h, w, p, m, eps):
    a, r = m["left"], m["right"]
    left = windowed_attention(h @ w[p + "left.q"].T, h @ w[p + "left.k"].T, a["heads"], a["kv_heads"], a["dim"], a["scale"], a["softcap"],
                              a["mask"]["size"], a["mask"]["keep_first"], w[p + "left.rel"], a["bias_max"], w[p + "left.sink"], eps) @ w[p + "left.o"].T
    o = decayed_linear_attention(silu(h @ w[p + "right.q"].T), silu(h @ w[p + "right.k"].T), silu(h @ w[p + "right.v"].T), r["heads"], r["dim"],
                                 r["vdim"], r["decay"])
    o = rms_unit(o, eps) * w[p + "right.norm"] * torch.sigmoid(h @ w[p + "right.g"].T)
    return m["left_scale"] * left + m["right_scale"] * (o @ w[p + "right.o"].T)


def mixer_delta(h, w, p, m, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, dk)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, dk)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"]))
    q = unit_vectors(q) * dk ** -0.5
    k = unit_vectors(k)
    beta, g = delta_gates(h @ w[p + "b"].T, h @ w[p + "a"].T, w[p + "A_log"], w[p + "dt_bias"])
    o = gated_delta_rule(q.reshape(T, G * dk), k.reshape(T, G * dk), v, beta, g, H, G, dk, dv).reshape(T, H, dv)
    o = rms_unit(o, eps) * w[p + "norm"] * silu(h @ w[p + "g"].T).reshape(T, H, dv)
    return o.reshape(T, H * dv) @ w[p + "o"].T


def forward(cfg, w, tokens, residuals=None):
    """Logits [T, vocab] of a whole sequence; residuals (a list) receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = w["embed"][torch.as_tensor(tokens)] + sinusoid(range(T), cfg["width"])
    for li, layer in enumerate(cfg["layers"]):
        p = "l%d." % li
        h = layer_norm_nobias(x, w[p + "norm1"], eps)
        if layer["type"] == "parallel":
            upd = mixer_parallel(h, w, p + "mix.", layer["mixer"], eps) * w[p + "ls1"]
        else:
            upd = mixer_delta(h, w, p + "mix.", layer["mixer"], eps) * w[p + "ls1"]
        if layer.get("mlp"):
            upd = upd + gated_ffn(h, w[p + "mlp.gate"], w[p + "mlp.gate.b"], w[p + "mlp.up"], w[p + "mlp.up.b"], w[p + "mlp.down"],
                                  w[p + "mlp.down.b"]) * w[p + "ls2"]
        x = x + upd
        if residuals is not None:
            residuals.append(x.clone())
    return layer_norm_nobias(x, w["final.norm"], eps) @ w["head"].T
