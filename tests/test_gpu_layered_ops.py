"""Each mechanism of the layer-list worker alone, through its C-ABI op, against the float64 functions of tests/gelarax_oracle.py:
linear layers with bfloat16 weights (row kernel and both matrix-core modes, ragged shapes, every epilogue), embedding + sinusoid,
norms, gated activations, argmax, short convolutions with their carried tail, delta-rule gates, both state recurrences (whole,
continued, several sequences, slots reused), gated group norm, and the windowed attention with sink / soft cap / bucket bias."""
import ctypes as C

import numpy as np
import pytest
import torch

import inferflow_amd as ia
from tests import gelarax_oracle as orc
from tests.gpu_util import capi, p, sync

pytestmark = pytest.mark.gpu


def dev32(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).cuda()


def devbf(a):
    return torch.from_numpy(orc.bf16_bits(a).view(np.int16)).cuda()


def devi(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.int32)).cuda()


def stream():
    return None


class Slots:
    """a slot arena table like the worker's: n slots of `floats` fp32 each, filled with garbage so that stale state shows"""

    def __init__(self, n, floats):
        self.mem = [torch.full((floats,), 1e9, dtype=torch.float32, device="cuda") for _ in range(n)]
        self.table = torch.tensor([m.data_ptr() for m in self.mem], dtype=torch.int64).cuda()


def seq_tables(seqs):
    """seqs: [(n, pos0, slot)] -> device (descs, row_seq), total rows"""
    d, rs, r = [], [], 0
    for i, (n, pos0, slot) in enumerate(seqs):
        d += [r, n, pos0, slot]; rs += [i] * n; r += n
    return devi(d), devi(rs), r


@pytest.mark.parametrize("T", [1, 2, 3, 8, 9, 64, 70, 131])
@pytest.mark.parametrize("N,K", [(64, 64), (5, 36), (130, 200), (48, 7)])
def test_linear_bf16_weights(T, N, K):
    rng = np.random.default_rng(T * 1000 + N + K)
    W = orc.bf16_round(rng.standard_normal((N, K)))
    A = rng.standard_normal((T, K + 4)).astype(np.float32)            # lda > K
    bias, mul = orc.bf16_round(rng.standard_normal(N)), orc.bf16_round(rng.standard_normal(N))
    C0 = rng.standard_normal((T, N + 2)).astype(np.float32)
    prod = A[:, :K].astype(np.float64) @ W.astype(np.float64).T
    for ops32 in (1, 0):
        for use_bias, use_mul, alpha, acc in ((0, 0, 1.0, 0), (1, 0, 1.0, 0), (1, 1, 0.7, 1), (0, 1, 1.3, 1)):
            c = dev32(C0)
            ia.check(capi().ifa_linear_bf16w(p(devbf(W)), N, K, p(dev32(A)), K + 4, T, p(devbf(bias)) if use_bias else None,
                                             p(devbf(mul)) if use_mul else None, alpha, acc, ops32, p(c), N + 2, 2, min(N, 40) if use_mul else 0, stream()))
            sync()
            want = prod + (bias if use_bias else 0)
            if use_mul:                                                 # columns [2, 40) through SiLU after the bias
                want[:, 2:min(N, 40)] = orc.silu(orc.t64(want[:, 2:min(N, 40)])).numpy()
            if use_mul:
                want = want * mul
            want = want * alpha + (C0[:, :N] if acc else 0)
            got = c.cpu().numpy()
            assert np.array_equal(got[:, N:], C0[:, N:])                # columns past N untouched
            tol = 2e-5 if (ops32 or T <= 8) else 2e-2
            assert np.abs(got[:, :N] - want).max() < tol * max(1.0, np.abs(want).max()), (ops32, use_bias, use_mul, acc)


def test_embedding_with_sinusoid_norms_glu_argmax():
    rng = np.random.default_rng(1)
    V, W, T = 37, 50, 9
    E = orc.bf16_round(rng.standard_normal((V, W)))
    toks = rng.integers(0, V, T); pos = np.array([0, 1, 2, 500, 1115, 4095, 7, 8, 100000])
    x = torch.empty((T, W), dtype=torch.float32, device="cuda")
    ia.check(capi().ifa_embed_sinpos_f32(p(devbf(E)), V, W, p(devi(toks)), p(devi(pos)), T, 10000.0, p(x), stream()))
    want = orc.t64(E)[torch.as_tensor(toks)] + orc.sinusoid(pos, W)
    assert np.abs(x.cpu().numpy() - want.numpy()).max() < 2e-6
    g = orc.bf16_round(1 + 0.3 * rng.standard_normal(W))
    xin = (3 * rng.standard_normal((T, W)) + 2).astype(np.float32)
    for kind, f in ((1, lambda a: orc.layer_norm_nobias(a, orc.t64(g), 1e-5)), (0, lambda a: orc.rms_unit(a, 1e-5) * orc.t64(g))):
        y = torch.empty((T, W), dtype=torch.float32, device="cuda")
        ia.check(capi().ifa_layernorm_f32(kind, p(dev32(xin)), W, T, W, p(devbf(g)), 1e-5, p(y), W, stream()))
        assert np.abs(y.cpu().numpy() - f(orc.t64(xin)).numpy()).max() < 1e-5
    F = 21
    gu = rng.standard_normal((T, 2 * F)).astype(np.float32) * 3
    o = torch.empty((T, F), dtype=torch.float32, device="cuda")
    ia.check(capi().ifa_glu_f32(1, p(dev32(gu)), 2 * F, T, F, p(o), F, stream()))
    want = orc.gelu_tanh(orc.t64(gu[:, :F])) * orc.t64(gu[:, F:])
    assert np.abs(o.cpu().numpy() - want.numpy()).max() < 1e-5
    lg = rng.standard_normal((T, 300)).astype(np.float32)
    lg[2, 17] = lg[2, 250] = 9.0
    best = torch.empty(T, dtype=torch.int32, device="cuda")
    excl = devi([2, int(lg[0].argmax()), 17, -1])
    ia.check(capi().ifa_argmax_rows_f32(p(dev32(lg)), 300, 300, T, p(excl), p(best), stream()))
    b = best.cpu().numpy()
    masked = lg.copy(); masked[:, int(lg[0].argmax())] = -np.inf; masked[:, 17] = -np.inf
    assert list(b) == [int(r.argmax()) for r in masked] and b[2] == 250


@pytest.mark.parametrize("C_,gdim,nq,nsc", [(40, 8, 16, 8), (1100, 100, 600, 300)])      # (the second: a row's channels in two workgroups)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_convolution_with_carried_tail(taps, C_, gdim, nq, nsc):
    rng = np.random.default_rng(taps)
    # channels [0, nq) unit-normed in groups of gdim, channels [0, nsc) scaled
    w = orc.bf16_round(0.5 * rng.standard_normal((C_, taps)))
    full = {s: rng.standard_normal((23, C_ + 5)).astype(np.float32) for s in (0, 1, 2)}

    def want(xs):
        y = orc.silu(orc.short_conv(orc.t64(xs[:, :C_]), orc.t64(w)))
        y[:, :nq] = orc.unit_vectors(y[:, :nq].reshape(-1, nq // gdim, gdim)).reshape(-1, nq)
        y[:, :nsc] *= 0.25
        return y.numpy()

    sl = Slots(3, max(1, (taps - 1)) * C_)
    at = {0: 0, 1: 0, 2: 0}
    # steps of several sequences with portions shorter than the tail; slot 2 is then reused by a new sequence from position 0
    plan = [[(0, 5), (1, 1), (2, 2)], [(1, 1), (0, 1)], [(2, 9), (1, 2), (0, 3)], [(0, 14), (1, 19)]]
    for step in plan:
        seqs = [(n, at[s], s) for s, n in step]
        x = np.concatenate([full[s][at[s]:at[s] + n] for s, n in step], 0)
        d, rs, T = seq_tables(seqs)
        y = torch.empty((T, C_), dtype=torch.float32, device="cuda")
        xd = dev32(x)
        ia.check(capi().ifa_shortconv_silu_f32(p(xd), C_ + 5, C_, taps, p(devbf(w)), p(d), p(rs), T, p(sl.table), 0, nq, gdim, 1e-6, nsc, 0.25, p(y), C_, stream()))
        ia.check(capi().ifa_shortconv_tail_f32(p(xd), C_ + 5, C_, taps, p(d), len(seqs), p(sl.table), 0, stream()))
        sync()
        got, r = y.cpu().numpy(), 0
        for s, n in step:
            assert np.abs(got[r:r + n] - want(full[s][:at[s] + n])[at[s]:]).max() < 1e-5, (taps, s, at[s])
            r += n; at[s] += n
    # reuse: a new sequence on slot 2 must not see the old tail
    new = rng.standard_normal((4, C_ + 5)).astype(np.float32)
    d, rs, T = seq_tables([(4, 0, 2)])
    y = torch.empty((T, C_), dtype=torch.float32, device="cuda")
    ia.check(capi().ifa_shortconv_silu_f32(p(dev32(new)), C_ + 5, C_, taps, p(devbf(w)), p(d), p(rs), T, p(sl.table), 0, nq, gdim, 1e-6, nsc, 0.25, p(y), C_, stream()))
    assert np.abs(y.cpu().numpy() - want(new)).max() < 1e-5


@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("heads,qk_heads,dk,dv", [(2, 2, 8, 8), (4, 2, 24, 70), (3, 1, 130, 33), (2, 1, 32, 40), (4, 2, 64, 64), (2, 2, 128, 100), (2, 1, 16, 17)])
def test_state_recurrences(kind, heads, qk_heads, dk, dv):
    if kind == 0:
        qk_heads = heads
    rng = np.random.default_rng(dk + dv + kind)
    L = 37
    data = {}
    for s in (0, 1):
        q = rng.standard_normal((L, qk_heads * dk)).astype(np.float32) * 0.5
        k = rng.standard_normal((L, qk_heads * dk)).astype(np.float32) * 0.5
        v = rng.standard_normal((L, heads * dv)).astype(np.float32)
        beta = rng.uniform(0, 1, (L, heads)).astype(np.float32)
        g = rng.uniform(0.7, 1, (L, heads)).astype(np.float32)
        if kind == 1:      # unit keys like the design's, one of them far back with a long-lived state
            kk = orc.unit_vectors(orc.t64(k).reshape(L, qk_heads, dk)).reshape(L, -1).numpy().astype(np.float32); k = kk
        data[s] = (q, k, v, beta, g)
    decay = np.array([0.999, 0.5, 0.9, 0.97][:heads], np.float32)

    def want(s, n):
        q, k, v, beta, g = (orc.t64(a[:n]) for a in data[s])
        if kind == 0:
            return orc.decayed_linear_attention(orc.silu(q), orc.silu(k), orc.silu(v), heads, dk, dv, orc.t64(decay)).numpy()
        return orc.gated_delta_rule(q, k, v, beta, g, heads, qk_heads, dk, dv).numpy()

    sl = Slots(2, heads * dk * dv + 8)
    at = {0: 0, 1: 0}
    for step in ([(0, 6), (1, 1)], [(1, 1), (0, 1)], [(0, 2), (1, 30)], [(0, 28)]):
        seqs = [(n, at[s], s) for s, n in step]
        d, rs, T = seq_tables(seqs)
        cat = [np.concatenate([data[s][i][at[s]:at[s] + n] for s, n in step], 0) for i in range(5)]
        out = torch.empty((T, heads * dv), dtype=torch.float32, device="cuda")
        ia.check(capi().ifa_state_scan_f32(kind, 1 if kind == 0 else 0, p(dev32(cat[0])), qk_heads * dk, p(dev32(cat[1])), qk_heads * dk, p(dev32(cat[2])), heads * dv,
                                           heads, qk_heads, dk, dv, p(dev32(decay)) if kind == 0 else None, p(dev32(cat[4])) if kind == 1 else None,
                                           p(dev32(cat[3])) if kind == 1 else None, p(d), len(seqs), p(sl.table), 8, p(out), heads * dv, stream()))
        sync()
        got, r = out.cpu().numpy(), 0
        for s, n in step:
            w_ = want(s, at[s] + n)[at[s]:]
            assert np.abs(got[r:r + n] - w_).max() < 3e-5 * max(1.0, np.abs(w_).max()), (kind, s, at[s], n)
            r += n; at[s] += n


def test_delta_gates_and_gated_group_norm():
    rng = np.random.default_rng(5)
    T, H, dv = 7, 3, 20
    b, a = rng.standard_normal((T, H + 2)).astype(np.float32) * 3, rng.standard_normal((T, H + 1)).astype(np.float32) * 3
    alog, dtb = orc.bf16_round(rng.uniform(-2, 1, H)), orc.bf16_round(rng.uniform(-1, 1, H))
    beta, g = (torch.empty((T, H), dtype=torch.float32, device="cuda") for _ in range(2))
    ia.check(capi().ifa_delta_gates_f32(p(dev32(b)), H + 2, p(dev32(a)), H + 1, H, T, p(devbf(alog)), p(devbf(dtb)), p(beta), p(g), stream()))
    wb, wg = orc.delta_gates(orc.t64(b[:, :H]), orc.t64(a[:, :H]), orc.t64(alog), orc.t64(dtb))
    assert np.abs(beta.cpu().numpy() - wb.numpy()).max() < 1e-6 and np.abs(g.cpu().numpy() - wg.numpy()).max() < 1e-6
    o = rng.standard_normal((T, H * dv)).astype(np.float32) * 4
    gate = rng.standard_normal((T, H * dv + 4)).astype(np.float32) * 2
    for group, wlen, act, f in ((dv, dv, 1, orc.silu), (H * dv, H * dv, 0, torch.sigmoid)):
        w = orc.bf16_round(1 + 0.2 * rng.standard_normal(wlen))
        y = dev32(o)
        ia.check(capi().ifa_gated_groupnorm_f32(p(y), H * dv, T, H * dv, group, p(devbf(w)), wlen, p(dev32(gate)), H * dv + 4, act, 1e-5, p(y), H * dv, stream()))
        want = orc.rms_unit(orc.t64(o).reshape(T, -1, group), 1e-5).reshape(T, -1) * orc.t64(np.tile(w, H * dv // wlen)) * f(orc.t64(gate[:, :H * dv]))
        assert np.abs(y.cpu().numpy() - want.numpy()).max() < 1e-5


@pytest.mark.parametrize("tile_min", [16, 1 << 30])       # prompts through the tiled matrix-core kernel / every row through the per-row kernel
@pytest.mark.parametrize("heads,kv_heads,dim,window,keep,nb,dmax", [(4, 2, 16, 9, 2, 8, 30), (2, 2, 8, 1, 0, 4, 6), (3, 1, 68, 300, 5, 24, 200), (6, 3, 32, 17, 40, 10, 12),
                                                                    (2, 1, 64, 20, 3, 8, 30), (2, 1, 32, 2000, 4, 8, 30), (2, 2, 128, 50, 0, 16, 100), (1, 1, 96, 9, 2, 8, 30), (4, 2, 64, 33, 33, 6, 7), (8, 2, 16, 12, 1, 8, 30), (8, 1, 32, 25, 2, 8, 30)])
def test_windowed_attention_with_sink_cap_and_bucket_bias(heads, kv_heads, dim, window, keep, nb, dmax, tile_min):
    rng = np.random.default_rng(heads + dim + window)
    L, eps, scale, cap = 150, 1e-6, 0.3, 6.0
    q = rng.standard_normal((L, heads * dim + 4)).astype(np.float32)
    k = rng.standard_normal((L, kv_heads * dim + 2)).astype(np.float32)
    # one key far back, one just inside and one just outside the window get large matching queries at the last rows
    k[1, :dim] *= 6; k[max(0, L - window), :dim] *= 6; k[max(0, L - 1 - window), :dim] *= 6
    q[-1, :dim] = k[1, :dim]; q[-2, :dim] = k[max(0, L - 1 - window), :dim]
    rel = orc.bf16_round(rng.standard_normal((nb, heads)))
    sink = orc.bf16_round(rng.standard_normal(heads) * 2)
    want = orc.windowed_attention(orc.t64(q[:, :heads * dim]), orc.t64(k[:, :kv_heads * dim]), heads, kv_heads, dim, scale, cap, window, keep, orc.t64(rel), dmax,
                                  orc.t64(sink), eps).numpy()
    ctx = 160
    bucket_of = devi([orc.distance_bucket(n, nb, dmax) for n in range(ctx)])
    kvd = kv_heads * dim
    sl = Slots(2, 2 * ctx * kvd)
    ws = torch.full((2 * heads * 32 * (dim + 2),), float('nan'), dtype=torch.float32, device='cuda')      # single tokens: the keys shared out over workgroups
    at = 0
    for n in (1, 2, 60, 1, 1, 80, 5):                # prompt portions and single tokens; the same sequence lives on slot 1
        d, rs, T = seq_tables([(n, at, 1)])
        kd = dev32(k[at:at + n])
        ia.check(capi().ifa_kv_store_f32(p(kd), kv_heads * dim + 2, p(kd), kv_heads * dim + 2, kv_heads, dim, 1, eps, p(d), p(rs), T, p(sl.table), 0, ctx * kvd, stream()))
        out = torch.empty((T, heads * dim), dtype=torch.float32, device="cuda")
        ia.check(capi().ifa_attention_window_f32(p(dev32(q[at:at + n])), heads * dim + 4, heads, kv_heads, dim, 1, eps, scale, cap, window, keep, p(devbf(rel)),
                                                 p(bucket_of), nb, p(devbf(sink)), p(d), p(rs), T, p(sl.table), 0, ctx * kvd, p(out), heads * dim,
                                                 (C.c_int * 4)(0, n, at, 1), 1, tile_min, p(ws) if n <= 2 else None, ws.numel() * 4, stream()))
        sync()
        assert np.abs(out.cpu().numpy() - want[at:at + n]).max() < 2e-5 * max(1.0, np.abs(want).max()), (at, n)
        at += n
    assert at == L
    # without the sink the weights sum to one: a different result, so the sink is really counted
    d, rs, T = seq_tables([(1, L - 1, 1)])
    out = torch.empty((1, heads * dim), dtype=torch.float32, device="cuda")
    ia.check(capi().ifa_attention_window_f32(p(dev32(q[L - 1:])), heads * dim + 4, heads, kv_heads, dim, 1, eps, scale, cap, window, keep, p(devbf(rel)),
                                             p(bucket_of), nb, None, p(d), p(rs), T, p(sl.table), 0, ctx * kvd, p(out), heads * dim, None, 0, 0, None, 0, stream()))
    assert np.abs(out.cpu().numpy() - want[L - 1:]).max() > 1e-4


def test_windowed_attention_tiles_over_several_sequences():
    """one step holds a 150-token prompt, a single continued token and a 40-token continued portion: tiles must not cross sequences"""
    rng = np.random.default_rng(77)
    heads, kv_heads, dim, window, keep, nb, dmax, eps, scale, cap = 4, 2, 32, 40, 2, 8, 60, 1e-6, 0.4, 8.0
    L, ctx, kvd = 200, 208, kv_heads * dim
    seq = {s_: (rng.standard_normal((L, heads * dim)).astype(np.float32), rng.standard_normal((L, kvd)).astype(np.float32)) for s_ in (0, 1, 2)}
    rel, sink = orc.bf16_round(rng.standard_normal((nb, heads))), orc.bf16_round(rng.standard_normal(heads))
    want = {s_: orc.windowed_attention(orc.t64(q), orc.t64(k), heads, kv_heads, dim, scale, cap, window, keep, orc.t64(rel), dmax, orc.t64(sink), eps).numpy()
            for s_, (q, k) in seq.items()}
    bucket_of = devi([orc.distance_bucket(n, nb, dmax) for n in range(ctx)])
    sl = Slots(3, 2 * ctx * kvd)
    at = {0: 0, 1: 0, 2: 0}
    for step in ([(1, 30), (2, 100)], [(0, 150), (1, 1), (2, 40)], [(2, 60), (0, 50), (1, 129)]):
        seqs = [(n, at[s_], s_) for s_, n in step]
        d, rs, T = seq_tables(seqs)
        kd = dev32(np.concatenate([seq[s_][1][at[s_]:at[s_] + n] for s_, n in step], 0))
        qd = dev32(np.concatenate([seq[s_][0][at[s_]:at[s_] + n] for s_, n in step], 0))
        ia.check(capi().ifa_kv_store_f32(p(kd), kvd, p(kd), kvd, kv_heads, dim, 1, eps, p(d), p(rs), T, p(sl.table), 0, ctx * kvd, stream()))
        out = torch.empty((T, heads * dim), dtype=torch.float32, device="cuda")
        host, r = [], 0
        for n, pos0, slot in seqs:
            host += [r, n, pos0, slot]; r += n
        ia.check(capi().ifa_attention_window_f32(p(qd), heads * dim, heads, kv_heads, dim, 1, eps, scale, cap, window, keep, p(devbf(rel)), p(bucket_of), nb,
                                                 p(devbf(sink)), p(d), p(rs), T, p(sl.table), 0, ctx * kvd, p(out), heads * dim, (C.c_int * len(host))(*host),
                                                 len(seqs), 16, None, 0, stream()))
        sync()
        got, r = out.cpu().numpy(), 0
        for s_, n in step:
            assert np.abs(got[r:r + n] - want[s_][at[s_]:at[s_] + n]).max() < 2e-5 * max(1.0, np.abs(want[s_]).max()), (s_, at[s_], n)
            r += n; at[s_] += n


@pytest.mark.parametrize("T", [1, 2, 3, 5, 8])
def test_row_products_with_the_norm_or_the_gated_gelu_folded_in(T):
    rng = np.random.default_rng(40 + T)
    N, K = 77, 96
    W = orc.bf16_round(rng.standard_normal((N, K)) / 8)
    bias, mul, g = (orc.bf16_round(rng.standard_normal(n)) for n in (N, N, K))
    x = (2 * rng.standard_normal((T, K + 4)) + 1).astype(np.float32)
    c0 = rng.standard_normal((T, N)).astype(np.float32)
    c = dev32(c0)
    ia.check(capi().ifa_linear_bf16w_rows(1, p(devbf(g)), 1e-5, p(devbf(W)), N, K, p(dev32(x)), K + 4, T, p(devbf(bias)), p(devbf(mul)), 0.5, 1, p(c), N, 3, 9, stream()))
    h = orc.layer_norm_nobias(orc.t64(x[:, :K]), orc.t64(g), 1e-5)
    want = h @ orc.t64(W).T + orc.t64(bias)
    want[:, 3:9] = orc.silu(want[:, 3:9])
    want = (want * orc.t64(mul) * 0.5 + orc.t64(c0)).numpy()
    assert np.abs(c.cpu().numpy() - want).max() < 2e-5 * max(1.0, np.abs(want).max())
    gu = (2 * rng.standard_normal((T, 2 * K + 4))).astype(np.float32)
    c = torch.empty((T, N), dtype=torch.float32, device="cuda")
    ia.check(capi().ifa_linear_bf16w_rows(2, None, 0.0, p(devbf(W)), N, K, p(dev32(gu)), 2 * K + 4, T, None, None, 1.0, 0, p(c), N, 0, 0, stream()))
    want = ((orc.gelu_tanh(orc.t64(gu[:, :K])) * orc.t64(gu[:, K:2 * K])) @ orc.t64(W).T).numpy()
    assert np.abs(c.cpu().numpy() - want).max() < 2e-5 * max(1.0, np.abs(want).max())
