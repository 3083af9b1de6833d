"""The layer-list worker serving Gelarax models through the InferenceEngine (loader registry, slots, scheduler, sampling entry points)
against the float64 oracle of tests/gelarax_oracle.py: whole prompts, token-by-token decoding, portions, mixed batches, slot reuse,
window / kept-first edges, long decoding, other sizes, greedy generation."""
import os
import subprocess
import json

import numpy as np
import pytest
import torch

from tests import gelarax_oracle as orc
from tests import layered_fixtures as fx

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL32 = 2e-5        # fp32 operands: rounding of fp32 sums only
TOL16 = 3e-2        # operands of the matrix products rounded to bfloat16


def engine_for(tmp_path, cfg, weights, dtype="float32", ctx=512, queries=6):
    from inferflow_amd.engine import InferenceEngine
    d = fx.write_model_dir(str(tmp_path / ("m%d" % len(os.listdir(tmp_path)))), cfg, weights)
    return InferenceEngine.from_model_dir(d, dtype, ctx, queries, True)


def tokens_for(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


def oracle_logits(cfg, weights, tokens):
    with torch.no_grad():
        return orc.forward(cfg, fx.oracle_weights(weights), tokens).numpy()


def run_whole(eng, tokens):
    q = eng.add_query(tokens)
    assert q > 0
    out = eng.infer()
    assert [i for i, _ in out] == [q]
    lg = eng.last_logits_f32(q)
    eng.remove_query(q)
    return lg, out[0][1]


def run_portions(eng, tokens, sizes):
    """the prompt in portions of the given sizes (the last size repeats); logits of every token"""
    q = eng.add_query(tokens[:sizes[0]])
    rows, at, k = [], sizes[0], 0
    eng.infer(); rows.append(eng.last_logits_f32(q))
    while at < len(tokens):
        k = min(k + 1, len(sizes) - 1)
        n = min(sizes[k], len(tokens) - at)
        for t in tokens[at:at + n]:
            assert eng.commit({q: t})
        eng.infer(); rows.append(eng.last_logits_f32(q))
        at += n
    eng.remove_query(q)
    return np.concatenate(rows, 0)


MIXED = fx.config([fx.parallel_layer(), fx.delta_layer(), fx.parallel_layer(heads=2, kv_heads=1, dim=16, window=9, keep_first=0, lin_heads=3, lin_dim=8, lin_vdim=24,
                                                                           ff=0)], width=64, vocab=97)


@pytest.mark.parametrize("dtype,tol", [("float32", TOL32), ("bfloat16", TOL16)])
def test_whole_prompt_matches_the_oracle(tmp_path, dtype, tol):
    w = fx.random_weights(MIXED, 1)
    toks = tokens_for(MIXED, 71, 2)
    eng = engine_for(tmp_path, MIXED, w, dtype)
    lg, nxt = run_whole(eng, toks)
    want = oracle_logits(MIXED, w, toks)
    assert lg.shape == want.shape
    assert fx.rel_err(lg, want).max() < tol
    if dtype == "float32":
        assert nxt == int(want[-1].argmax())
    eng.close()


def test_residual_after_every_layer_matches_the_oracle(tmp_path):
    import ctypes as C
    import inferflow_amd as ia
    w = fx.random_weights(MIXED, 3)
    toks = tokens_for(MIXED, 40, 4)
    eng = engine_for(tmp_path, MIXED, w)
    L = ia.lib()
    ia.check(L.ifa_model_set_option(eng.worker(), b"tap_layers", 1))
    run_whole(eng, toks)
    res = []
    with torch.no_grad():
        orc.forward(MIXED, fx.oracle_weights(w), toks, res)
    for li, want in enumerate(res):
        p, b = C.c_void_p(), C.c_size_t()
        ia.check(L.ifa_model_get_buffer(eng.worker(), b"layer_taps", li, C.byref(p), C.byref(b)))
        got = np.zeros((len(toks), MIXED["width"]), np.float32)
        ia.check(L.ifa_memcpy_d2h(got.ctypes.data_as(C.c_void_p), p, got.nbytes, None)); ia.check(L.ifa_stream_sync(None))
        assert np.abs(got - want.numpy()).max() < 2e-4 * max(1.0, np.abs(want.numpy()).max()), li
    eng.close()


@pytest.mark.parametrize("sizes", [[1], [2], [5, 3], [30, 1], [7, 2, 1], [64, 4]])
def test_portions_and_token_by_token_equal_the_whole_prompt(tmp_path, sizes):
    w = fx.random_weights(MIXED, 5)
    toks = tokens_for(MIXED, 83, 6)
    eng = engine_for(tmp_path, MIXED, w)
    whole, _ = run_whole(eng, toks)
    parts = run_portions(eng, toks, sizes)
    assert parts.shape == whole.shape
    assert fx.rel_err(parts, whole).max() < TOL32
    assert fx.rel_err(parts, oracle_logits(MIXED, w, toks)).max() < TOL32
    eng.close()


def test_batches_of_unequal_requests_equal_each_alone_and_slots_are_reused(tmp_path):
    w = fx.random_weights(MIXED, 7)
    eng = engine_for(tmp_path, MIXED, w, queries=3)
    prompts = [tokens_for(MIXED, n, 10 + n) for n in (1, 37, 64, 5, 90, 2)]
    tails = [tokens_for(MIXED, 12, 50 + i) for i in range(len(prompts))]
    alone = []
    for p, t in zip(prompts, tails):
        alone.append(oracle_logits(MIXED, w, p + t))
    # two rounds of three queries on three slots: the second round reuses the slots of the first
    for rnd in range(2):
        qs = [eng.add_query(p) for p in prompts[3 * rnd:3 * rnd + 3]]
        assert all(q > 0 for q in qs) and eng.add_query([1, 2]) == 0          # busy: every slot is taken
        got = {q: [] for q in qs}
        assert sorted(i for i, _ in eng.infer()) == sorted(qs)                 # ONE step for the three prompts
        for q in qs:
            got[q].append(eng.last_logits_f32(q))
        for step in range(12):
            live = [q for k, q in enumerate(qs) if not (k == 0 and step >= 6)]  # the first query ends earlier
            if step == 6:
                eng.remove_query(qs[0])
            eng.commit({q: tails[3 * rnd + qs.index(q)][step] for q in live})
            assert sorted(i for i, _ in eng.infer()) == sorted(live)
            for q in live:
                got[q].append(eng.last_logits_f32(q))
        for k, q in enumerate(qs):
            g = np.concatenate(got[q], 0)
            assert fx.rel_err(g, alone[3 * rnd + k][:len(g)]).max() < TOL32, (rnd, k)
            eng.remove_query(q)
    eng.close()


def test_window_and_kept_first_edges_in_prompts_and_decoding(tmp_path):
    """One attention layer whose weights make one key stand out: the token `probe` has a query that matches the key of token `mark`.
    The logits then depend strongly on whether `mark` is visible, so a window or kept-first range that is one token off shows."""
    window, keep = 11, 3
    cfg = fx.config([fx.parallel_layer(heads=2, kv_heads=2, dim=16, window=window, keep_first=keep, scale=1.0, softcap=30.0, lin_heads=1, lin_dim=8, lin_vdim=8,
                                       ff=0)], width=32, vocab=50)
    w = fx.random_weights(cfg, 9, buckets=8)
    mark, probe = 7, 9
    e = w["embed"]
    e[mark] = 0; e[probe] = 0
    e[mark, 0] = 8.0; e[probe, 1] = 8.0
    # keys read feature 0, queries feature 1, both onto head dimension 0
    wq, wk = w["l0.mix.left.q"], w["l0.mix.left.k"]
    wq[:, :2] = 0; wk[:, :2] = 0
    for h in range(2):
        wq[h * 16, 1] = 4.0; wk[h * 16, 0] = 4.0
    w = {k: orc.bf16_round(v) for k, v in w.items()}
    eng = engine_for(tmp_path, cfg, w, ctx=128)
    filler = [t for t in range(10, 50)]
    for mark_at in (0, keep - 1, keep, keep + 1, 20):
        for dist in (1, window - 1, window, window + 1, 40):
            n = mark_at + dist + 1
            toks = [filler[(3 * i + mark_at + dist) % len(filler)] for i in range(n)]
            toks[mark_at] = mark; toks[-1] = probe
            want = oracle_logits(cfg, w, toks)
            whole, _ = run_whole(eng, toks)
            assert fx.rel_err(whole, want).max() < TOL32, ("prompt", mark_at, dist)
            if n > 2:
                dec = run_portions(eng, toks, [max(1, n - 3), 1])
                assert fx.rel_err(dec, want).max() < TOL32, ("decoded", mark_at, dist)
            # the oracle itself must see the edge: with the mark masked out (one past the window, not kept) the last row differs
            seen = mark_at < keep or dist < window
            blind = list(toks); blind[mark_at] = filler[0]
            moved = fx.rel_err(oracle_logits(cfg, w, blind)[-1:], want[-1:]).max()
            assert (moved > 1e-3) == seen or not seen, (mark_at, dist, moved)
    eng.close()


def test_far_key_among_hundreds_and_long_decoding(tmp_path):
    cfg = fx.config([fx.delta_layer(heads=2, kv_heads=1, dim=8, vdim=8, conv=4, ff=32), fx.parallel_layer(heads=2, kv_heads=1, dim=16, window=50, keep_first=4,
                                                                                                          lin_heads=2, lin_dim=8, lin_vdim=16, decay=[0.999, 0.9],
                                                                                                          ff=32)], width=32, vocab=61)
    w = fx.random_weights(cfg, 11, buckets=[0, 10])
    toks = tokens_for(cfg, 330, 12)
    want = oracle_logits(cfg, w, toks)
    eng = engine_for(tmp_path, cfg, w, ctx=400)
    got = run_portions(eng, toks, [200, 1])        # 130 tokens decoded one by one: the window passes over decoded tokens
    assert fx.rel_err(got, want).max() < 5e-5
    # the state reaches far back: another first token changes the last logits (slow decay, kept first tokens)
    other = list(toks); other[0] = (toks[0] + 1) % cfg["vocab"]
    assert fx.rel_err(oracle_logits(cfg, w, other)[-1:], want[-1:]).max() > 1e-4
    eng.close()


@pytest.mark.parametrize("case", ["gqa_1", "mha", "delta_first_taps2", "no_ffn_anywhere", "odd_sizes", "tiny_unaligned", "wide_heads"])
def test_other_sizes(tmp_path, case):
    if case == "gqa_1":
        cfg = fx.config([fx.parallel_layer(heads=4, kv_heads=1, dim=8, window=1, keep_first=1, lin_heads=1, lin_dim=4, lin_vdim=4, ff=16)], width=16, vocab=11)
    elif case == "mha":
        cfg = fx.config([fx.parallel_layer(heads=3, kv_heads=3, dim=12, window=200, keep_first=0, lin_heads=2, lin_dim=20, lin_vdim=70, ff=40),
                         fx.delta_layer(heads=3, kv_heads=3, dim=12, vdim=70, conv=1, ff=40)], width=48, vocab=33)
    elif case == "delta_first_taps2":
        cfg = fx.config([fx.delta_layer(heads=1, kv_heads=1, dim=4, vdim=4, conv=2, ff=8), fx.delta_layer(heads=6, kv_heads=2, dim=24, vdim=8, conv=5, ff=0),
                         fx.parallel_layer()], width=40, vocab=29)
    elif case == "no_ffn_anywhere":
        cfg = fx.config([fx.parallel_layer(ff=0), fx.delta_layer(ff=0)], width=24, vocab=19)
    elif case == "tiny_unaligned":
        cfg = fx.config([fx.parallel_layer(heads=2, kv_heads=1, dim=6, window=5, keep_first=1, lin_heads=1, lin_dim=3, lin_vdim=5, ff=10),
                         fx.delta_layer(heads=2, kv_heads=2, dim=6, vdim=5, conv=3, ff=0)], width=14, vocab=9)
    elif case == "wide_heads":
        cfg = fx.config([fx.parallel_layer(heads=2, kv_heads=1, dim=160, window=30, keep_first=2, lin_heads=1, lin_dim=128, lin_vdim=96, ff=64),
                         fx.delta_layer(heads=2, kv_heads=1, dim=64, vdim=72, conv=4, ff=64), fx.parallel_layer(heads=4, kv_heads=4, dim=32, window=7, keep_first=9,
                                                                                                              lin_heads=2, lin_dim=32, lin_vdim=16, ff=0)],
                        width=128, vocab=50)
    else:
        cfg = fx.config([fx.parallel_layer(heads=5, kv_heads=5, dim=20, window=13, keep_first=2, lin_heads=3, lin_dim=12, lin_vdim=36, ff=52),
                         fx.delta_layer(heads=5, kv_heads=1, dim=12, vdim=20, conv=4, ff=52)], width=36, vocab=23)
    w = fx.random_weights(cfg, 13, buckets=9)
    toks = tokens_for(cfg, 45, 14)
    want = oracle_logits(cfg, w, toks)
    for dtype, tol in (("float32", TOL32), ("bfloat16", TOL16)):
        eng = engine_for(tmp_path, cfg, w, dtype)
        whole, _ = run_whole(eng, toks)
        assert fx.rel_err(whole, want).max() < tol, (case, dtype)
        assert fx.rel_err(run_portions(eng, toks, [20, 9, 1]), want).max() < tol, (case, dtype, "portions")
        eng.close()


def test_greedy_generation_through_the_engine(tmp_path):
    w = fx.random_weights(MIXED, 15)
    prompt = tokens_for(MIXED, 19, 16)
    eng = engine_for(tmp_path, MIXED, w)
    # Generate(): prompt step + decode steps replayed from a captured graph with the token fed back on the device
    q = eng.add_query(prompt)
    gen, _ = eng.generate(q, 24)
    eng.remove_query(q)
    # the serving loop: Infer -> Commit of the greedy token
    q = eng.add_query(prompt)
    loop = []
    for _ in range(24):
        (qq, tok), = eng.infer()
        loop.append(tok); eng.commit({q: tok})
    eng.remove_query(q)
    assert gen == loop
    # the oracle follows the same tokens and agrees wherever its two best logits are clearly apart
    want = oracle_logits(MIXED, w, prompt + gen)
    for i, tok in enumerate(gen):
        row = want[len(prompt) - 1 + i]
        top2 = np.sort(row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
            assert tok == int(row.argmax()), i
    # sampled queries draw from the same logits (top-k with a seed: reproducible)
    a = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    b = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    out = dict(eng.infer())
    assert out[a] == out[b] and 0 <= out[a] < MIXED["vocab"]
    eng.close()


def test_ini_route_and_trace_replay_tool(tmp_path):
    from inferflow_amd.engine import InferenceEngine
    w = fx.random_weights(MIXED, 17)
    d = fx.write_model_dir(str(tmp_path / "model"), MIXED, w)
    ini = tmp_path / "serve.ini"
    ini.write_text("[transformer_engine]\nmodels = m\ndevices = 0\nmax_concurrent_queries = 2\nreturn_output_tensors_f32 = true\n\n"
                   "[model.m]\nmodel_dir = %s/\ncompute_dtype = float32\nmax_context_len = 100\n" % d)
    eng = InferenceEngine.from_ini(str(ini))
    toks = tokens_for(MIXED, 30, 18)
    lg, _ = run_whole(eng, toks)
    want = oracle_logits(MIXED, w, toks)
    assert fx.rel_err(lg, want).max() < TOL32
    assert eng.model_info("vocab_size") == MIXED["vocab"] and eng.model_info("decoder_layers") == 3
    eng.close()
    # the trace tool: two requests start together, go on token by token, one ends earlier
    a, b = tokens_for(MIXED, 26, 19), tokens_for(MIXED, 9, 20)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [0, 19]}, {"id": "b", "tokens": b[:6], "want": [5]}], "end": []}]
    for s in range(1, 7):
        ent = [{"id": "a", "tokens": [a[19 + s]], "want": [0]}]
        if s <= 3:
            ent.append({"id": "b", "tokens": [b[5 + s]], "want": [0] if s != 2 else []})
        steps.append({"step": s, "entries": ent, "end": (["b"] if s == 3 else []) + (["a"] if s == 6 else [])})
    out = tmp_path / "out"; out.mkdir()
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                       input="".join(json.dumps(s) + "\n" for s in steps).encode(), stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=900)
    assert r.returncode == 0, r.stderr.decode()[-2000:]
    assert [l for l in r.stdout.decode().split() if l != "done"] == [str(s) for s in range(7)]
    wa, wb = oracle_logits(MIXED, w, a), oracle_logits(MIXED, w, b)
    V = MIXED["vocab"]
    g0 = np.fromfile(out / "0.f32", np.float32).reshape(-1, V)
    assert fx.rel_err(g0, np.stack([wa[0], wa[19], wb[5]])).max() < TOL32
    for s in range(1, 7):
        g = np.fromfile(out / ("%d.f32" % s), np.float32).reshape(-1, V)
        exp = [wa[19 + s]] + ([wb[5 + s]] if s <= 3 and s != 2 else [])
        assert fx.rel_err(g, np.stack(exp)).max() < TOL32, s
