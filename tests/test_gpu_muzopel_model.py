"""The layer-list worker serving Muzopel models through the InferenceEngine (registry, expert stacking, slots, scheduler, sampling entry
points) against the float64 oracle of tests/muzopel_oracle.py: whole prompts, the residual after every layer, token-by-token decoding,
portions, mixed batches with slots reused, far keys at the edges of key blocks and key shares, the first tokens of a sequence, long
decoding, other sizes, greedy generation, the trace tool."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import muzopel_fixtures as fx
from tests import muzopel_oracle as orc
from tests.gelarax_oracle import bf16_round

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL32 = 2e-5        # fp32 operands: rounding of fp32 sums only
TOL16 = 4e-2        # operands of the matrix products rounded to bfloat16


def assert_close(err, dtype, tol, what=None):
    """fp32: every row within tol.  bfloat16 operands: a router's close call may fall the other way for a row (its experts change, a
    discrete step), so most rows must be within tol and no row far off."""
    if dtype == "float32":
        assert err.max() < tol, (what, err.max())
    else:
        assert np.quantile(err, 0.85) < tol and err.max() < 0.35, (what, np.quantile(err, 0.85), err.max())


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


# both mixer types, a layer without feed-forward, unequal head / latent sizes
MIXED = fx.config([fx.latent2_layer(), fx.latent_layer(), fx.latent2_layer(heads=2, dim=8, rot_dim=24, vdim=16, kv_rank=40, mlp=None),
                   fx.latent_layer(heads=3, dim=24, rot_dim=8, vdim=8, kv_rank=16, q_rank=12, mlp=fx.moe(experts=3, identity=1, top=2, ff=40))],
                  width=64, vocab=97)


@pytest.mark.parametrize("dtype,tol", [("float32", TOL32), ("bfloat16", TOL16)])
def test_whole_prompt_matches_the_oracle(tmp_path, dtype, tol):
    w = fx.random_weights(MIXED, 1)
    toks = tokens_for(MIXED, 71, 2)
    eng = engine_for(tmp_path, MIXED, w, dtype)
    lg, nxt = run_whole(eng, toks)
    want = oracle_logits(MIXED, w, toks)
    assert lg.shape == want.shape
    assert_close(fx.rel_err(lg, want), dtype, tol)
    if dtype == "float32":
        assert nxt == int(want[-1].argmax())
    eng.close()


def test_residual_after_every_layer_matches_the_oracle(tmp_path):
    import ctypes as C
    import inferflow_amd as ia
    w = fx.random_weights(MIXED, 3)
    eng = engine_for(tmp_path, MIXED, w)
    L = ia.lib()
    ia.check(L.ifa_model_set_option(eng.worker(), b"tap_layers", 1))
    for n in (40, 5):          # the tiled and the single-row attention, the grouped and the row form of the experts
        toks = tokens_for(MIXED, n, 4)
        run_whole(eng, toks)
        res = []
        with torch.no_grad():
            orc.forward(MIXED, fx.oracle_weights(w), toks, res)
        for li, want in enumerate(res):
            p, b = C.c_void_p(), C.c_size_t()
            ia.check(L.ifa_model_get_buffer(eng.worker(), b"layer_taps", li, C.byref(p), C.byref(b)))
            got = np.zeros((len(toks), MIXED["width"]), np.float32)
            ia.check(L.ifa_memcpy_d2h(got.ctypes.data_as(C.c_void_p), p, got.nbytes, None)); ia.check(L.ifa_stream_sync(None))
            assert np.abs(got - want.numpy()).max() < 2e-4 * max(1.0, np.abs(want.numpy()).max()), (n, li)
    eng.close()


@pytest.mark.parametrize("sizes", [[1], [2], [5, 3], [30, 1], [7, 2, 1], [64, 4], [17, 16, 2]])
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


def test_small_steps_as_fused_launches_and_as_separate_ops_agree(tmp_path):
    """steps of a few rows run norm-add / depth average / input convolution / tail as one launch and the router's product inside its choice;
    with the option off they take the row-parallel ops of the larger steps"""
    import inferflow_amd as ia
    w = fx.random_weights(MIXED, 25)
    toks = tokens_for(MIXED, 60, 26)
    want = oracle_logits(MIXED, w, toks)
    eng = engine_for(tmp_path, MIXED, w)
    for fuse in (1, 0, 1):
        ia.check(ia.lib().ifa_model_set_option(eng.worker(), b"fuse_post", fuse))
        for sizes in ([33, 1], [3, 2], [8, 7, 1]):
            assert fx.rel_err(run_portions(eng, toks, sizes), want).max() < TOL32, (fuse, sizes)
    eng.close()


@pytest.mark.parametrize("n", [1, 2, 3, 4])
def test_first_tokens_of_a_sequence(tmp_path, n):
    """prompts no longer than the convolution's taps, whole and token by token, on a slot that held a longer sequence before"""
    cfg = fx.config([fx.latent_layer(), fx.latent2_layer()], taps=4)
    w = fx.random_weights(cfg, 21)
    eng = engine_for(tmp_path, cfg, w, queries=1)
    run_whole(eng, tokens_for(cfg, 50, 22))          # leaves its cache rows and convolution tails in the only slot
    toks = tokens_for(cfg, n, 23 + n)
    want = oracle_logits(cfg, w, toks)
    assert fx.rel_err(run_whole(eng, toks)[0], want).max() < TOL32
    assert fx.rel_err(run_portions(eng, toks, [1]), want).max() < TOL32
    eng.close()


def test_batches_of_unequal_requests_equal_each_alone_and_slots_are_reused(tmp_path):
    w = fx.random_weights(MIXED, 7)
    eng = engine_for(tmp_path, MIXED, w, queries=3)
    prompts = [tokens_for(MIXED, n, 10 + n) for n in (1, 37, 64, 5, 90, 2)]
    tails = [tokens_for(MIXED, 12, 50 + i) for i in range(len(prompts))]
    alone = [oracle_logits(MIXED, w, p + t) for p, t in zip(prompts, tails)]
    # three queries on three slots, twice: the second time reuses the slots of the first
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


def marked_model(kind):
    """One attention layer whose weights make one key stand out: the token `probe` has a query that matches the key of token `mark`
    (through the latent: the mark's embedding drives latent channel 0, which the key map sends to head dimension 0).  The last row's
    logits then depend strongly on whether the mark's cache row is read, wherever it lies."""
    layer = fx.latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=16, q_rank=12, scale=1.0, mlp=None) if kind == 1 else \
        fx.latent2_layer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=16, scale=1.0, mlp=None)
    cfg = fx.config([layer], width=32, vocab=50, groups=2, taps=2)
    w = fx.random_weights(cfg, 9)
    mark, probe = 7, 9
    e = w["embed"]
    e[mark] = 0; e[probe] = 0
    e[mark, 0] = 8.0; e[probe, 1] = 8.0
    w["l0.canon1"][:2] = 0                                  # features 0 and 1 pass the input convolution unmixed
    dkv, uk = w["l0.mix.dkv"], w["l0.mix.uk"]
    dkv[:, :2] = 0; dkv[0, 0] = 4.0                         # latent channel 0 reads feature 0
    uk[:, 0] = 0
    for h in range(2):
        uk[h * 16, 0] = 4.0                                 # ... and becomes head dimension 0 of every head's key
    if kind == 1:
        dq, uq = w["l0.mix.dq"], w["l0.mix.uq"]
        dq[:, :2] = 0; dq[0, 1] = 4.0; uq[:, 0] = 0
        for h in range(2):
            uq[h * 24, 0] = 4.0
    else:
        q = w["l0.mix.q"]
        q[:, :2] = 0
        for h in range(2):
            q[h * 24, 1] = 4.0
    return cfg, {k: bf16_round(v) for k, v in w.items()}, mark, probe


@pytest.mark.parametrize("kind", [1, 2])
def test_far_keys_at_block_and_share_edges_in_prompts_and_decoding(tmp_path, kind):
    """the marked key at the borders of the tiled kernel's key blocks (32) and query tiles (128) and of the single-row kernel's
    key shares (64 keys a workgroup, 16 a wave step), hundreds of tokens back"""
    cfg, w, mark, probe = marked_model(kind)
    eng = engine_for(tmp_path, cfg, w, ctx=700)
    filler = [t for t in range(10, 50)]
    for mark_at, n in ((0, 2), (0, 33), (31, 300), (32, 300), (63, 129), (64, 129), (127, 128), (128, 130), (15, 600), (16, 600), (255, 257), (256, 258), (5, 640)):
        toks = [filler[(3 * i + mark_at + n) % len(filler)] for i in range(n)]
        toks[mark_at] = mark; toks[-1] = probe
        want = oracle_logits(cfg, w, toks)
        whole, _ = run_whole(eng, toks)
        assert fx.rel_err(whole, want).max() < TOL32, ("prompt", mark_at, n)
        dec = run_portions(eng, toks, [max(1, n - 3), 1])
        assert fx.rel_err(dec, want).max() < TOL32, ("decoded", mark_at, n)
        # the oracle itself must see the key: without the mark the last row differs clearly
        blind = list(toks); blind[mark_at] = filler[0]
        assert fx.rel_err(oracle_logits(cfg, w, blind)[-1:], want[-1:]).max() > 1e-3, (mark_at, n)
    eng.close()


def test_long_decoding_and_scaled_rotation_far_from_the_start(tmp_path):
    cfg = fx.config([fx.latent_layer(heads=2, dim=8, rot_dim=16, vdim=8, kv_rank=16, q_rank=8, scaling={"factor": 8.0, "original": 32, "fast": 8.0, "slow": 1.0},
                                     mlp=fx.moe(experts=4, identity=1, top=2, ff=16)),
                     fx.latent2_layer(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=8, base=200.0, mlp=fx.moe(experts=2, identity=2, top=3, ff=8))], width=32, vocab=61)
    w = fx.random_weights(cfg, 11)
    toks = tokens_for(cfg, 330, 12)
    want = oracle_logits(cfg, w, toks)
    eng = engine_for(tmp_path, cfg, w, ctx=400)
    got = run_portions(eng, toks, [200, 1])        # 130 tokens decoded one by one
    assert fx.rel_err(got, want).max() < 5e-5
    eng.close()


CASES = {
    # one head, one part in the norm, one expert chosen, no identity expert, taps 1, latent layer first
    "ones": lambda: fx.config([fx.latent_layer(heads=1, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8, mlp=fx.moe(experts=3, identity=0, top=1, ff=8)),
                               fx.latent2_layer(heads=1, dim=4, rot_dim=4, vdim=4, kv_rank=4, mlp=fx.moe(experts=1, identity=0, top=1, ff=4))],
                              width=16, vocab=11, groups=1, taps=1),
    # every expert chosen, more identity experts than chosen ones elsewhere, only part of the rotated dimensions turn, no soft cap
    "all_chosen": lambda: fx.config([fx.latent2_layer(mlp=fx.moe(experts=2, identity=1, top=3, ff=12)),
                                     fx.latent_layer(rot_dim=12, rot_dims=8, mlp=fx.moe(experts=1, identity=4, top=2, ff=20))], width=48, vocab=33, groups=3, taps=5,
                                    softcap=0.0),
    # identity experts only; no feed-forward at all; no input convolution; plain rotation on the first type
    "no_experts": lambda: fx.config([fx.latent_layer(scaling=None, mlp=fx.moe(experts=0, identity=3, top=2, ff=8)), fx.latent2_layer(mlp=None)], width=32, vocab=19, taps=0),
    # sizes that keep every 16-byte path off: odd latent, odd head sizes, width 14
    "unaligned": lambda: fx.config([fx.latent_layer(heads=3, dim=5, rot_dim=6, vdim=7, kv_rank=9, q_rank=5, mlp=fx.moe(experts=3, identity=1, top=2, ff=10)),
                                    fx.latent2_layer(heads=2, dim=7, rot_dim=2, vdim=3, kv_rank=11, mlp=fx.moe(experts=2, identity=1, top=1, ff=6))],
                                   width=14, vocab=9, groups=2, taps=2),
    # the widest heads the tiled kernel takes (keys 192, values 128) and a cache row beyond 256
    "wide_heads": lambda: fx.config([fx.latent2_layer(heads=2, dim=128, rot_dim=64, vdim=128, kv_rank=224, mlp=fx.moe(experts=4, identity=1, top=2, ff=64)),
                                     fx.latent_layer(heads=2, dim=96, rot_dim=32, vdim=72, kv_rank=64, q_rank=48, mlp=None)], width=128, vocab=50),
    # heads beyond the tiled kernel: prompts take the single-row form too
    "beyond_the_tile": lambda: fx.config([fx.latent2_layer(heads=2, dim=160, rot_dim=64, vdim=136, kv_rank=48, mlp=fx.moe(experts=2, identity=1, top=2, ff=32))],
                                         width=64, vocab=23),
    # many experts, eight chosen
    "many_experts": lambda: fx.config([fx.latent2_layer(mlp=fx.moe(experts=70, identity=3, top=8, ff=16))], width=32, vocab=29, groups=8),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_other_sizes(tmp_path, case):
    cfg = CASES[case]()
    w = fx.random_weights(cfg, 13)
    toks = tokens_for(cfg, 45, 14)
    want = oracle_logits(cfg, w, toks)
    for dtype, tol in (("float32", TOL32), ("bfloat16", TOL16)):
        eng = engine_for(tmp_path, cfg, w, dtype)
        whole, _ = run_whole(eng, toks)
        assert_close(fx.rel_err(whole, want), dtype, tol, (case, dtype))
        assert_close(fx.rel_err(run_portions(eng, toks, [20, 9, 1]), want), dtype, tol, (case, dtype, "portions"))
        eng.close()


def test_router_close_calls_follow_the_correction_not_the_score(tmp_path):
    """a large correction moves the choice to experts with small scores; the weights stay the plain scores"""
    cfg = fx.config([fx.latent2_layer(mlp=fx.moe(experts=5, identity=2, top=2, ff=16))], width=32, vocab=31)
    w = fx.random_weights(cfg, 31)
    c = w["l0.mlp.correction"]
    c[:] = 0; c[4] = 2.0; c[6] = 1.5          # expert 4 and the second identity expert win whatever their scores are
    w = {k: bf16_round(v) for k, v in w.items()}
    toks = tokens_for(cfg, 40, 32)
    eng = engine_for(tmp_path, cfg, w)
    want = oracle_logits(cfg, w, toks)
    assert fx.rel_err(run_whole(eng, toks)[0], want).max() < TOL32
    assert fx.rel_err(run_portions(eng, toks, [1]), want).max() < TOL32
    plain = dict(w); plain["l0.mlp.correction"] = np.zeros_like(c)
    assert fx.rel_err(oracle_logits(cfg, plain, toks), want).max() > 1e-3
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
    # a second generation on the same slot replays the captured step against a new sequence
    q = eng.add_query(prompt[:7])
    gen2, _ = eng.generate(q, 10)
    eng.remove_query(q)
    want2 = oracle_logits(MIXED, w, prompt[:7] + gen2)
    for i, tok in enumerate(gen2):
        row = want2[6 + i]
        top2 = np.sort(row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
            assert tok == int(row.argmax()), i
    # sampled queries draw from the same logits (top-k with a seed: reproducible)
    a = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    b = eng.add_query(prompt, strategy="sample.top_k", seed=5)
    out = dict(eng.infer())
    assert out[a] == out[b] and 0 <= out[a] < MIXED["vocab"]
    eng.close()


def test_generation_with_a_cache_row_that_needs_the_large_lds_grant(tmp_path):
    """a latent of 640 channels: the single-token kernel's LDS passes 48 KB, granted when the model is finalized, before the step is captured"""
    cfg = fx.config([fx.latent2_layer(heads=5, dim=16, rot_dim=16, vdim=24, kv_rank=640, mlp=fx.moe(experts=3, identity=1, top=2, ff=16))], width=32, vocab=37)
    w = fx.random_weights(cfg, 41)
    prompt = tokens_for(cfg, 21, 42)
    eng = engine_for(tmp_path, cfg, w)
    q = eng.add_query(prompt)
    gen, _ = eng.generate(q, 12)
    eng.remove_query(q)
    want = oracle_logits(cfg, w, prompt + gen)
    for i, tok in enumerate(gen):
        row = want[len(prompt) - 1 + i]
        top2 = np.sort(row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
            assert tok == int(row.argmax()), i
    assert fx.rel_err(run_portions(eng, prompt + gen, [17, 1]), want).max() < TOL32
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
    assert eng.model_info("vocab_size") == MIXED["vocab"] and eng.model_info("decoder_layers") == len(MIXED["layers"])
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
