"""Each mechanism that the Muzopel layers add to the layer-list worker alone, through its C-ABI op, against the float64 functions of
tests/muzopel_oracle.py: grouped RMS norm (store / accumulate), the residual short convolution with its carried tail, depth average,
soft cap, embedding rows, latent attention in both forms (cache writer + rotation, absorbed single-row form, expanded tiled form,
portions, several sequences, slots reused), the router, and the experts in the row form and the grouped matrix-core form."""
import ctypes as C

import numpy as np
import pytest
import torch

import inferflow_amd as ia
from tests import muzopel_oracle as orc
from tests.gelarax_oracle import bf16_bits, bf16_round
from tests.gpu_util import capi, p, sync
from tests.test_gpu_layered_ops import Slots, dev32, devbf, devi, seq_tables

pytestmark = pytest.mark.gpu


def t64(a):
    return orc.t64(a)


@pytest.mark.parametrize("rows,cols,groups", [(1, 64, 4), (5, 96, 1), (33, 40, 40), (3, 14, 2), (2, 1024, 8)])
def test_group_rms_norm_store_and_accumulate(rows, cols, groups):
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols + 3)).astype(np.float32)
    w = bf16_round(1.0 + 0.3 * rng.standard_normal(cols))
    y0 = rng.standard_normal((rows, cols + 1)).astype(np.float32)
    want = orc.group_rms_norm(t64(x[:, :cols]), t64(w), groups, 1e-6).numpy()
    L = capi()
    for acc in (0, 1):
        xd, wd, yd = dev32(x), devbf(w), dev32(y0)
        ia.check(L.ifa_group_rmsnorm_f32(p(xd), cols + 3, rows, cols, groups, p(wd), 1e-6, acc, p(yd), cols + 1, None)); sync()
        got = yd.cpu().numpy()
        ref = want + (y0[:, :cols] if acc else 0)
        assert np.abs(got[:, :cols] - ref).max() < 1e-5 * max(1.0, np.abs(ref).max())
        assert np.array_equal(got[:, cols:], y0[:, cols:])


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_residual_convolution_whole_and_in_portions_with_reused_slots(taps):
    rng = np.random.default_rng(taps)
    C_, n = 70, 23
    w = bf16_round(0.5 * rng.standard_normal((C_, taps)))
    L = capi()
    slots = Slots(2, (taps - 1) * C_ + 4)
    wd = devbf(w)
    for seq in range(3):          # the third sequence reuses slot 0 after another one
        x = rng.standard_normal((n, C_)).astype(np.float32)
        want = orc.input_conv(t64(x), t64(w)).numpy()
        for sizes in ([n], [1] * n, [2, 1, 7, 13], [taps + 2, 1, 1, 1, n]):
            at, out = 0, []
            for sz in sizes:
                sz = min(sz, n - at)
                if sz <= 0:
                    break
                sd, rs, rows = seq_tables([(sz, at, seq % 2)])
                xd = dev32(x[at:at + sz]); yd = torch.zeros((sz, C_), dtype=torch.float32, device="cuda")
                ia.check(L.ifa_shortconv_residual_f32(p(xd), C_, C_, taps, p(wd), p(sd), p(rs), rows, p(slots.table), 0, p(yd), C_, None))
                ia.check(L.ifa_shortconv_tail_f32(p(xd), C_, C_, taps, p(sd), 1, p(slots.table), 0, None)); sync()
                out.append(yd.cpu().numpy()); at += sz
            assert np.abs(np.concatenate(out, 0) - want).max() < 1e-5, (seq, sizes)


def test_depth_average_soft_cap_and_embedding_rows():
    rng = np.random.default_rng(3)
    rows, cols, count = 7, 24, 4
    L = capi()
    stack = rng.standard_normal((count, 9, cols)).astype(np.float32)      # planes of 9 rows, 7 used
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    w = bf16_round(rng.standard_normal(count))
    sd, xd, wd = dev32(stack), dev32(x), devbf(w)
    ia.check(L.ifa_depth_average_f32(p(xd), rows, cols, p(sd), 9 * cols, count, p(wd), None)); sync()
    planes = [stack[j, :rows] for j in range(count - 1)] + [x]
    want = sum(float(w[j]) * planes[j].astype(np.float64) for j in range(count))
    assert np.abs(xd.cpu().numpy() - want).max() < 1e-5
    assert np.array_equal(sd.cpu().numpy()[count - 1, :rows], x)
    z = (20 * rng.standard_normal(300)).astype(np.float32)
    zd = dev32(z)
    ia.check(L.ifa_softcap_f32(p(zd), 300, 7.5, None)); sync()
    assert np.abs(zd.cpu().numpy() - 7.5 * np.tanh(z.astype(np.float64) / 7.5)).max() < 1e-5
    emb = bf16_round(rng.standard_normal((13, 10)))
    toks = np.array([3, 0, 12, 3], np.int32)
    out = torch.zeros((4, 10), dtype=torch.float32, device="cuda")
    ia.check(L.ifa_embed_rows_f32(p(devbf(emb)), 13, 10, p(devi(toks)), 4, p(out), None)); sync()
    assert np.array_equal(out.cpu().numpy(), emb[toks])


def yarn_freq(rot):
    """frequencies (float64) and the factor on cos / sin, from the oracle's own tables at position 1"""
    import math
    dims, base = rot["dims"], float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        d = lambda t: dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
        lo, hi = max(math.floor(d(sc["fast"])), 0), min(math.ceil(d(sc["slow"])), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mult = 0.1 * math.log(sc["factor"]) + 1.0
    return f, mult


def latent_case(rng, H, dn, dr, dv, R, rot, first):
    mx = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "kv_rank": R, "rot": rot, "scale": 1.0 / np.sqrt(dn + dr)}
    P = {"m.dkv.norm": bf16_round(1.0 + 0.2 * rng.standard_normal(R)), "m.uk": bf16_round(rng.standard_normal((H * dn, R)) / np.sqrt(R)),
         "m.uv": bf16_round(rng.standard_normal((H * dv, R)) / np.sqrt(R))}
    return mx, P


def run_latent(L, mx, P, q, kv, gate, seqs, slots, expanded, first, ops32=1, window_kernel=False):
    """the worker's sequence of ops over one step; q [rows, H (dn + dr)], kv [rows, R + dr], gate [rows, H] or None.  expanded: keys / values
    from the cached latents + the tiled kernel; else the absorbed form through the head-sharing single-row kernel, or (window_kernel)
    through the general single-row kernel with one shared KV head whose value row is its key row"""
    H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    CR, QD, OV = R + dr, H * (dn + dr), H * dv
    rot = dict(mx["rot"])
    if not first:
        rot.pop("scaling", None)
    f, mult = yarn_freq(rot)
    fd = torch.from_numpy(np.ascontiguousarray(f if len(f) else np.zeros(1))).cuda()
    sd, rs, rows = seq_tables(seqs)
    qd, kvd = dev32(q), dev32(kv)
    gd = dev32(gate) if gate is not None else None
    ia.check(L.ifa_latent_prepare_f32(p(kvd), CR, R, dr, rot["dims"], p(devbf(P["m.dkv.norm"])), 1e-6, p(qd), QD, H, dn, p(fd), mult, p(sd), p(rs), rows, p(slots.table), 0,
                                      None))
    out = torch.zeros((rows, OV), dtype=torch.float32, device="cuda")
    uk, uv = devbf(P["m.uk"]), devbf(P["m.uv"])
    if expanded:
        ctx0, tot = [], 0
        for (n, pos0, slot) in seqs:
            ctx0.append(tot); tot += pos0 + n
        kx = torch.zeros((tot, H * dn), dtype=torch.float32, device="cuda"); vx = torch.zeros((tot, OV), dtype=torch.float32, device="cuda")
        for i, (n, pos0, slot) in enumerate(seqs):
            lat = slots.mem[slot].data_ptr()
            ia.check(L.ifa_linear_bf16w(p(uk), H * dn, R, C.c_void_p(lat), CR, pos0 + n, None, None, 1.0, 0, ops32, C.c_void_p(kx.data_ptr() + ctx0[i] * H * dn * 4), H * dn,
                                        0, 0, None))
            ia.check(L.ifa_linear_bf16w(p(uv), OV, R, C.c_void_p(lat), CR, pos0 + n, None, None, 1.0, 0, ops32, C.c_void_p(vx.data_ptr() + ctx0[i] * OV * 4), OV, 0, 0, None))
        host = np.array([v for (r0, (n, pos0, slot)) in zip(np.cumsum([0] + [s[0] for s in seqs[:-1]]), seqs) for v in (r0, n, pos0, slot)], np.int32)
        assert L.ifa_attention_latent_tile_fits(dn, dr, dv) == 1
        ia.check(L.ifa_attention_latent_tile_f32(p(qd), QD, H, dn, dr, dv, R, mx["scale"], p(kx), H * dn, p(vx), OV, p(devi(ctx0)), p(gd) if gd is not None else None, H,
                                                 p(sd), host.ctypes.data_as(C.c_void_p), len(seqs), p(slots.table), 0, p(out), OV, None))
    else:
        qa = torch.zeros((rows, H * CR), dtype=torch.float32, device="cuda")
        ia.check(L.ifa_latent_absorb_q_f32(p(qd), QD, H, dn, dr, R, p(uk), rows, p(qa), H * CR, None))
        if window_kernel:
            ol = torch.zeros_like(qa)
            ws = torch.zeros(rows * H * 32 * (CR + 2), dtype=torch.float32, device="cuda")
            ia.check(L.ifa_attention_window_f32(p(qa), H * CR, H, 1, CR, 0, 1e-6, mx["scale"], 0.0, 4096, 0, None, None, 0, None, p(sd), p(rs), rows, p(slots.table), 0, 0,
                                                p(ol), H * CR, None, 0, 1 << 30, p(ws), ws.numel() * 4, None))
            ia.check(L.ifa_latent_expand_out_f32(p(ol), H * CR, CR, H, dv, R, p(uv), p(gd) if gd is not None else None, H, rows, p(out), OV, None))
        else:
            ol = torch.zeros((rows, H * R), dtype=torch.float32, device="cuda")
            ws = torch.zeros(rows * H * 8 * (R + 2), dtype=torch.float32, device="cuda")          # room for 8 key shares a row
            ia.check(L.ifa_attention_latent_rows_f32(p(qa), H * CR, H, R, dr, mx["scale"], p(sd), p(rs), rows, p(slots.table), 0, 160, p(ws), ws.numel() * 4, p(ol), H * R, None))
            ia.check(L.ifa_latent_expand_out_f32(p(ol), H * R, R, H, dv, R, p(uv), p(gd) if gd is not None else None, H, rows, p(out), OV, None))
    sync()
    return out.cpu().numpy()


@pytest.mark.parametrize("H,dn,dr,dv,R,rdims,first", [(2, 16, 8, 24, 32, 8, True), (4, 32, 16, 72, 48, 16, False), (1, 5, 6, 7, 9, 4, True), (2, 128, 64, 128, 224, 64, False),
                                                      (3, 48, 0, 16, 20, 0, False), (6, 24, 16, 32, 600, 16, True), (9, 8, 4, 8, 144, 4, False)])
def test_latent_attention_both_forms_whole_portions_and_several_sequences(H, dn, dr, dv, R, rdims, first):
    rng = np.random.default_rng(H * 100 + dn + R)
    rot = {"base": 500.0, "dims": rdims}
    if first:
        rot["scaling"] = {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}
    mx, P = latent_case(rng, H, dn, dr, dv, R, rot, first)
    Pt = {k: t64(v) for k, v in P.items()}
    L = capi()
    lens = [150, 37, 1]
    data = []
    for n in lens:
        q = rng.standard_normal((n, H * (dn + dr))).astype(np.float32)
        kv = rng.standard_normal((n, R + dr)).astype(np.float32)
        g = rng.standard_normal((n, H)).astype(np.float32) if first else None
        want = orc.latent_attention_core(t64(q), t64(kv), Pt, "m.", mx, first, 1e-6, t64(g) if first else None).numpy()
        data.append((q, kv, g, want))
    slots = Slots(3, 160 * (R + dr) + 4)
    tol = 2e-5 * max(1.0, max(np.abs(d[3]).max() for d in data))
    # whole sequences in one step, in the tiled form and in the single-row form
    for expanded, window_kernel in ((True, False), (False, False), (False, True)):
        seqs = [(n, 0, i) for i, n in enumerate(lens)]
        q = np.concatenate([d[0] for d in data]); kv = np.concatenate([d[1] for d in data])
        g = np.concatenate([d[2] for d in data]) if first else None
        got = run_latent(L, mx, P, q, kv, g, seqs, slots, expanded, first, window_kernel=window_kernel)
        assert np.abs(got - np.concatenate([d[3] for d in data])).max() < tol, (expanded, window_kernel)
    # the first two sequences in portions (slots swapped: reused), a prefix in one form and the rest in the other or token by token
    for (first_part, rest_expanded, step) in ((100, True, 50), (129, False, 1), (31, True, 33), (2, False, 1)):
        for si, slot in ((0, 1), (1, 0)):
            q, kv, g, want = data[si]
            n, at, out = lens[si], 0, []
            sizes = [min(first_part, n)]
            while sum(sizes) < n:
                sizes.append(min(step, n - sum(sizes)))
            for k, sz in enumerate(sizes):
                exp = True if k == 0 and sz >= 16 else (rest_expanded and sz >= 2)
                out.append(run_latent(L, mx, P, q[at:at + sz], kv[at:at + sz], g[at:at + sz] if first else None, [(sz, at, slot)], slots, exp, first))
                at += sz
            assert np.abs(np.concatenate(out) - want).max() < tol, (first_part, rest_expanded, si)


@pytest.mark.parametrize("rows,n_all,top", [(1, 20, 3), (9, 5, 5), (40, 73, 8), (3, 1, 1), (70, 130, 2)])
def test_router_scores_choices_and_ties(rows, n_all, top):
    rng = np.random.default_rng(rows * n_all)
    z = rng.standard_normal((rows, n_all + 2)).astype(np.float32)
    z[0, :n_all] = 0.25                      # one row of equal scores: the lowest indices win
    corr = bf16_round(0.1 * rng.standard_normal(n_all))
    if rows > 1:
        corr_used = corr
    else:
        corr_used = np.zeros_like(corr)
    L = capi()
    idx = torch.zeros((rows, top), dtype=torch.int32, device="cuda"); wgt = torch.zeros((rows, top), dtype=torch.float32, device="cuda")
    ia.check(L.ifa_moe_route_f32(p(dev32(z)), n_all + 2, rows, n_all, top, p(devbf(corr_used)), p(idx), p(wgt), None)); sync()
    wi, ww = orc.route(t64(z[:, :n_all]), t64(corr_used), top)
    gi, gw = idx.cpu().numpy(), wgt.cpu().numpy()
    s = torch.softmax(t64(z[:, :n_all]), -1).numpy()
    for t in range(rows):
        # the chosen sets agree wherever the oracle's choice scores are not within rounding of each other
        ch = np.sort(s[t] + corr_used.astype(np.float64))[::-1]
        if top == n_all or ch[top - 1] - ch[top] > 1e-6:
            assert sorted(gi[t]) == sorted(wi[t].tolist()), t
        assert np.abs(gw[t] - s[t][gi[t]]).max() < 1e-6
    if rows == 1:
        assert gi[0].tolist() == list(range(top))


@pytest.mark.parametrize("rows,W,n_all,top", [(1, 64, 21, 4), (8, 30, 5, 5), (3, 256, 130, 6)])
def test_router_with_its_product_inside(rows, W, n_all, top):
    rng = np.random.default_rng(rows + W)
    h = rng.standard_normal((rows, W + 2)).astype(np.float32)
    R = bf16_round(rng.standard_normal((n_all, W)) * 0.3)
    corr = bf16_round(0.1 * rng.standard_normal(n_all))
    L = capi()
    idx = torch.zeros((rows, top), dtype=torch.int32, device="cuda"); wgt = torch.zeros((rows, top), dtype=torch.float32, device="cuda")
    ia.check(L.ifa_moe_route_rows_f32(p(dev32(h)), W + 2, rows, W, p(devbf(R)), n_all, top, p(devbf(corr)), p(idx), p(wgt), None)); sync()
    z = t64(h[:, :W]) @ t64(R).T
    wi, ww = orc.route(z, t64(corr), top)
    s = torch.softmax(z, -1).numpy()
    gi, gw = idx.cpu().numpy(), wgt.cpu().numpy()
    for t in range(rows):
        ch = np.sort(s[t] + corr.astype(np.float64))[::-1]
        if top == n_all or ch[top - 1] - ch[top] > 1e-5:
            assert sorted(gi[t]) == sorted(wi[t].tolist()), t
        assert np.abs(gw[t] - s[t][gi[t]]).max() < 1e-5


def test_norm_add_depth_average_convolution_in_one_launch_equals_the_separate_ops():
    rng = np.random.default_rng(8)
    W, taps, groups, count = 48, 3, 4, 3
    L = capi()
    seqs = [(2, 5, 0), (1, 0, 1), (3, 1, 2)]          # continued, new, continued
    sd, rs, rows = seq_tables(seqs)
    cw, nw, dw = devbf(bf16_round(0.5 * rng.standard_normal((W, taps)))), devbf(bf16_round(1 + 0.2 * rng.standard_normal(W))), devbf(bf16_round(rng.standard_normal(count)))
    x0 = rng.standard_normal((rows, W)).astype(np.float32); sub = rng.standard_normal((rows, W + 4)).astype(np.float32)
    stack0 = rng.standard_normal((count, 8, W)).astype(np.float32)
    tails = [rng.standard_normal(((taps - 1) * W + 4,)).astype(np.float32) for _ in range(3)]
    res = []
    for fused in (True, False):
        slots = Slots(3, (taps - 1) * W + 4)
        for i in range(3):
            slots.mem[i].copy_(torch.from_numpy(tails[i]))
        x, st, h = dev32(x0), dev32(stack0), torch.zeros((rows, W), dtype=torch.float32, device="cuda")
        if fused:
            ia.check(L.ifa_norm_add_conv_rows_f32(p(x), rows, W, p(dev32(sub)), W + 4, p(nw), groups, 1e-6, p(st), 8 * W, count, p(dw), p(cw), taps, p(sd), len(seqs), p(rs),
                                                  p(slots.table), 0, p(h), None))
        else:
            ia.check(L.ifa_group_rmsnorm_f32(p(dev32(sub)), W + 4, rows, W, groups, p(nw), 1e-6, 1, p(x), W, None))
            ia.check(L.ifa_depth_average_f32(p(x), rows, W, p(st), 8 * W, count, p(dw), None))
            ia.check(L.ifa_shortconv_residual_f32(p(x), W, W, taps, p(cw), p(sd), p(rs), rows, p(slots.table), 0, p(h), W, None))
            ia.check(L.ifa_shortconv_tail_f32(p(x), W, W, taps, p(sd), len(seqs), p(slots.table), 0, None))
        sync()
        res.append([x.cpu().numpy(), st.cpu().numpy(), h.cpu().numpy()] + [mm.cpu().numpy()[:(taps - 1) * W] for mm in slots.mem])
    for a, b in zip(*res):
        assert np.abs(a - b).max() < 1e-5


@pytest.mark.parametrize("rows,W,F,E,I,top", [(1, 64, 32, 6, 2, 3), (8, 64, 32, 6, 2, 8), (9, 64, 32, 6, 2, 3), (200, 96, 40, 12, 3, 5), (130, 30, 7, 3, 0, 1), (33, 32, 16, 0, 3, 2),
                                               (70, 64, 24, 70, 3, 8)])
def test_experts_row_form_and_grouped_form(rows, W, F, E, I, top):
    rng = np.random.default_rng(rows + W + E)
    h = rng.standard_normal((rows, W + 4)).astype(np.float32)
    P = {"x.router": bf16_round(rng.standard_normal((E + I, W)) * 0.3), "x.correction": bf16_round(0.05 * rng.standard_normal(E + I))}
    for e in range(E):
        P["x.e%d.up" % e] = bf16_round(rng.standard_normal((F, W)) / np.sqrt(W)); P["x.e%d.down" % e] = bf16_round(rng.standard_normal((W, F)) / np.sqrt(F))
    mlp = {"router": {"experts": E, "identity": I, "top": top}, "expert": {"ff": F}}
    Pt = {k: t64(v) for k, v in P.items()}
    want = orc.mixture(t64(h[:, :W]), Pt, "x.", mlp).numpy()
    zi, zw = orc.route(t64(h[:, :W]) @ Pt["x.router"].T, Pt["x.correction"], top)
    L = capi()
    up = devbf(np.concatenate([P["x.e%d.up" % e] for e in range(E)])) if E else None
    down = devbf(np.concatenate([P["x.e%d.down" % e] for e in range(E)])) if E else None
    idx = devi(zi.numpy()); wgt = dev32(zw.numpy())
    nbytes = L.ifa_moe_workspace_bytes(rows, top, W, F, E)
    ws = torch.zeros(nbytes // 4 + 4, dtype=torch.float32, device="cuda")
    y0 = rng.standard_normal((rows, W)).astype(np.float32)
    for ops32, tol in ((1, 2e-5), (0, 2e-2)):
        for acc in (0, 1):
            yd = dev32(y0)
            ia.check(L.ifa_moe_experts_f32(p(dev32(h)), W + 4, rows, W, F, E, I, top, 0, p(up) if E else None, p(down) if E else None, p(idx), p(wgt), ops32, p(ws), nbytes, p(yd), W,
                                           acc, None)); sync()
            ref = want + (y0 if acc else 0)
            assert np.abs(yd.cpu().numpy() - ref).max() < tol * max(1.0, np.abs(want).max()), (ops32, acc)
