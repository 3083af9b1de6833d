"""The float64 Muzopel oracle checked against properties that follow from its equations (CPU only): causality, the zero history in
front of a sequence, the router's tie rule and plain-score weights, identity experts, the depth average, the rotation's scaling."""
import math

import numpy as np
import torch

from tests import muzopel_fixtures as fx
from tests import muzopel_oracle as orc

CFG = fx.config([fx.latent2_layer(), fx.latent_layer(), fx.latent2_layer(mlp=None)], width=32, vocab=41)


def test_a_prefix_has_the_logits_it_has_inside_the_longer_sequence():
    P = fx.oracle_weights(fx.random_weights(CFG, 1))
    toks = [int(t) for t in np.random.default_rng(2).integers(0, 41, 30)]
    whole = orc.forward(CFG, P, toks)
    for n in (1, 2, 3, 17):
        assert (orc.forward(CFG, P, toks[:n]) - whole[:n]).abs().max() < 1e-10


def test_input_convolution_sees_zeros_before_the_sequence():
    w = orc.t64(np.array([[0.5, -1.0, 2.0], [1.0, 1.0, 1.0]]))
    h = orc.t64(np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]]))
    got = orc.input_conv(h, w)
    want = np.array([[1 + 2 * 1, 10 + 10], [2 + 2 * 2 - 1, 20 + 30], [3 + 2 * 3 - 2 + 0.5, 30 + 60], [4 + 2 * 4 - 3 + 1.0, 40 + 90]])
    assert np.allclose(got.numpy(), want)


def test_router_ties_weights_and_identity_experts():
    z = orc.t64(np.zeros((1, 5)))
    idx, wgt = orc.route(z, orc.t64(np.zeros(5)), 2)
    assert idx.tolist() == [[0, 1]] and np.allclose(wgt.numpy(), 0.2)
    idx, wgt = orc.route(z, orc.t64(np.array([0, 0, 0, 1.0, 0.5])), 2)
    assert idx.tolist() == [[3, 4]] and np.allclose(wgt.numpy(), 0.2)          # the correction chooses, the plain score weighs
    mlp = fx.moe(experts=0, identity=2, top=2, ff=4)
    h = orc.t64(np.random.default_rng(3).standard_normal((3, 8)))
    P = {"x.router": orc.t64(np.zeros((2, 8))), "x.correction": orc.t64(np.zeros(2))}
    assert np.allclose(orc.mixture(h, P, "x.", mlp).numpy(), h.numpy())        # two identity experts of weight one half each


def test_depth_average_that_keeps_only_the_newest_result_changes_nothing():
    w = fx.random_weights(CFG, 4)
    plain = dict(w)
    for li in range(len(CFG["layers"])):
        d = np.zeros(li + 2, np.float32); d[-1] = 1.0
        plain["l%d.dwa" % li] = d
    toks = [1, 5, 9, 2, 2, 7]
    a = orc.forward(CFG, fx.oracle_weights(plain), toks)
    # the same stack written without any averaging
    P = fx.oracle_weights(plain)
    eps, G = CFG["norm"]["eps"], CFG["norm"]["groups"]
    x = orc.group_rms_norm(P["embed"][torch.as_tensor(toks)], P["embed.norm"], G, eps)
    for li, L in enumerate(CFG["layers"]):
        p = "l%d." % li
        x = x + orc.group_rms_norm(orc.latent_attention(orc.input_conv(x, P[p + "canon1"]), P, p + "mix.", L["mixer"], L["type"], eps), P[p + "norm1"], G, eps)
        if L.get("mlp"):
            x = x + orc.group_rms_norm(orc.mixture(orc.input_conv(x, P[p + "canon2"]), P, p + "mlp.", L["mlp"]), P[p + "norm2"], G, eps)
    lg = orc.group_rms_norm(x, P["final.norm"], G, eps) @ P["head"].T
    assert np.allclose(a.numpy(), (CFG["logit_softcap"] * torch.tanh(lg / CFG["logit_softcap"])).numpy())


def test_scaled_rotation_keeps_fast_pairs_and_slows_slow_pairs():
    rot = {"base": 5000.0, "dims": 12, "scaling": {"factor": 4.0, "original": 512, "fast": 16.0, "slow": 2.0}}
    cos, sin = orc.rotation_tables(rot, 2)
    mult = 0.1 * math.log(4.0) + 1.0
    f = 5000.0 ** (-2.0 * np.arange(6) / 12)
    ang = np.arctan2(sin[1].numpy(), cos[1].numpy())
    assert np.allclose(np.hypot(cos[1].numpy(), sin[1].numpy()), mult)
    assert np.isclose(ang[0], f[0]) and np.isclose(ang[-1], f[-1] / 4.0)       # the fastest pair is untouched, the slowest divided by the factor
    assert np.all(ang <= f + 1e-12) and np.all(ang >= f / 4.0 - 1e-12)
