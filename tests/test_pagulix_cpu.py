"""Pagulix without a GPU: configuration checks, registry, loader (fused input products, the reordered rotary rows, stacked expert
weights, optional stream coefficients; surplus / missing / misshapen tensors), cache shapes, and closed forms of the restatement."""
import json

import numpy as np
import pytest
import torch

import pagulix_util as U
from oracle import pagulix as O

D, L, A = U.delta_layer, U.latent_layer, U.attn_layer


def small():
    return U.make_config([D(), L(), A(), A(heads=4, kv_heads=2, dim=8, vdim=16, rot_dims=4, mlp=None)])


def test_registry_and_config_checks():
    from aphrodite_engine_amd import registry
    from aphrodite_engine_amd.pagulix import PagulixConfig
    assert "Pagulix" in registry.supported_architectures()
    cfg = PagulixConfig.from_dict(small())
    assert cfg.streams == 3 and cfg.logit_softcap == 9.0 and len(cfg.layers) == 4
    bad = small()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        PagulixConfig.from_dict(bad)
    bad = small()
    bad["layers"][1]["mlp"]["kind"] = "dense"
    with pytest.raises(ValueError):
        PagulixConfig.from_dict(bad)
    bad = small()
    bad["layers"][3]["mixer"]["vdim"] = 24                      # values that cannot be blended with the first blending layer's
    bad["layers"][3]["mixer"]["v_mix"] = True
    with pytest.raises(ValueError):
        PagulixConfig.from_dict(bad)
    plain = small()
    del plain["streams"], plain["residual_mult"], plain["logit_softcap"]
    c = PagulixConfig.from_dict(plain)
    assert (c.streams, c.residual_mult, c.logit_softcap) == (1, 1.0, 0.0)


def load(cfg, W):
    from aphrodite_engine_amd.pagulix import PagulixConfig, PagulixForCausalLM
    m = PagulixForCausalLM(PagulixConfig.from_dict(cfg), torch.float32)
    m.load_weights((k, torch.from_numpy(np.ascontiguousarray(v))) for k, v in W.items())
    return m


def test_loader_places_every_tensor():
    cfg = small()
    W = U.make_weights(cfg, seed=1)
    m = load(cfg, W)
    d0, l1, a2 = m.layers[0].mix, m.layers[1].mix, m.layers[2].mix
    # the delta layer: one input product [q | k | v | g | b | a | padding], the three convolutions stacked alike
    rows = np.concatenate([W["l0.mix." + n] for n in ("q", "k", "v", "g", "b", "a")])
    got = d0.in_proj.weight.numpy()
    np.testing.assert_array_equal(got[:rows.shape[0]], rows)
    assert got.shape[0] % 8 == 0 and not got[rows.shape[0]:].any()
    np.testing.assert_array_equal(d0.conv.numpy(), np.concatenate([W["l0.mix." + n + ".conv"] for n in ("q", "k", "v")]))
    np.testing.assert_array_equal(d0.a_log.numpy(), W["l0.mix.A_log"])
    # the latent layer: rotary rows reordered from neighbouring pairs to pairs half the part apart
    H, d, r, R = l1.heads, l1.dim, l1.rot_dim, l1.kv_rank
    q = l1.in_proj.weight.numpy()[:H * (d + r)].reshape(H, d + r, -1)
    src = W["l1.mix.q"].reshape(H, d + r, -1)
    np.testing.assert_array_equal(q[:, :d], src[:, :d])
    np.testing.assert_array_equal(q[:, d:d + r // 2], src[:, d::2])
    np.testing.assert_array_equal(q[:, d + r // 2:], src[:, d + 1::2])
    dkv = l1.in_proj.weight.numpy()[H * (d + r):H * (d + r) + R + r]
    np.testing.assert_array_equal(dkv[:R], W["l1.mix.dkv"][:R])
    np.testing.assert_array_equal(dkv[R:R + r // 2], W["l1.mix.dkv"][R::2])
    np.testing.assert_array_equal(l1.sink.numpy(), W["l1.mix.sink"])
    assert l1.window == 13 and l1.uq is None and not l1.gated
    # attention, experts, stream coefficients
    np.testing.assert_array_equal(a2.in_proj.weight.numpy()[:a2.heads * a2.dim], W["l2.mix.q"])
    assert abs(float(a2.v_blend) - float(W["l2.mix.vmix"])) < 1e-7 and m.first_blend == 2
    e = m.layers[0].mlp
    np.testing.assert_array_equal(e.w_gate_up.numpy()[3], np.concatenate([W["l0.mlp.e3.gate"], W["l0.mlp.e3.up"]]))
    np.testing.assert_array_equal(e.router_bias.numpy(), W["l0.mlp.router.b"])
    np.testing.assert_array_equal(e.shared_in.weight.numpy()[:2 * e.shared_ff], np.concatenate([W["l0.mlp.shared.gate"], W["l0.mlp.shared.up"]]))
    np.testing.assert_array_equal(m.layers[1].hc2.mix.numpy(), W["l1.hc2.mix"])
    assert m.layers[3].mlp is None and m.layers[3].hc2 is None
    # caches: convolution state + matrix state, a latent cache, two paged caches
    shapes = [[tuple(t.shape) for t in (c if isinstance(c, tuple) else (c,))] for c in m.make_caches(5, 16, 2, "cpu")]
    assert shapes[0] == [(2, 2, 2 * 2 * 24 + 4 * 40)] and shapes[1] == [(2, 4, 24, 40)] and shapes[2] == [(5, 16, 48 + 8)]
    assert shapes[3] == [(5, 16, 2, 24), (5, 16, 2, 16)]


def test_loader_refuses_surplus_missing_and_misshapen_tensors():
    cfg = small()
    W = U.make_weights(cfg, seed=2)
    with pytest.raises(ValueError, match="unexpected"):
        load(cfg, dict(W, **{"l0.mix.extra": W["l0.norm1"]}))
    with pytest.raises(ValueError, match="lacks"):
        load(cfg, {k: v for k, v in W.items() if k != "l1.mix.sink"})
    with pytest.raises(ValueError, match="does not fit"):
        load(cfg, dict(W, **{"l2.mix.k": W["l2.mix.k"][:-1]}))
    # stream coefficients and layer scales are optional: without them a layer is the plain pre-norm residual
    m = load(cfg, {k: v for k, v in W.items() if ".hc" not in k and ".ls" not in k})
    assert torch.equal(m.layers[0].hc1.mix, torch.eye(3)) and float(m.layers[0].hc1.scale.min()) == 1.0


def test_wavelength_scaled_frequencies():
    from aphrodite_engine_amd.mixers import RotaryFrequencies
    for rot in ({"base": 500000.0, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}},
                {"base": 3000.0, "dims": 12, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}},
                {"base": 100.0, "dims": 6, "scaling": {"factor": 2.0, "low": 2.0, "high": 16.0, "original": 50}}):
        sc = rot["scaling"]
        got = RotaryFrequencies.wavelength_scaled(rot["dims"], rot["base"], sc["factor"], sc["low"], sc["high"], sc["original"]).inv_freq
        want = O.rotary_frequencies(rot)
        np.testing.assert_allclose(got.numpy(), want, rtol=1e-6)
        plain = O.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]})
        assert (want <= plain + 1e-15).all() and (want >= plain / sc["factor"] - 1e-15).all()
        if rot["dims"] == 64:                                     # short waves kept, long ones slowed down by the whole factor
            assert want[0] == plain[0] and abs(want[-1] - plain[-1] / sc["factor"]) < 1e-15 and 0 < (want < plain).sum() < 32


def test_restatement_closed_forms():
    rng = np.random.default_rng(0)
    # a rotation keeps lengths and makes scores depend on the distance only, in both layouts
    rot = {"base": 100.0, "dims": 8}
    x, y = rng.standard_normal((1, 12)), rng.standard_normal((1, 12))
    for layout in ("half", "interleaved"):
        a = O.rotate(x, [5], rot, layout) @ O.rotate(y, [2], rot, layout).T
        b = O.rotate(x, [105], rot, layout) @ O.rotate(y, [102], rot, layout).T
        assert abs(a - b) < 1e-9
        np.testing.assert_allclose(np.linalg.norm(O.rotate(x, [7], rot, layout)), np.linalg.norm(x))
        np.testing.assert_array_equal(O.rotate(x, [7], rot, layout)[:, 8:], x[:, 8:])
    # the reordering the loader applies turns one layout into the other
    from aphrodite_engine_amd.mixers import interleaved_to_half
    w = torch.arange(14.0).unsqueeze(1)
    perm = interleaved_to_half(w, 8, at=3).squeeze(1).long().numpy()
    z = rng.standard_normal((3, 14))
    z[:, :3] = z[:, 11:] = 0
    np.testing.assert_allclose(O.rotate(z[:, 3:], [4, 5, 6], rot, "interleaved")[:, perm[3:11] - 3],
                               O.rotate(z[:, perm][:, 3:], [4, 5, 6], rot, "half")[:, :8])
    # the window: row i sees i - j < window; the sink takes weight but gives nothing
    q, k, v = rng.standard_normal((9, 4)), rng.standard_normal((9, 4)), rng.standard_normal((9, 3))
    full = O.masked_attention(q, k, v, 0.5)
    np.testing.assert_allclose(O.masked_attention(q, k, v, 0.5, window=9), full)
    np.testing.assert_allclose(O.masked_attention(q, k, v, 0.5, window=1), v)
    s = (k[:5] @ q[4]) * 0.5
    w = np.exp(s) / (np.exp(s).sum() + np.exp(0.7))
    np.testing.assert_allclose(O.masked_attention(q, k, v, 0.5, sink=0.7)[4], w @ v[:5])
    # the delta rule with beta = 1, g = 1 and orthonormal keys stores the last value per key
    keys = np.eye(4)[[0, 1, 0]]
    vals = rng.standard_normal((3, 2))
    out = O.delta_rule(np.eye(4)[[0, 0, 0]], keys, vals, np.ones(3), np.ones(3))
    np.testing.assert_allclose(out, vals[[0, 0, 2]], atol=1e-12)
    # the router: softmax over the chosen logits only
    ids, wts = O.route(np.array([0.1, 2.0, -1.0, 2.0, 0.5]), 3)
    assert ids == [1, 3, 4] and abs(wts.sum() - 1) < 1e-12 and abs(wts[0] - wts[1]) < 1e-12
    # convolution: the last column is the current token's tap
    u = rng.standard_normal((5, 2))
    wc = np.array([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]])
    y = O.causal_conv(u, wc)
    np.testing.assert_allclose(y[:, 0], u[:, 0])
    np.testing.assert_allclose(y[2:, 1], u[:3, 1])
    assert (y[:2, 1] == 0).all()


def test_one_stream_without_coefficients_is_the_plain_residual():
    cfg = U.make_config([A(v_mix=False, mlp=None), D(mlp=None)], streams=1, residual_mult=0.5, softcap=0.0)
    W = {k: v for k, v in U.make_weights(cfg, seed=3).items() if ".hc" not in k and ".ls" not in k}
    toks = [3, 9, 27, 81, 5]
    trace = []
    O.forward(cfg, W, toks, trace)
    x = W["embed"][toks].astype(np.float64)
    h = O.rms_norm(x, W["l0.norm1"], cfg["norm"]["eps"])
    y, _ = O.attention(h, W, "l0.mix.", cfg["layers"][0]["mixer"], cfg["norm"]["eps"])
    np.testing.assert_allclose(trace[0], x + 0.5 * y)
