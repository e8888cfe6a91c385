"""Fekotar without a GPU: configuration checks, the registry, the loader (fused projections, stacked expert weights, biases;
surplus / missing / misshapen tensors), the rotation's frequencies, the pair hash, and closed forms of the restatement
(oracle/fekotar.py) -- among them the identity the kernels rest on: attention over per-head keys and values made from the
latent equals attention IN the latent with the key matrix carried over to the query and the value matrix applied afterwards."""
import math

import numpy as np
import pytest
import torch

import fekotar_util as U
from oracle import fekotar as O

A = U.latent_layer


def small_config():
    return U.make_config([A(), A(heads=2, dim=16, rot_dim=12, vdim=24, q_rank=40, kv_rank=36, scaling=None, mlp="moe"), A(mlp=None, rot_dim=4)])


def test_registry_names_the_architecture():
    from aphrodite_engine_amd import registry
    assert "Fekotar" in registry.supported_architectures()
    assert registry.architecture_of(small_config()) == "Fekotar"
    assert callable(registry.resolve(small_config()))


def test_config_refuses_what_it_does_not_know():
    from aphrodite_engine_amd.fekotar import FekotarConfig
    c = small_config()
    cfg = FekotarConfig.from_dict(c)
    assert cfg.bigram == {"buckets": 61, "mul_prev": 13, "mul_cur": 5} and len(cfg.layers) == 3
    bad = small_config()
    bad["layers"][1]["type"] = "attention"
    with pytest.raises(ValueError):
        FekotarConfig.from_dict(bad)
    bad = small_config()
    bad["layers"][0]["mlp"]["kind"] = "sparse"
    with pytest.raises(ValueError):
        FekotarConfig.from_dict(bad)
    assert FekotarConfig.from_dict(U.make_config([A()], bigram=None)).bigram is None


def test_router_configuration_is_checked():
    from aphrodite_engine_amd.mixers import RoutedExperts
    with pytest.raises(ValueError):
        RoutedExperts(16, 8, 6, 2, 0, 0.0, torch.float32, score="sigmoid_grouped", groups=4, keep=1)       # 6 experts in 4 groups
    with pytest.raises(ValueError):
        RoutedExperts(16, 8, 6, 3, 0, 0.0, torch.float32, score="sigmoid_grouped", groups=3, keep=1)       # top 3 of one group of 2
    with pytest.raises(ValueError):
        RoutedExperts(16, 8, 6, 2, 0, 0.0, torch.float32, score="sigmoid_grouped", groups=3, keep=4)


def test_loader_fills_fused_products_and_refuses_wrong_checkpoints(tmp_path):
    from aphrodite_engine_amd.loader import load_model
    cfg = small_config()
    W = U.make_weights(cfg)
    path = U.write_checkpoint(str(tmp_path / "m"), cfg, W)
    m = load_model(path, dtype=torch.float32, device="cpu")
    assert type(m).__name__ == "FekotarForCausalLM" and m.vocab_size == cfg["vocab"]
    mix = m.layers[0].mix
    w = mix.in_proj.weight.detach().numpy()
    np.testing.assert_array_equal(w[:56], W["l0.mix.dq"])
    np.testing.assert_array_equal(w[56:56 + 56], W["l0.mix.dkv"])
    np.testing.assert_array_equal(w[112:112 + 120], W["l0.mix.g"])
    assert w.shape[0] % 8 == 0 and not w[232:].any()
    np.testing.assert_array_equal(mix.w_uk.detach().numpy().reshape(3 * 24, 48), W["l0.mix.uk"])
    np.testing.assert_array_equal(mix.w_uv.detach().numpy().reshape(3 * 40, 48), W["l0.mix.uv"])
    np.testing.assert_array_equal(mix.q_norm.detach().numpy(), W["l0.mix.dq.norm"])
    mlp = m.layers[0].mlp
    np.testing.assert_array_equal(mlp.gate_up.weight.detach().numpy(), np.concatenate([W["l0.mlp.gate"], W["l0.mlp.up"]]))
    np.testing.assert_array_equal(mlp.gate_up.bias.detach().numpy(), np.concatenate([W["l0.mlp.gate.b"], W["l0.mlp.up.b"]]))
    np.testing.assert_array_equal(mlp.down.bias.detach().numpy(), W["l0.mlp.down.b"])
    moe = m.layers[1].mlp
    np.testing.assert_array_equal(moe.w_gate_up[4, 88:].detach().numpy(), W["l1.mlp.e4.up"])
    np.testing.assert_array_equal(moe.w_down[5].detach().numpy(), W["l1.mlp.e5.down"])
    assert moe.router.dtype == torch.float32 and m.layers[2].mlp is None
    np.testing.assert_array_equal(m.embed.pair_table.detach().numpy(), W["bigram"])
    # caches: the previous tokens, then one latent cache per layer, rows of rank + rotary part
    caches = m.make_caches(6, 16, 3, "cpu")
    assert caches[0].dtype == torch.int32 and tuple(caches[0].shape) == (3,)
    assert [tuple(c.shape) for c in caches[1:]] == [(6, 16, 56), (6, 16, 48), (6, 16, 52)]
    for change in ("surplus", "missing", "shape"):
        W2 = dict(W)
        if change == "surplus":
            W2["l0.mix.k"] = W["l0.mix.uk"]
        elif change == "missing":
            del W2["l1.mlp.e2.down"]
        else:
            W2["l0.mix.dq.norm"] = W["l0.mix.dkv.norm"]
        with pytest.raises(ValueError):
            load_model(U.write_checkpoint(str(tmp_path / change), cfg, W2), dtype=torch.float32, device="cpu")
    W2 = dict(W)
    del W2["head"]                                    # no output matrix: the embedding's
    tied = load_model(U.write_checkpoint(str(tmp_path / "tied"), cfg, W2), dtype=torch.float32, device="cpu")
    assert tied.head is tied.embed.table


def test_rotation_frequencies_plain_and_scaled():
    from aphrodite_engine_amd.mixers import RotaryFrequencies
    plain = RotaryFrequencies(8, 100.0)
    np.testing.assert_allclose(plain.inv_freq.numpy(), [1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75], rtol=1e-6)
    assert plain.mscale == 1.0
    rot = {"base": 5000.0, "dims": 16, "scaling": {"factor": 4.0, "original": 128, "fast": 8.0, "slow": 0.5}}
    f, mult = O.rotary_frequencies(rot)
    r = RotaryFrequencies(16, 5000.0, 4.0, 128, 8.0, 0.5)
    np.testing.assert_allclose(r.inv_freq.numpy(), f, rtol=1e-6)
    assert abs(r.mscale - (0.1 * math.log(4.0) + 1)) < 1e-12 and abs(mult - r.mscale) < 1e-12
    base = np.array([5000.0 ** (-2 * i / 16) for i in range(8)])
    assert f[0] == base[0]                                 # the fastest number keeps its frequency
    assert abs(f[-1] - base[-1] / 4.0) < 1e-15             # the slowest is interpolated
    assert all(base[i] / 4.0 - 1e-15 <= f[i] <= base[i] + 1e-15 for i in range(8))
    with pytest.raises(ValueError):
        RotaryFrequencies(7, 100.0)


def test_rotate_is_a_rotation_of_pairs_and_passes_the_rest():
    rot = {"base": 50.0, "dims": 4}
    x = np.array([[1.0, 2.0, 3.0, 4.0, 9.0]])
    y = O.rotate(np.repeat(x, 3, 0), [0, 1, 5], rot)
    np.testing.assert_allclose(y[0], x[0])
    f = [1.0, 50.0 ** -0.5]
    for row, p in ((1, 1), (2, 5)):
        for i in range(2):
            a = p * f[i]
            np.testing.assert_allclose([y[row, i], y[row, i + 2]], [x[0, i] * math.cos(a) - x[0, i + 2] * math.sin(a),
                                                                     x[0, i + 2] * math.cos(a) + x[0, i] * math.sin(a)])
        assert y[row, 4] == 9.0
    # relative positions only: <rot(q, i), rot(k, j)> depends on i - j
    rng = np.random.default_rng(0)
    q, k = rng.standard_normal((1, 4)), rng.standard_normal((1, 4))
    d1 = O.rotate(q, [7], rot) @ O.rotate(k, [3], rot).T
    d2 = O.rotate(q, [24], rot) @ O.rotate(k, [20], rot).T
    np.testing.assert_allclose(d1, d2)


def test_pair_rows():
    assert O.pair_rows([5], 7, 3, 2) == [7]
    assert O.pair_rows([5, 6, 1], 7, 3, 2) == [7, (5 * 3 + 6 * 2) % 7, (6 * 3 + 1 * 2) % 7]
    assert O.pair_rows([4, 4, 4], 1, 3, 2) == [1, 0, 0]


def test_route_closed_forms():
    z = np.array([3.0, -9, -9, -9, 2.0, 1.9, -9, -9])
    assert O.route(z, 2, 2, 1, 1.0)[0] == [4, 5]          # one loud expert loses to a group with two
    chosen, w = O.route(z, 2, 2, 2, 2.0)
    assert chosen == [0, 4]
    np.testing.assert_allclose(w, [2 * O.sigmoid(3.0), 2 * O.sigmoid(2.0)])
    assert O.route(np.zeros(6), 3, 3, 2, 1.0)[0] == [0, 1, 2]      # ties: the lower index


def test_attention_in_the_latent_equals_attention_over_materialised_heads():
    cfg = U.make_config([A(heads=3, dim=10, rot_dim=6, vdim=14, q_rank=20, kv_rank=12, mlp=None)], width=24)
    W = {k: v.astype(np.float64) for k, v in U.make_weights(cfg, seed=3, round_bf16=False).items()}
    mc, eps = cfg["layers"][0]["mixer"], 1e-5
    rng = np.random.default_rng(1)
    T, H, d, r, e, R = 17, 3, 10, 6, 14, 12
    h = rng.standard_normal((T, 24))
    want = O.latent_attention(h, W, "l0.mix.", mc, eps)
    p = "l0.mix."
    q = (O.rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps) @ W[p + "uq"].T).reshape(T, H, d + r)
    down = h @ W[p + "dkv"].T
    rows = np.concatenate([O.rms_norm(down[:, :R], W[p + "dkv.norm"], eps), O.rotate(down[:, R:], np.arange(T), mc["rot"])], -1)
    uk, uv = W[p + "uk"].reshape(H, d, R), W[p + "uv"].reshape(H, e, R)
    out = np.zeros((T, H, e))
    for a in range(H):
        qa = np.concatenate([q[:, a, :d] @ uk[a], O.rotate(q[:, a, d:], np.arange(T), mc["rot"])], -1)      # [T, R + r]
        s = qa @ rows.T * mc["scale"]
        s[np.triu_indices(T, 1)] = -np.inf
        pr = np.exp(s - s.max(-1, keepdims=True))
        pr /= pr.sum(-1, keepdims=True)
        out[:, a] = (pr @ rows[:, :R]) @ uv[a].T
    got = (out.reshape(T, H * e) * O.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-9)


def test_forward_first_token_and_prefix_property():
    cfg = small_config()
    W = U.make_weights(cfg, seed=2)
    toks = [5, 9, 9, 100, 3, 77]
    full = O.forward(cfg, W, toks)
    np.testing.assert_allclose(O.forward(cfg, W, toks[:4]), full[:4], rtol=1e-9, atol=1e-9)      # causal
    assert np.abs(O.forward(cfg, W, [9, 100])[1] - full[3]).max() > 1e-3                          # the context matters
    # the dense feed-forward's clamps are live at these weights
    h = np.random.default_rng(0).standard_normal((50, cfg["width"])) * 2
    g = h @ W["l0.mlp.gate"].T + W["l0.mlp.gate.b"]
    assert (g > cfg["layers"][0]["mlp"]["limit"]).any()
