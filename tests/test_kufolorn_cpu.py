"""Kufolorn without a GPU: pins of the plain implementation (tests/plain_kufolorn.py) against closed forms written
another way, the typed configuration and its errors, the model as data (order, tensors), and what the entries ask of
the cache."""
import copy
import math

import numpy as np
import pytest

import kufolorn_cases as cases
import plain_kufolorn as plain


# ------------------------------------------------------------------------------------- the plain implementation
def test_gelu_values():
    assert plain.gelu_tanh(np.array(0.0)) == 0.0
    assert abs(plain.gelu_tanh(np.array(1.0)) - 0.8411919906082768) < 1e-12
    assert abs(plain.gelu_tanh(np.array(-3.0)) + 0.0036373920817729943) < 1e-12


def test_half_split_rotation_is_a_complex_multiplication_with_scaled_frequencies():
    rng = np.random.default_rng(0)
    v = rng.normal(size=(5, 2, 10))
    pos = np.array([0, 1, 7, 100, 3])
    out = plain.rotate_half(v, pos, {"base": 50.0, "dims": 8, "scaling": {"factor": 4.0}})
    z = (v[..., :4] + 1j * v[..., 4:8]) * np.exp(1j * pos[:, None, None] * 50.0 ** (-2.0 * np.arange(4) / 8) / 4.0)
    assert np.allclose(out[..., :4], z.real) and np.allclose(out[..., 4:8], z.imag) and np.array_equal(out[..., 8:], v[..., 8:])
    assert np.array_equal(out[0], v[0])
    # without scaling the angles are four times as large
    plain4 = plain.rotate_half(v, pos * 4, {"base": 50.0, "dims": 8, "scaling": {"factor": 4.0}})
    assert np.allclose(plain4, plain.rotate_half(v, pos, {"base": 50.0, "dims": 8}))


def test_causal_convolution_against_numpy():
    rng = np.random.default_rng(1)
    u, w = rng.normal(size=(11, 3)), rng.normal(size=(3, 4))
    out = plain.causal_conv(u, w)
    for c in range(3):
        assert np.allclose(out[:, c], np.convolve(u[:, c], w[c, ::-1])[:11])
    assert np.allclose(out[0], w[:, -1] * u[0])              # the last column is the current token's


def test_delta_rule_stores_and_overwrites_a_value():
    """With beta = 1 and no decay, writing v under a unit key k stores it exactly (S^T k = v), writing another value
    under the same key replaces it, and a key at a right angle leaves it alone."""
    k1, k2 = np.array([1.0, 0.0, 0.0]), np.array([0.0, 1.0, 0.0])
    v1, v2, v3 = np.array([2.0, -1.0]), np.array([0.5, 4.0]), np.array([7.0, 7.0])
    k = np.stack([k1, k2, k1, k1])[:, None]
    v = np.stack([v1, v2, v3, v3])[:, None]
    q = np.stack([k1, k1, k1, k2])[:, None]
    ones = np.ones((4, 1))
    o = plain.delta_rule(q, k, v, ones, ones)[:, 0]
    assert np.allclose(o[0], v1) and np.allclose(o[1], v1) and np.allclose(o[2], v3) and np.allclose(o[3], v2)
    # beta = 1/2 moves the stored value half way; a decay g shrinks what was stored BEFORE the token's own write
    o = plain.delta_rule(q[:3], k[[0, 0, 0]], v[[0, 1, 1]], np.array([[1.0], [0.5], [1.0]]), np.array([[1.0], [1.0], [0.5]]))[:, 0]
    assert np.allclose(o[1], 0.5 * (v1 + v2)) and np.allclose(o[2], v2)
    S_read = plain.delta_rule(np.stack([k1, k2])[:, None], np.stack([k1, k2])[:, None], np.stack([v1, v2])[:, None],
                              np.ones((2, 1)), np.array([[1.0], [0.25]]))[:, 0]
    assert np.allclose(S_read[1], v2)                           # reading k2 sees its own write in full
    o = plain.delta_rule(np.stack([k1, k1])[:, None], np.stack([k1, k2])[:, None], np.stack([v1, v2])[:, None],
                         np.ones((2, 1)), np.array([[1.0], [0.25]]))[:, 0]
    assert np.allclose(o[1], 0.25 * v1)                         # ... and what k1 stored has decayed


def test_delta_rule_as_a_product_of_matrices():
    """S_t = g_t (I - beta_t k_t k_t^T) S_(t-1) + beta_t k_t v_t^T, written out with matrices."""
    rng = np.random.default_rng(2)
    T, D, V = 7, 5, 3
    q, k, v = rng.normal(size=(T, 1, D)), plain.unit(rng.normal(size=(T, 1, D))), rng.normal(size=(T, 1, V))
    beta, g = rng.uniform(0.1, 0.9, (T, 1)), rng.uniform(0.5, 1.0, (T, 1))
    S = np.zeros((D, V))
    for t in range(T):
        kk = k[t, 0][:, None]
        S = g[t, 0] * (np.eye(D) - beta[t, 0] * kk @ kk.T) @ S + beta[t, 0] * kk @ v[t, 0][None]
        assert np.allclose(plain.delta_rule(q[:t + 1], k[:t + 1], v[:t + 1], beta[:t + 1], g[:t + 1])[t, 0], S.T @ q[t, 0])


def test_retention_in_closed_form():
    """o_t = sum_{j <= t} decay^(t - j) (q_t . k_j) v_j, scores by distance only."""
    cfg = cases.CONFIG_A
    m = cfg["layers"][1]["mixer"]["right"]
    W = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 3).items()}
    rng = np.random.default_rng(3)
    T, H, D, V = 9, m["heads"], m["dim"], m["vdim"]
    h = rng.normal(size=(T, cfg["width"]))
    p, eps = "l1.mix.right.", cfg["norm"]["eps"]
    ref = plain.retention(h, W, p, m, eps, np.arange(T) + 50)
    q = plain.rotate_half((h @ W[p + "q"].T).reshape(T, H, D), np.arange(T), m["rot"])      # positions shifted: the same scores
    k = plain.rotate_half((h @ W[p + "k"].T).reshape(T, H, D), np.arange(T), m["rot"])
    v = (h @ W[p + "v"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for hd in range(H):
        for t in range(T):
            for j in range(t + 1):
                out[t, hd] += m["decay"][hd] ** (t - j) * (q[t, hd] @ k[j, hd]) / math.sqrt(D) * v[j, hd]
    out = out / np.sqrt(np.mean(out ** 2, axis=-1, keepdims=True) + eps)
    assert np.allclose((out.reshape(T, -1) * plain.silu(h @ W[p + "g"].T)) @ W[p + "o"].T, ref)


def test_softmax_with_a_sink_by_hand():
    """One head, one key size: the weights are exp(s_j) / (sum exp(s) + exp(sink)); a sink of minus infinity is the
    plain softmax, a large one sends the output to zero."""
    cfg = copy.deepcopy(cases.CONFIG_D)
    m = cfg["layers"][1]["mixer"]["left"]
    W = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 4).items()}
    p, eps, T = "l1.mix.left.", cfg["norm"]["eps"], 6
    h = np.random.default_rng(5).normal(size=(T, cfg["width"]))
    pos = np.arange(T)
    W[p + "o"] = np.eye(cfg["width"])[:, :m["vdim"]]             # the heads' outputs themselves
    q = plain.rotate_half((plain.rms(h @ W[p + "q"].T + W[p + "q.b"], eps) * W[p + "q.norm"])[:, None], pos, m["rot"])[:, 0]
    k = plain.rotate_half((plain.rms(h @ W[p + "k"].T + W[p + "k.b"], eps) * W[p + "k.norm"])[:, None], pos, m["rot"])[:, 0]
    v = h @ W[p + "v"].T + W[p + "v.b"]
    gate = plain.sigmoid(h @ W[p + "g"].T)[:, 0]
    for sink in (-1e9, 0.3, 40.0):
        W[p + "sink"] = np.array([sink])
        out = plain.sink_attention(h, W, p, m, eps, pos)[:, :m["vdim"]]
        for t in range(T):
            e = np.exp(k[:t + 1] @ q[t] * m["scale"])
            assert np.allclose(out[t], gate[t] * (e @ v[:t + 1]) / (e.sum() + math.exp(sink)), atol=1e-12)
        if sink == 40.0:
            assert np.abs(out).max() < 1e-12


def test_routing_groups_identity_outputs_and_negative_choice_values():
    W = {"r.correction": np.array([0.0, 0.0, 0.0, 0.0, -5.0, -5.0])}
    # six outputs in three groups of two; scores through the logits; outputs 4, 5 are identity experts
    W["r.router"] = np.eye(6)
    r = {"experts": 4, "identity": 2, "top": 2, "groups": {"count": 3, "keep": 2}}
    h = np.log(np.array([[0.30, 0.05, 0.20, 0.19, 0.25, 0.01]]))
    idx, wt = plain.route(h, W, "r.", r)
    # the last group's choice values are negative (-4.75, -4.99): it is not kept although its score 0.25 is second
    assert idx.tolist() == [[0, 2]] and np.allclose(wt, [[0.30, 0.20]])          # the weights are not renormalised
    W["r.correction"] = np.array([0.0, 0.0, 0.0, 0.0, 0.0, 0.0])
    idx, wt = plain.route(h, W, "r.", r)
    assert idx.tolist() == [[0, 4]] and np.allclose(wt, [[0.30, 0.25]])          # a group's score is its LARGEST choice value
    # all choice values negative: a group that is not kept counts as minus infinity, not as 0
    W["r.correction"] = np.array([-9.0, -9.0, -1.0, -1.0, -2.0, -2.0])
    idx, _ = plain.route(h, W, "r.", {**r, "groups": {"count": 3, "keep": 1}})
    assert idx.tolist() == [[2, 3]]
    # the feed-forward: an identity expert hands the input back, times its weight
    W.update({"r.e%d.%s" % (e, n): np.zeros((6, 6)) for e in range(4) for n in ("gate", "up", "down")})
    W["r.correction"] = np.array([-9.0, -9.0, -9.0, -9.0, 0.0, 0.0])
    out = plain.moe_ff(h, W, "r.", {"router": {**r, "groups": {"count": 1, "keep": 1}}, "expert": {"limit": 1.0}})
    assert np.allclose(out, (0.25 + 0.01) * h)


def test_expert_activation_is_clamped():
    W = {"e.gate": np.eye(3), "e.up": np.eye(3), "e.down": np.eye(3)}
    out = plain.expert(np.array([[5.0, -5.0, 0.5]]), W, "e.", 2.0)[0]
    sg = lambda z: 1.0 / (1.0 + math.exp(-z))
    assert np.allclose(out, [2.0 * sg(3.404) * 3.0, -5.0 * sg(-8.51) * (-2.0 + 1.0), 0.5 * sg(0.851) * 1.5])


def test_the_first_token_sees_the_sink_and_itself_only():
    cfg = cases.CONFIG_D
    W = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 6).items()}
    a = plain.forward(cfg, W, [3, 9, 11])
    b = plain.forward(cfg, W, [3, 1, 2])
    assert np.allclose(a[0], b[0]) and not np.allclose(a[1], b[1])
    assert np.abs(a).max() <= cfg["logit_softcap"]


# ------------------------------------------------------------------------------------------------ configuration
def test_configuration_reads_every_key():
    from litinfer_amd.config import KufolornConfig
    c = KufolornConfig.from_dict(cases.CONFIG_A)
    assert (c.vocab, c.width, c.eps, c.logit_softcap) == (211, 96, 1e-5, 9.0)
    d, p = c.layers[0], c.layers[1]
    assert (d.type, d.mixer.heads, d.mixer.kv_heads, d.mixer.dim, d.mixer.vdim, d.mixer.conv) == ("delta", 6, 3, 24, 16, 4)
    assert (p.mixer.left.heads, p.mixer.left.kv_heads, p.mixer.left.scale, p.mixer.left.rot.dims, p.mixer.left.rot.factor) == (4, 2, 0.2, 8, 4.0)
    assert p.mixer.right.decay == (0.9, 0.97, 0.995) and p.mixer.right.rot.factor == 1.0
    assert (p.mixer.left_scale, p.mixer.right_scale) == (0.7, 0.4)
    assert (p.mlp.experts, p.mlp.identity, p.mlp.top, p.mlp.groups, p.mlp.keep_groups, p.mlp.limit) == (6, 2, 2, 4, 2, 1.5)
    assert c.layers[2].mlp is None and KufolornConfig.from_dict(cases.CONFIG_B).logit_softcap == 0.0


@pytest.mark.parametrize("path,value", [
    (("layers", 0, "type"), "conv"), (("layers", 0, "mixer", "heads"), 4), (("layers", 0, "mixer", "dim"), 0),
    (("layers", 1, "mixer", "left", "kv_heads"), 3), (("layers", 1, "mixer", "left", "rot", "dims"), 7),
    (("layers", 1, "mixer", "left", "rot", "dims"), 26), (("layers", 1, "mixer", "right", "decay"), [0.9, 0.9]),
    (("layers", 1, "mixer", "left", "scale"), None), (("layers", 1, "mixer", "left_scale"), "x"),
    (("layers", 1, "mlp", "router", "top"), 5), (("layers", 1, "mlp", "router", "groups", "count"), 3),
    (("layers", 1, "mlp", "expert", "limit"), 0), (("layers", 0, "mlp", "kind"), "gated"), (("norm", "eps"), -1.0),
    (("vocab",), 0), (("layers",), [])])
def test_configuration_errors(path, value):
    from litinfer_amd.config import ConfigError, KufolornConfig
    cfg = copy.deepcopy(cases.CONFIG_A)
    node = cfg
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ConfigError):
        KufolornConfig.from_dict(cfg)


def test_model_as_data():
    from litinfer_amd.config import architecture_name, lookup
    from litinfer_amd.engine.model import expected_params_of_spec
    arch = lookup(architecture_name(cases.CONFIG_A))
    spec = arch.model_spec(arch.config_from_dict(cases.CONFIG_A))
    spec.validate()
    assert spec.architecture == "Kufolorn" and [e.layer for e in spec.order] == [0, 1, 2, 3]
    assert all(l.block == "sandwich" and "norm1" not in l.parts and "norm2" not in l.parts for l in spec.layers)
    assert [l.parts["mixer"].kind for l in spec.layers] == ["gated_delta", "mixer_pair", "gated_delta", "mixer_pair"]
    assert "feed_forward" not in spec.layers[2].parts and "norm2b" not in spec.layers[2].parts
    names = expected_params_of_spec(spec)
    assert "head" not in names and names["embed"].shape == (211, 96)           # the head is the embedding table
    assert names["l0.mix.q.conv"].shape == (72, 4) and names["l0.mix.v"].shape == (96, 96) and names["l0.mix.norm"].shape == (16,)
    assert names["l1.mix.left.sink"].shape == (4,) and names["l1.mix.left.g"].shape == (4, 96) and names["l1.mix.left.k.b"].shape == (48,)
    assert names["l1.mix.right.g"].shape == (60, 96) and names["l1.mlp.router"].shape == (8, 96) and names["l1.mlp.correction"].shape == (8,)
    assert "l1.mlp.e5.down" in names and "l1.mlp.e6.down" not in names         # identity experts have no tensors
    assert "l2.norm2" not in names and names["l3.mlp.gate"].shape == (64, 96)


def test_what_the_entries_ask_of_the_cache():
    import torch
    from litinfer_amd.config import architecture_name, lookup
    from litinfer_amd.engine.model import Model
    from litinfer_amd.parts import PagedNeed, Runtime, StateNeed, needs_of
    arch = lookup(architecture_name(cases.CONFIG_A))
    model = Model(arch.model_spec(arch.config_from_dict(cases.CONFIG_A)), Runtime(torch.device("cpu"), torch.float32))
    needs, sources = model.cache_needs()
    assert sources == [None] * 4
    paged, states = needs_of(needs[0])
    assert paged is None and {s.name: s.shape for s in states} == {"delta": (6, 24, 16), "conv": (3, 96 + 2 * 72)}
    assert all(s.dtype is torch.float32 for s in states)
    paged, states = needs_of(needs[1])
    assert isinstance(paged, PagedNeed) and paged.window == 0 and [(t.name, t.shape) for t in paged.tensors] == [("k", (2, 24)), ("v", (2, 16))]
    assert [(s.name, s.shape, s.dtype) for s in states] == [("retention", (3, 12, 20), torch.float32)]
    # one tap: no tail of the convolution
    archb = lookup(architecture_name(cases.CONFIG_B))
    mb = Model(archb.model_spec(archb.config_from_dict(cases.CONFIG_B)), Runtime(torch.device("cpu"), torch.float32))
    assert [s.name for s in needs_of(mb.cache_needs()[0][1])[1]] == ["delta"]


def test_a_pair_of_mixers_refuses_factors_without_a_branch():
    import torch
    from litinfer_amd.config import PartSpec
    from litinfer_amd.parts import Runtime, build_part
    ret = lambda name: PartSpec("retention", "x.", {"hidden_size": 8, "num_heads": 1, "head_dim": 4, "decay": [0.5], "state_name": name})
    rt = Runtime(torch.device("cpu"), torch.float32)
    pair = build_part("mixer", PartSpec("mixer_pair", "", {"left": ret("a"), "right": ret("b"), "left_scale": 0.5}), rt)
    assert [s.name for s in pair.cache_need()] == ["a", "b"]
    with pytest.raises(NotImplementedError):
        pair.forward(None, object(), None, None)
    with pytest.raises(ValueError):                            # two states of one name
        build_part("mixer", PartSpec("mixer_pair", "", {"left": ret("a"), "right": ret("a")}), rt)
