"""Nusuvik without a GPU: pins of the plain implementation (tests/plain_nusuvik.py) against closed forms written
another way, the typed configuration and its errors, the model as data (order, injections, tensors), and what the
entries and the embedding ask of the cache."""
import copy
import math

import numpy as np
import pytest

import nusuvik_cases as cases
import plain_nusuvik as plain


# ------------------------------------------------------------------------------------- the plain implementation
def test_pair_rows_first_token_and_hash():
    assert plain.bigram_rows([7], 13, 5, 3) == [13]
    assert plain.bigram_rows([7, 2, 2], 13, 5, 3) == [13, (7 * 5 + 2 * 3) % 13, (2 * 5 + 2 * 3) % 13]
    # multipliers beyond 32 bits
    assert plain.bigram_rows([300, 299], 1021, 1000003, 77)[1] == (300 * 1000003 + 299 * 77) % 1021


def test_layer_norm_by_hand():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    w, b = np.array([1.0, 2.0, 1.0, 0.5]), np.array([0.0, 1.0, 0.0, -1.0])
    var = np.mean((x - 3.0) ** 2)
    assert np.allclose(plain.layer_norm(x, w, b, 0.1), (x - 3.0) / math.sqrt(var + 0.1) * w + b)
    assert abs(var - 3.5) < 1e-12


def test_gelu_values():
    assert plain.gelu_tanh(np.array(0.0)) == 0.0
    assert abs(plain.gelu_tanh(np.array(1.0)) - 0.8411919906082768) < 1e-12
    assert abs(plain.gelu_tanh(np.array(-3.0)) + 0.0036373920817729943) < 1e-12


def test_half_split_rotation_is_a_complex_multiplication():
    rng = np.random.default_rng(0)
    v = rng.normal(size=(5, 10))
    pos = np.array([0, 1, 7, 100, 3])
    out = plain.rotate_half(v, pos, 50.0, 8)
    z = (v[:, :4] + 1j * v[:, 4:8]) * np.exp(1j * pos[:, None] * 50.0 ** (-2.0 * np.arange(4) / 8))
    assert np.allclose(out[:, :4], z.real) and np.allclose(out[:, 4:8], z.imag) and np.array_equal(out[:, 8:], v[:, 8:])
    assert np.array_equal(out[0], v[0])


def test_scores_depend_on_the_distance_only():
    """The rotated parts' product at positions (p, j) equals that at (p + s, j + s)."""
    rng = np.random.default_rng(1)
    q, k = rng.normal(size=(1, 6)), rng.normal(size=(1, 6))
    a = plain.rotate_half(q, [9], 100.0, 6) @ plain.rotate_half(k, [4], 100.0, 6).T
    b = plain.rotate_half(q, [109], 100.0, 6) @ plain.rotate_half(k, [104], 100.0, 6).T
    assert np.allclose(a, b)


def test_latent_attention_against_the_absorbed_form():
    """Head h's score and output written the other way round: queries moved into the latent space, the values'
    expansion applied to the summed latents."""
    cfg = cases.CONFIG_A
    W = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 3).items()}
    m = cfg["layers"][0]["mixer"]
    rng = np.random.default_rng(2)
    T, H, dn, dr, dv, rank = 9, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = rng.normal(size=(T, cfg["width"]))
    eps = cfg["norm"]["eps"]
    ref = plain.latent_attention(h, W, "l0.mix.", m, eps)
    p = "l0.mix."
    cq = plain.rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(T, H, dn + dr)
    down = h @ W[p + "dkv"].T
    c = plain.rms(down[:, :rank], eps) * W[p + "dkv.norm"]
    kr = plain.rotate_half(down[:, rank:], np.arange(T), m["rot"]["base"], dr)
    gate = plain.sigmoid(h @ W[p + "g"].T)
    heads = np.zeros((T, H, dv))
    for hd in range(H):
        uk = W[p + "uk"][hd * dn:(hd + 1) * dn]                       # [dn, rank]
        uv = W[p + "uv"][hd * dv:(hd + 1) * dv]                       # [dv, rank]
        qr = plain.rotate_half(q[:, hd, dn:], np.arange(T), m["rot"]["base"], dr)
        qc = q[:, hd, :dn] @ uk                                       # into the latent space
        for i in range(T):
            s = (c[:i + 1] @ qc[i] + kr[:i + 1] @ qr[i]) * m["scale"]
            w = np.exp(s - s.max())
            heads[i, hd] = uv @ ((w / w.sum()) @ c[:i + 1]) * gate[i, hd]
    assert np.allclose(heads.reshape(T, -1) @ W[p + "o"].T, ref)


def test_routing_groups_correction_and_weights():
    W = {"router": np.eye(6), "correction": np.array([0.0, 0.0, 0.0, 0.0, 0.3, -0.6])}
    z = np.array([[2.0, -9.0, 1.0, 0.9, 0.5, 3.0]])
    s = plain.sigmoid(z[0])
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}
    # groups (0,1), (2,3), (4,5): choice sums s0+s1, s2+s3, s4+0.3+s5-0.6; the middle group and the last win
    picks, weights = plain.route(z, W, "", r)
    sums = [s[0] + s[1], s[2] + s[3], s[4] + 0.3 + s[5] - 0.6]
    assert sorted(range(3), key=lambda g: -sums[g])[:2] == [1, 2]
    assert picks[0] == [4, 2]                                          # choice 0.92, 0.73, 0.71, 0.35: expert 0 is not allowed
    assert np.allclose(weights[0], np.array([s[4], s[2]]) / (s[4] + s[2]))
    # without groups the largest choice values win wherever they are; the weights do not see the correction
    picks, weights = plain.route(z, W, "", {"experts": 6, "top": 2})
    assert picks[0] == [4, 0] and np.allclose(weights[0], np.array([s[4], s[0]]) / (s[0] + s[4]))
    # an expert outside the kept groups counts as minus infinity, not zero: negative choice values inside still win
    W2 = {"router": np.eye(4), "correction": np.array([-5.0, -5.0, -7.0, -7.0])}
    picks, _ = plain.route(np.zeros((1, 4)), W2, "", {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}})
    assert picks[0] == [0, 1]
    # equal values: the lower expert, the lower group
    picks, _ = plain.route(np.zeros((1, 4)), {"router": np.eye(4), "correction": np.zeros(4)}, "",
                           {"experts": 4, "top": 1, "groups": {"count": 2, "keep": 1}})
    assert picks[0] == [0]


def test_order_of_layer_runs():
    assert plain.layer_runs(cases.CONFIG_A) == [(0, True), (1, False)] * 3 + [(2, False)]
    assert plain.layer_runs(cases.CONFIG_B) == [(0, False), (1, False), (2, False)]
    assert plain.layer_runs(cases.CONFIG_C) == [(0, False), (1, False), (2, True), (2, True)]
    assert plain.layer_runs(cases.CONFIG_D) == [(0, False), (1, True), (2, False), (3, False)]


def test_a_prefix_gives_the_same_logits():
    cfg = cases.CONFIG_D
    W = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 5).items()}
    toks = [3, 9, 9, 60, 1, 0, 17]
    full = plain.forward(toks, W, cfg)
    assert np.allclose(plain.forward(toks[:4], W, cfg), full[:4])
    assert np.abs(full).max() <= cfg["logit_softcap"]


# --------------------------------------------------------------------------------------------- configuration
def test_configuration_and_model_as_data():
    from litinfer_amd.config import NusuvikConfig, nusuvik_model_spec
    c = NusuvikConfig.from_dict(cases.CONFIG_A)
    assert (c.vocab, c.width, c.eps, c.logit_softcap, c.loop, c.bigram) == (211, 96, 1e-5, 9.0, (0, 2, 3), (97, 5, 3))
    assert c.layers[2].mlp is None and c.layers[0].mlp.kind == "dense" and c.layers[1].mlp.kind == "moe"
    assert (c.layers[1].mlp.experts, c.layers[1].mlp.top, c.layers[1].mlp.groups, c.layers[1].mlp.keep_groups) == (6, 2, 3, 2)
    assert c.layers[1].mixer.rot.base == 500.0 and c.layers[1].mixer.q_rank == 36
    spec = nusuvik_model_spec(c)
    assert [(e.layer, e.inject) for e in spec.order] == [(0, (0, 0)), (1, None), (0, (0, 1)), (1, None), (0, (0, 2)), (1, None), (2, None)]
    assert spec.layers[0].block == "parallel" and "feed_forward" not in spec.layers[2].parts
    assert spec.embedding.kind == "pair_hash_embedding" and spec.final_norm.kind == "layernorm" and spec.head.args["softcap"] == 9.0
    assert spec.injections[0].kind == "loop_mix"
    b = NusuvikConfig.from_dict(cases.CONFIG_B)
    assert b.loop is None and b.logit_softcap == 0.0 and b.layers[0].mlp.groups == 1 and b.layers[0].mlp.keep_groups == 1
    assert not nusuvik_model_spec(b).injections
    d = nusuvik_model_spec(NusuvikConfig.from_dict(cases.CONFIG_D))
    assert d.embedding.kind == "token_embedding" and [(e.layer, e.inject) for e in d.order] == [(0, None), (1, (0, 0)), (2, None), (3, None)]


def test_tensors_of_the_model():
    from litinfer_amd.config import NusuvikConfig, nusuvik_model_spec
    from litinfer_amd.engine.model import expected_params_of_spec
    p = expected_params_of_spec(nusuvik_model_spec(NusuvikConfig.from_dict(cases.CONFIG_A)))
    assert {"embed", "bigram", "head", "final.norm", "final.norm.b", "loop.in", "l0.norm1", "l0.norm1.b", "l0.mix.dq", "l0.mix.dq.norm",
            "l0.mix.uq", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk", "l0.mix.uv", "l0.mix.g", "l0.mix.o", "l0.mlp.up", "l0.mlp.up.b",
            "l0.mlp.down", "l0.mlp.down.b", "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e5.gate", "l1.mlp.e0.up", "l1.mlp.e3.down"} <= set(p)
    assert not any(n.startswith("l2.mlp") for n in p) and "l1.mlp.e6.up" not in p and "l1.mlp.router.b" not in p
    assert p["bigram"].shape == (98, 96) and p["loop.in"].shape == (96, 192)
    assert p["l0.mix.dq"].shape == (56, 96) and p["l0.mix.uq"].shape == (3 * 32, 56) and p["l0.mix.dkv"].shape == (48, 96)
    assert p["l0.mix.uk"].shape == (72, 40) and p["l0.mix.uv"].shape == (48, 40) and p["l0.mix.g"].shape == (3, 96)
    assert p["l0.mix.o"].shape == (96, 48) and p["l1.mlp.e0.gate"].shape == (40, 96) and p["l1.mlp.correction"].shape == (6,)
    d = expected_params_of_spec(nusuvik_model_spec(NusuvikConfig.from_dict(cases.CONFIG_D)))
    assert "bigram" not in d and "loop.in" in d


@pytest.mark.parametrize("change,where", [
    (lambda c: c["layers"][0].update(type="attention"), "unknown mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "not supported"),
    (lambda c: c["layers"][0]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=6), "rot_dim"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "choices"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=4), "groups"),
    (lambda c: c["loop"].update(stop=4), "loop"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_bad_configurations_are_refused(change, where):
    from litinfer_amd.config import ConfigError, NusuvikConfig
    cfg = copy.deepcopy(cases.CONFIG_A)
    change(cfg)
    with pytest.raises(ConfigError, match=where):
        NusuvikConfig.from_dict(cfg)


def test_what_the_entries_and_the_embedding_ask_of_the_cache():
    import torch
    from litinfer_amd.cache import group_needs
    from litinfer_amd.config import NusuvikConfig, nusuvik_model_spec
    from litinfer_amd.engine.model import Model
    from litinfer_amd.parts import Runtime, needs_of
    model = Model(nusuvik_model_spec(NusuvikConfig.from_dict(cases.CONFIG_A)), Runtime(torch.device("cpu"), torch.float32))
    needs, sources = model.cache_needs()
    assert len(needs) == 8 and sources == [None] * 8                              # seven layer runs, and the embedding
    paged, states = needs_of(needs[0])
    assert not states and paged.window == 0 and [(t.name, t.shape) for t in paged.tensors] == [("latent", (1, 48))]
    assert needs_of(needs[1])[0].tensors[0].shape == (1, 36) and needs_of(needs[6])[0].tensors[0].shape == (1, 24)
    assert len(group_needs(needs, sources)) == 3                                  # every pass of the loop has pages of its own in its layer's group
    emb_paged, emb_states = needs_of(needs[7])
    assert emb_paged is None and [(s.name, s.shape, s.dtype) for s in emb_states] == [("last_token", (1,), torch.int32)]
    assert model.graph_safe
    plain_model = Model(nusuvik_model_spec(NusuvikConfig.from_dict(cases.CONFIG_D)), Runtime(torch.device("cpu"), torch.float32))
    assert len(plain_model.cache_needs()[0]) == 4                                 # no pair table: the embedding keeps nothing


def test_the_command_line_knows_the_architecture(tmp_path):
    """`random` writes a model folder for the configuration; its tensors are those the model expects."""
    import json
    from litinfer_amd.__main__ import main
    from litinfer_amd.weights.safetensors_io import SafetensorsFile
    (tmp_path / "c.json").write_text(json.dumps(cases.CONFIG_B))
    assert main(["random", "--config", str(tmp_path / "c.json"), "--seed", "3", "--out", str(tmp_path / "m")]) == 0
    names = set(SafetensorsFile(tmp_path / "m" / "model.safetensors").entries)
    assert {"embed", "bigram", "l0.mix.dq.norm", "l1.mlp.correction", "l1.mlp.e2.gate", "l2.mlp.down.b", "final.norm.b"} <= names
    assert "loop.in" not in names and "l0.mlp.e4.up" not in names
