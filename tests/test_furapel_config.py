"""The Furapel design without a GPU: its configuration and the errors it names, the parts and cache groups a configuration
becomes (a layer that runs again is a layer of its own with the same tensors), and pins of the plain implementation
(tests/plain_furapel.py) on inputs with known answers."""
import copy
import json
import os

import numpy as np
import pytest
import torch

import furapel_cases as cases
import plain_furapel as plain


def test_configurations_round_trip_and_name_every_bad_key():
    from kvcm_amd.config.furapel_config import FurapelConfig
    from kvcm_amd.config.model_config import ConfigError
    for raw in cases.CONFIGS.values():
        cfg = FurapelConfig.from_dict(raw)
        assert FurapelConfig.from_dict(cfg.to_dict()) == cfg
        assert FurapelConfig.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    assert FurapelConfig.from_dict(cases.CONFIGS["W"]).logit_scale == 1.0 and FurapelConfig.from_dict(cases.CONFIGS["U"]).loop is None
    bad = copy.deepcopy(cases.CONFIGS["V"])
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    bad["layers"][0]["mixer"]["rot"]["dims"] = 7
    bad["layers"][1]["mixer"]["mask"] = {}
    bad["layers"][2]["type"] = "lstm"
    bad["layers"][3]["mlp"]["router"]["top"] = 9
    bad["loop"] = {"start": 2, "stop": 2, "times": 0}
    del bad["width"]
    with pytest.raises(ConfigError) as e:
        FurapelConfig.from_dict(bad)
    text = str(e.value)
    for piece in ("config.width", "kv_heads 3", "rot.dims 7", "layers[1].mixer.mask.size", "'lstm' is not supported", "top 9 exceeds",
                  "loop.times", "are not a stretch"):
        assert piece in text, (piece, text)
    # what a file may leave out: the embedding's factor, the logit scale, kv_heads (= heads), vdim (= dim), the rotation's
    # base, the latent attention's mask (then every earlier token is seen)
    lean = copy.deepcopy(cases.CONFIGS["U"])
    del lean["embedding"], lean["logit_scale"], lean["layers"][1]["mixer"]["kv_heads"], lean["layers"][1]["mixer"]["vdim"]
    del lean["layers"][1]["mixer"]["rot"]["base"], lean["layers"][2]["mixer"]["mask"], lean["layers"][2]["mixer"]["vdim"]
    cfg = FurapelConfig.from_dict(lean)
    a, l = cfg.layers[1].mixer, cfg.layers[2].mixer
    assert (cfg.embedding_scale, cfg.logit_scale, a.kv_heads, a.vdim, a.rot_base, l.window, l.vdim) == (1.0, 1.0, 4, 16, 10000.0, 0, 12)
    assert FurapelConfig.from_dict(cfg.to_dict()) == cfg
    dense = copy.deepcopy(cases.CONFIGS["U"])
    dense["layers"][1]["mlp"]["kind"] = "dense"
    with pytest.raises(ConfigError, match="mlp.kind 'dense' is not supported"):
        FurapelConfig.from_dict(dense)


def test_a_layer_that_runs_again_is_a_layer_of_its_own_with_the_same_tensors():
    from kvcm_amd.architectures.furapel import furapel_spec, layer_runs
    from kvcm_amd.config.furapel_config import FurapelConfig
    from kvcm_amd.parts.base import BuildContext, KVCacheNeed, StateNeed
    from kvcm_amd.parts.model import Model
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = FurapelConfig.from_dict(cases.CONFIGS["V"])
    assert [(i, leads) for i, _, leads in layer_runs(cfg)] == plain.layer_runs(cases.CONFIGS["V"])
    spec = furapel_spec(cfg)
    assert [l.name for l in spec.layers] == ["l0", "l1", "l2", "l1.pass1", "l2.pass1", "l3"] and spec.keep_embedding
    assert ["reentry" in l.parts for l in spec.layers] == [False, True, False, True, False, False]
    assert spec.layers[1].parts["mixer"].prefix == spec.layers[3].parts["mixer"].prefix == "l1.mix."
    model = Model(spec, BuildContext(torch.float32, torch.device("cpu"), spec.hidden_size, 16, None))
    assert model.capturable, model.not_capturable()
    # every pass has a place of its own: two latent layers of one shape share a group, the third has another window
    owners = {key: place for key, place in model._cache_of.items()}
    assert owners[("l1", "mixer")][0] == owners[("l1.pass1", "mixer")][0] and owners[("l1", "mixer")][1] != owners[("l1.pass1", "mixer")][1]
    needs = [g.need for g in model.groups]
    assert KVCacheNeed(2, 64, 0, value_dim=64) in needs and KVCacheNeed(1, 32, 20, value_dim=32) in needs and KVCacheNeed(1, 16, 33, value_dim=16) in needs
    assert StateNeed((2, 32, 16), torch.float32) in needs and StateNeed((2, 32), torch.float32) in needs and StateNeed((2,), torch.float32) in needs
    assert len(next(g for g in model.groups if g.need == StateNeed((2, 32, 16), torch.float32)).layers) == 2
    names = expected_tensors("Furapel", cfg)
    assert names["loop.in"] == ((64, 128), "matrix") and names["l0.norm1.alpha"] == ((), "vector") and "l1.pass1.norm1" not in names
    assert names["l2.mlp.e5.down"] == ((64, 16), "matrix") and names["l1.mix.dkv.norm"] == ((32,), "vector")
    # a layer without a feed-forward declares no second norm, and tolerates one in the checkpoint
    u = Model(furapel_spec(FurapelConfig.from_dict(cases.CONFIGS["U"])), BuildContext(torch.float32, torch.device("cpu"), 48, 16, None))
    first = u.layer_parts[0]
    assert "ffn" not in first and "norm_ffn" not in first and "l0.norm2.alpha" in first["norm_mixer"].ignorable_tensors()
    # a window group hands pages back, the others keep them
    from kvcm_amd.engine.runner import plan_groups
    kinds = {(g.kind, g.window) for g in plan_groups(model, 10, 2)}
    assert ("window", 20) in kinds and ("window", 33) in kinds and ("full", 0) in kinds and ("state", 0) in kinds


def test_random_model_folders_load_by_name(tmp_path):
    from kvcm_amd.config.furapel_config import FurapelConfig
    from kvcm_amd.config.model_config import read_config_json
    from kvcm_amd.weights.random_init import write_model_dir
    cfg = FurapelConfig.from_dict(cases.CONFIGS["W"])
    d = write_model_dir(str(tmp_path / "m"), "Furapel", cfg, seed=4, dtype=torch.bfloat16, std=0.1, norm_jitter=0.1, device="cpu")
    name, raw = read_config_json(d)
    assert name == "Furapel" and FurapelConfig.from_dict(raw) == cfg
    t = plain.read_safetensors(os.path.join(d, "model.safetensors"))
    assert t["l0.norm1.alpha"].shape == () and t["loop.in"].shape == (32, 64)
    logits = plain.forward(cases.CONFIGS["W"], t, [3, 1, 4, 1, 5, 9, 2, 6])
    assert logits.shape == (8, 64) and np.isfinite(logits).all()


# --------------------------------------------------------------- the plain implementation on inputs with known answers
def test_plain_frequencies_and_rotation():
    f, factor = plain.yarn_frequencies(8, 100.0)
    np.testing.assert_allclose(f, [1.0, 100 ** -0.25, 0.1, 100 ** -0.75])
    assert factor == 1.0
    # rescaled: pairs that turn often keep their frequency, pairs that turn seldom are slowed by the factor, a ramp between
    sc = {"factor": 4.0, "original": 2 * np.pi * 100, "fast": 10.0, "slow": 1.0}
    f4, factor = plain.yarn_frequencies(8, 100.0, sc)      # pair(t) = 8 ln(100 / t) / (2 ln 100): pair(10) = 2, pair(1) = 4
    np.testing.assert_allclose(f4, [f[0], f[1], f[2], 0.5 * f[3] / 4 + 0.5 * f[3]])
    assert abs(factor - (0.1 * np.log(4.0) + 1.0)) < 1e-15
    # limits: the ramp's end is cut at the last entry, a degenerate ramp is a step
    f5, _ = plain.yarn_frequencies(4, 100.0, {"factor": 2.0, "original": 2 * np.pi * 100, "fast": 1e9, "slow": 1e-9})
    np.testing.assert_allclose(f5, [1.0, 0.1 / 2 * (1 / 3) + 0.1 * (2 / 3)])
    x = np.arange(12, dtype=np.float64).reshape(1, 1, 12)
    y = plain.rotate_half(x, [3], 4, np.array([np.pi / 6, 0.0]), 2.0)      # entry 0 with entry 2 by 90 degrees, entry 1 with 3 by none
    np.testing.assert_allclose(y[0, 0], [-4.0, 2.0, 0.0, 6.0, 4, 5, 6, 7, 8, 9, 10, 11], atol=1e-12)


def test_plain_attention_sees_what_it_should():
    m = plain.visible(6, 0)
    assert m.sum() == 21 and m[3, 3] and not m[2, 3]
    w = plain.visible(6, 2)
    assert [list(np.nonzero(r)[0]) for r in w] == [[0], [0, 1], [1, 2], [2, 3], [3, 4], [4, 5]]
    assert (plain.visible(4, 1) == np.eye(4, dtype=bool)).all()
    # query head h reads key head h // (H / G); one key far ahead of the others takes all the weight
    q = np.zeros((3, 4, 2)); k = np.zeros((3, 2, 2)); v = np.arange(12, dtype=np.float64).reshape(3, 2, 2)
    q[2, :, 0] = 50.0
    k[1, 1, 0] = 1.0
    out = plain.attend(q, k, v, 1.0)
    np.testing.assert_allclose(out[2, 2], v[1, 1], atol=1e-9)
    np.testing.assert_allclose(out[2, 0], v[:, 0].mean(0), atol=1e-9)


def test_plain_matrix_memory_reduces_to_known_sums():
    # gates that neither damp nor grow (log keep 0, log in 0): m stays 0, S is the plain sum of k v^T, n the sum of k
    T, d, dv = 5, 3, 2
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(T, d)), rng.normal(size=(T, d)), rng.normal(size=(T, dv))
    o, (S, n, m) = plain.matrix_memory(q, k, v, np.zeros(T), np.zeros(T))
    np.testing.assert_allclose(S, k.T @ v)
    np.testing.assert_allclose(n, k.sum(0))
    assert m == 0.0
    np.testing.assert_allclose(o[-1], (k.T @ v).T @ q[-1] / (max(abs(k.sum(0) @ q[-1]), 1.0) + 1e-6))
    # the running maximum starts at 0: a first input gate far below leaves exp(li) of the token, not all of it
    o, (S, n, m) = plain.matrix_memory(q[:1], k[:1], v[:1], np.array([-5.0]), np.array([0.0]))
    assert m == 0.0
    np.testing.assert_allclose(S, np.exp(-5.0) * np.outer(k[0], v[0]))
    # a state handed over continues the same walk
    o_all, _ = plain.matrix_memory(q, k, v, np.linspace(-1, 2, T), np.linspace(-0.5, 0, T))
    o_a, st = plain.matrix_memory(q[:2], k[:2], v[:2], np.linspace(-1, 2, T)[:2], np.linspace(-0.5, 0, T)[:2])
    o_b, _ = plain.matrix_memory(q[2:], k[2:], v[2:], np.linspace(-1, 2, T)[2:], np.linspace(-0.5, 0, T)[2:], st)
    np.testing.assert_allclose(np.concatenate([o_a, o_b]), o_all)
    assert abs(plain.soft_cap(1e9, 7.0) - 7.0) < 1e-12 and abs(plain.log_sigmoid(0.0) + np.log(2.0)) < 1e-15


def test_plain_routing_and_layer_order():
    h = np.array([[1.0, 0.0], [0.0, 2.0]])
    w = np.array([[3.0, 0.0], [1.0, 1.0], [0.0, 2.0]])
    chosen, weight = plain.route(h, w, 2)
    assert chosen.tolist() == [[0, 1], [2, 1]]
    s = np.exp([3.0, 1.0, 0.0]) / np.exp([3.0, 1.0, 0.0]).sum()
    np.testing.assert_allclose(weight[0], s[:2])      # the scores as they are: they do not add up to one
    assert abs(plain.expert(np.array([1.0, -1.0]), np.array([[2.0, 0.0], [0.0, 3.0]]), np.array([[1.0, 1.0]]))[0] - 4.0) < 1e-12
    assert plain.layer_runs({"layers": [0] * 4, "loop": {"start": 1, "stop": 3, "times": 2}}) == \
        [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert plain.layer_runs({"layers": [0] * 2}) == [(0, False), (1, False)]
    np.testing.assert_allclose(plain.dynamic_tanh(np.array([0.0, 1e9]), 0.5, np.array([2.0, 2.0]), np.array([1.0, -1.0])), [1.0, 1.0])
