"""Without a GPU: the Kasuvik configuration reader, the description of its layers as parts, what the cache
planner makes of them, the loader's sizes that only the checkpoint gives, and pins of the plain implementation
on inputs whose answer is known."""
import json
import os

import numpy as np
import pytest
import torch

import kasuvik_cases as cases
import plain_kasuvik as plain


def _model(raw):
    from kvcm_amd.config.kasuvik_config import KasuvikConfig
    from kvcm_amd.parts.base import BuildContext
    from kvcm_amd.parts.model import Model
    from kvcm_amd.registry import ARCHITECTURES
    import kvcm_amd.architectures  # noqa: F401
    cfg = KasuvikConfig.from_dict(raw)
    spec = ARCHITECTURES.get("Kasuvik").build_spec(cfg)
    return cfg, Model(spec, BuildContext(torch.float32, torch.device("cpu"), spec.hidden_size, 16, None))


def test_config_round_trip_and_registry(tmp_path):
    from kvcm_amd.config.kasuvik_config import KasuvikConfig
    from kvcm_amd.engine.build import read_model_config
    for raw in cases.CONFIGS.values():
        cfg = KasuvikConfig.from_dict(raw)
        assert KasuvikConfig.from_dict(cfg.to_dict()) == cfg
        assert cfg.to_dict()["layers"][0]["type"] == raw["layers"][0]["type"]
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cases.CONFIGS["P"]))       # names its class as "architecture": a string
    arch, cfg = read_model_config(str(d))
    assert arch.name == "Kasuvik" and cfg.layers[1].left.pool == 5 and cfg.layers[1].ff == 0 and cfg.layers[0].delta.rank == 8


def test_config_errors_name_the_key():
    from kvcm_amd.config.kasuvik_config import KasuvikConfig
    from kvcm_amd.config.model_config import ConfigError
    raw = json.loads(json.dumps(cases.CONFIGS["P"]))
    raw["layers"][1]["mixer"]["left"]["kv_heads"] = 3
    raw["layers"][2]["mixer"]["left"]["rot"]["dims"] = 7
    raw["layers"][0]["type"] = "something"
    raw["layers"][2]["mlp"]["kind"] = "routed"
    del raw["norm"]
    with pytest.raises(ConfigError) as e:
        KasuvikConfig.from_dict(raw)
    for piece in ("layers[1].mixer.left: heads 4 is not a multiple of kv_heads 3", "layers[2].mixer.left.rot.dims 7", "layers[0].type",
                  "layers[2].mlp.kind", "norm.eps"):
        assert piece in str(e.value)


def test_layers_become_parts_and_cache_groups():
    from kvcm_amd.parts.base import KVCacheNeed, StateNeed
    cfg, model = _model(cases.CONFIGS["P"])
    assert [type(b).__name__ for b in model.blocks] == ["SandwichResidual"] * 3
    assert "ffn" in model.layer_parts[0] and "ffn" not in model.layer_parts[1]
    needs = {key: plan.need for plan in model.groups for key in plan.layers}
    assert needs[("l0", "mixer#delta")] == StateNeed((3, 16, 16), torch.float32)
    assert needs[("l1", "mixer.left")] == KVCacheNeed(2, 16, 20, value_dim=24, pool=5)
    assert needs[("l1", "mixer.left#conv")] == StateNeed((1, 4 * 16 + 2 * 16 + 2 * 24), torch.float32)
    assert needs[("l1", "mixer.right#scan")] == StateNeed((40, 6), torch.float32)
    assert needs[("l2", "mixer.right#conv")] == StateNeed((1, 56), torch.float32)
    # one tap: no state for the convolution at all
    _, q = _model(cases.CONFIGS["Q"])
    assert not any(key == ("l0", "mixer.left#conv") or key == ("l0", "mixer.right#conv") for plan in q.groups for key in plan.layers)
    # pooled entries live in their pages: such a group keeps every page, whatever the window
    from kvcm_amd.engine.runner import plan_groups
    kinds = [g.kind for g in plan_groups(model, 8, 4)]
    assert kinds.count("full") == 2 and "window" not in kinds
    assert model.capturable


def test_pages_hold_values_of_their_own_size_and_pooled_entries():
    from kvcm_amd.cache.storage import KVStorage, bytes_per_block
    from kvcm_amd.parts.base import KVCacheNeed
    need = KVCacheNeed(2, 16, 20, value_dim=24, pool=5)
    st = KVStorage(0, need, 3, 7, 16, torch.bfloat16, "cpu")
    assert tuple(st.k(1).shape) == (7, 2, 16, 16) and tuple(st.v(1).shape) == (7, 2, 24, 16)
    assert tuple(st.pooled_k(2).shape) == (7, 2, 4, 16) and tuple(st.pooled_v(2).shape) == (7, 2, 4, 24) and st.pooled_k(0).dtype == torch.float32
    assert st.bytes_per_block == bytes_per_block(need, 3, 16, torch.bfloat16) == 3 * 2 * (16 * 40 * 2 + 4 * 40 * 4)
    assert st.total_bytes == 7 * st.bytes_per_block
    plainer = KVStorage(0, KVCacheNeed(2, 16), 3, 7, 16, torch.bfloat16, "cpu")
    assert tuple(plainer.v(0).shape) == (7, 2, 16, 16) and plainer.bytes_per_block == 3 * 2 * 16 * 32 * 2


def test_a_size_that_only_the_checkpoint_gives():
    from kvcm_amd.weights.loader import DictSource, WeightsError, check_against, load_weights
    raw = json.loads(json.dumps(cases.CONFIGS["Q"]))
    cfg, tensors = cases.tensors_for(raw, seed=1)
    del raw["layers"][2]["mixer"]["rank"]                     # config.json does not carry the rank
    _, model = _model(raw)
    load_weights(model, DictSource(tensors), torch.float32, "cpu")
    mixer = model.layer_parts[2]["mixer"]
    assert mixer.rank == 5 and tuple(mixer.w["w_proj"].shape) == (5 * 24 + 5, 32)
    bad = dict(tensors)
    bad["l2.mix.w2"] = torch.zeros(24, 6)
    _, model = _model(raw)
    with pytest.raises(ValueError, match="do not agree on their rank"):
        load_weights(model, DictSource(bad), torch.float32, "cpu")
    bad = dict(tensors)
    bad["l2.mix.w2"] = torch.zeros(23, 5)
    with pytest.raises(WeightsError, match="l2.mix.w2"):
        check_against(model, DictSource(bad))


def test_random_model_folder_loads_by_name(tmp_path):
    from kvcm_amd.weights.loader import FolderSource, check_against
    from kvcm_amd.weights.random_init import write_model_dir
    cfg, model = _model(cases.CONFIGS["R"])
    d = write_model_dir(str(tmp_path / "r"), "Kasuvik", cfg, seed=3, dtype=torch.bfloat16, std=0.05, device="cpu")
    src = FolderSource(d)
    check_against(model, src)
    assert "l1.mix.w1" in src.names() and src.shape("l1.mix.w1") == (16, 64)
    src.close()


# ------------------------------------------------------------------ pins of the plain implementation
def test_plain_convolution_and_rotation():
    u = np.arange(12.0).reshape(6, 2)
    w = np.array([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]])
    y = plain.short_conv(u, w)
    assert y[0, 0] == 100.0 * u[0, 0] and y[2, 0] == u[0, 0] + 10 * u[1, 0] + 100 * u[2, 0] and (y[:, 1] == u[:, 1]).all()
    x = np.zeros((1, 1, 6))
    x[0, 0] = [1.0, 0.0, 0.0, 1.0, 5.0, 6.0]
    r = plain.rotate_interleaved(x, [3], 4, 100.0)
    np.testing.assert_allclose(r[0, 0], [np.cos(3.0), np.sin(3.0), -np.sin(0.3), np.cos(0.3), 5.0, 6.0], atol=1e-12)


def test_plain_attention_sees_window_and_whole_blocks_only():
    T, W, P = 30, 6, 4
    q = np.zeros((T, 1, 2))
    k = np.zeros((T, 1, 2))
    v = np.eye(T)[:, None, :]                       # value j is the unit vector e_j: the output holds the weights
    out = plain.window_pool_attention(q, k, v, 1.0, np.ones(1), W, P)
    i = 21                                          # window 16..21; blocks that end at or before 15: 0..3 (tokens 0..15)
    w = out[i, 0]
    np.testing.assert_allclose(w[16:22], 1.0 / 10.0)
    np.testing.assert_allclose(w[:16], 1.0 / 10.0 / 4.0)
    assert (w[22:] == 0).all()
    i = 22                                          # window 17..22; token 16's block (16..19) is not whole before the window: unseen
    w = out[i, 0]
    assert w[16] == 0 and w[17] > 0 and w[15] > 0


def test_plain_recurrences_reduce_to_known_sums():
    rng = np.random.default_rng(0)
    T, H, d = 7, 2, 3
    r, k, v = (rng.normal(size=(T, H, d)) for _ in range(3))
    one, zero = np.ones((T, H, d)), np.zeros((T, H, d))
    o = plain.delta_rule(r, k, v, one, zero)        # no decay, nothing removed: o_t = sum_{s<=t} (r_t . k_s) v_s
    want = np.einsum("thd,shd,she->the", r, k, v * 1.0) * 0
    for t in range(T):
        want[t] = sum(np.einsum("hd,hd->h", r[t], k[s])[:, None] * v[s] for s in range(t + 1))
    np.testing.assert_allclose(o, want, atol=1e-12)
    o = plain.delta_rule(r, k, v, one, one)         # everything along the key removed before it is written again
    S = np.zeros((d, d))
    u = k[0, 0] / np.sqrt(k[0, 0] @ k[0, 0] + 1e-6)
    S = np.outer(k[0, 0], v[0, 0])
    u = k[1, 0] / np.sqrt(k[1, 0] @ k[1, 0] + 1e-6)
    S = S - np.outer(u, u @ S) + np.outer(k[1, 0], v[1, 0])
    np.testing.assert_allclose(o[1, 0], S.T @ r[1, 0], atol=1e-12)
    x, dt = rng.normal(size=(T, 4)), np.full((T, 4), 0.5)
    A, B, C = -np.ones((4, 1)), np.ones((T, 1)), np.ones((T, 1))
    y = plain.selective_scan(x, dt, A, B, C, np.zeros(4))
    want = np.zeros((T, 4))
    for t in range(T):
        want[t] = sum(np.exp(-0.5 * (t - s)) * 0.5 * x[s] for s in range(t + 1))
    np.testing.assert_allclose(y, want, atol=1e-12)
