"""Host-side parts of the Fopezen decoder: its configuration, the model as data, the weight loader's optional
and scalar tensors, the cache manager's kept first pages, and the plain implementation's own properties."""
import json
import os

import pytest
import torch

import plain_fopezen as P
from test_gpu_fopezen import F1, F2, F3, _layer, _write_model

from infinicore_infer_amd.cache import CacheManager, GroupSpec
from infinicore_infer_amd.config import ConfigError, config_from_dict
from infinicore_infer_amd.parts import Runtime, build_model


def test_config_to_model_spec():
    cfg = config_from_dict(F1)
    spec = cfg.model_spec()
    assert spec.architecture == "Fopezen" and spec.vocab_size == 211 and spec.hidden_size == 128
    kinds = [l.mixer.params["value_mix"] for l in spec.layers]
    assert kinds == ["keep", None, "mix", "mix"]                 # the first mixing layer keeps, a layer between does not mix
    m0, m1, m3 = (spec.layers[i].mixer.params for i in (0, 1, 3))
    assert (m0["qk_norm"], m0["sink"], m0["gate"], m0["out_bias"]) == ("row", False, False, False)
    assert (m1["qk_norm"], m1["sink"], m1["gate"], m1["out_bias"]) == ("head", True, True, True)
    assert (m0["window"], m0["keep_first"], m0["softmax_scale"]) == (40, 3, 0.2)
    assert m3["window"] is None
    assert spec.layers[1].feed_forward is None and spec.layers[1].feed_forward_norm is None
    assert spec.layers[0].feed_forward.params["intermediate_size"] == 192
    assert spec.embedding.params["sinusoid_base"] == 10000.0 and spec.head.params["tensor"] == "embed"
    assert config_from_dict(cfg.to_dict()).model_spec().layers[2].mixer.params == spec.layers[2].mixer.params
    assert config_from_dict(F1, max_tokens=300).max_positions == 300
    assert cfg.context_is_open and cfg.max_positions == 65536


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="attention_9"), "type"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=32), "agree"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_config_errors(change, what):
    cfg = json.loads(json.dumps(F1))
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert what in str(e.value)


def test_cache_needs_and_groups():
    model = build_model(config_from_dict(F1).model_spec(), Runtime(torch.float32, "cpu"))
    needs = model.cache_needs()
    assert [(n.n_kv_heads, n.plane_dims, n.window, n.keep_first) for n in needs] == [
        (2, (32, 64), 40, 3), (1, (64, 32), 24, 0), (2, (32, 64), 56, 9), (2, (64, 64), None, 0)]


def test_weights_load_with_scalars_and_optional_tensors(tmp_path):
    folder = str(tmp_path / "m")
    W = _write_model(folder, F1, 3)
    assert "l1.mix.vmix" not in W and W["l0.mix.vmix"].shape == ()
    model = build_model(config_from_dict(F1).model_spec(), Runtime(torch.float32, "cpu"))
    model.load_from_dir(folder)
    assert model.head.weight is model.embedding.table
    mixers = [l.mixer for l in model.layers]
    assert mixers[0].mix_lambda is None and float(mixers[2].mix_lambda) == float(W["l2.mix.vmix"])
    assert torch.equal(mixers[1].w_rows, torch.cat([W["l1.mix." + n] for n in "qkvg"]))
    assert torch.equal(mixers[0].b_rows, torch.cat([W["l0.mix." + n + ".b"] for n in "qkv"]))
    assert torch.allclose(model.layers[0].mixer_norm.weight, 1.0 + W["l0.norm1"])
    # a mixing scalar in a layer that does not mix is taken in, not refused
    from safetensors.torch import load_file, save_file
    sd = load_file(os.path.join(folder, "model.safetensors"))
    sd["l1.mix.vmix"] = torch.tensor(0.25, dtype=torch.bfloat16)
    save_file(sd, os.path.join(folder, "model.safetensors"))
    model.load_from_dir(folder)


def test_window_group_keeps_its_first_pages():
    page = 16
    grp = GroupSpec("window", 2, 32, window=40, slots=(0,), planes=2, plane_dims=(32, 64), keep_first=20)
    m = CacheManager([grp], [12], page, max_requests=2, max_positions=4096)
    m.admit("a")
    held = []
    for step in range(60):
        m.append("a", 7)
        m.trim("a")
        m.check_invariants()
        table = m.block_table("a", 0)
        n = m.length("a")
        # the first two pages (keys 0..19) stay; pages wholly before the window are given back; the window's are held
        assert table[0] >= 0 and (len(table) < 2 or table[1] >= 0)
        for j, p in enumerate(table):
            first, last = j * page, j * page + page - 1
            dead = last < n - 40 + 1 and first >= 32
            assert (p < 0) == dead, (n, j, table)
        held.append(sum(p >= 0 for p in table))
    assert max(held) <= 2 + (40 + 7 + page - 1) // page + 1      # bounded: kept pages + the window's, not the length
    m.admit("b")
    m.append("b", 50)
    assert set(m.block_table("b", 0)) & {p for p in m.block_table("a", 0) if p >= 0} == set()
    m.release("a")
    m.release("b")
    assert m.free_pages(0) == 12
    # keep_first 0: the old behaviour
    m2 = CacheManager([GroupSpec("window", 2, 32, window=40, slots=(0,))], [12], page, max_requests=1)
    m2.admit("a")
    m2.append("a", 100)
    m2.trim("a")
    assert m2.block_table("a", 0)[0] == -1


# ---- the plain implementation itself -----------------------------------------------------------------------------
def test_plain_mask_and_sink():
    vis = P.visible(12, 4, 2)
    assert vis[10].tolist() == [True, True, False, False, False, False, False, True, True, True, True, False]
    assert vis[3].tolist() == [True, True, True, True] + [False] * 8
    assert P.visible(5, None, 0).tolist() == torch.tril(torch.ones(5, 5, dtype=torch.bool)).tolist()
    s = torch.tensor([[0.3, -1.0, 2.0]])
    w = P.weights_of_scores(s, torch.ones(1, 3, dtype=torch.bool), sink=True)
    e = torch.exp(s)
    assert torch.allclose(w, e / (1 + e.sum()))
    assert torch.allclose(P.weights_of_scores(s, torch.ones(1, 3, dtype=torch.bool), sink=False).sum(), torch.tensor(1.0))


@pytest.mark.parametrize("cfg", [F1, F2])
def test_plain_prefix_property(cfg):
    """A position's logits do not depend on later tokens, and a key that leaves every window and is not kept stops mattering."""
    W = P.random_weights(cfg, 1)
    toks = torch.randint(0, cfg["vocab"], (90,), generator=torch.Generator().manual_seed(2)).tolist()
    full = P.forward(cfg, W, toks, torch.float64)
    assert torch.allclose(full[:50], P.forward(cfg, W, toks[:50], torch.float64), atol=1e-9)
    layers = []
    P.forward(cfg, W, toks[:9], torch.float64, layers)
    assert len(layers) == len(cfg["layers"]) and layers[0].shape == (9, cfg["width"])
