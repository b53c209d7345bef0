"""Host-side parts of the Mezinex decoder: its configuration and its errors, the run order of looped layers, the model
as data, what its parts ask of the cache manager, weights loaded into fused layouts, and the plain implementation's own
properties (a sequence's results do not depend on what follows; the recurrences agree with their closed forms)."""
import json
import math

import pytest
import torch

import plain_mezinex as P
from test_gpu_mezinex import Z1, Z2, Z3, Z4, _write_model

from infinicore_infer_amd.config import ConfigError, config_from_dict
from infinicore_infer_amd.parts import Runtime, build_model


def test_config_to_model_spec():
    cfg = config_from_dict(Z1)
    spec = cfg.model_spec()
    assert spec.architecture == "Mezinex" and spec.vocab_size == 211 and spec.hidden_size == 96 and spec.residual_streams == 3
    assert cfg.run_order() == [0, 1, 0, 1, 0, 1, 2, 3] == P.run_order(Z1)
    assert [(e.layer, e.cache) for e in spec.schedule] == [(0, 0), (1, 1), (0, 2), (1, 3), (0, 4), (1, 5), (2, 6), (3, 7)]
    assert [l.mixer.kind for l in spec.layers] == ["mamba2", "latent_attention", "rglru", "latent_attention"]
    assert all(l.block.kind == "hyper_connections" and l.block.params["streams"] == 3 for l in spec.layers)
    m = spec.layers[1].mixer.params
    assert (m["num_heads"], m["head_dim"], m["rot_dim"], m["rot_dims"], m["value_dim"], m["q_rank"], m["kv_rank"]) == (3, 24, 16, 8, 40, 48, 40)
    assert (m["softmax_scale"], m["rot_base"], m["norm_eps"]) == (0.2, 10000.0, 1e-5)
    assert spec.layers[1].feed_forward is None and spec.layers[0].feed_forward.params["gate_name"] == "gate"
    assert spec.layers[2].mixer.params["decay_scale"] == 8.0
    e = spec.embedding.params
    assert (e["pair_tensor"], e["buckets"], e["mul_prev"], e["mul_cur"], e["streams"]) == ("bigram", 257, 31, 7, 3)
    assert spec.head.params["logit_scale"] == 0.7 and spec.head.params["tensor"] == "head"
    assert config_from_dict(cfg.to_dict()).model_spec().layers[3].mixer.params == spec.layers[3].mixer.params
    assert config_from_dict(Z1, max_tokens=300).max_positions == 300 and cfg.context_is_open
    # without streams, pair table and loop: the plain pre-norm block, the plain gather, every layer once
    plain = config_from_dict(Z2).model_spec()
    assert plain.residual_streams == 1 and all(l.block.kind == "prenorm_residual" for l in plain.layers)
    assert plain.embedding.params["pair_tensor"] is None and [e.layer for e in plain.schedule] == [0, 1, 2]
    assert config_from_dict(Z3).run_order() == [0, 1] and config_from_dict(Z4).run_order() == [0, 0, 1]


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="attention"), "type"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"]["rot"].pop("base"), "rot.base"),
    (lambda c: c["layers"][2]["mixer"].pop("blocks"), "blocks"),
    (lambda c: c["layers"][0]["mixer"].pop("norm_groups"), "norm_groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c.update(streams=9), "streams"),
    (lambda c: c["loop"].update(stop=7), "loop"),
    (lambda c: c["embedding"]["bigram"].pop("mul_cur"), "mul_cur"),
])
def test_config_errors(change, what):
    cfg = json.loads(json.dumps(Z1))
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert what in str(e.value)


def test_cache_needs_of_the_mixers_and_the_embedding():
    model = build_model(config_from_dict(Z1).model_spec(), Runtime(torch.float32, "cpu"))
    needs = model.cache_needs()
    assert [n.kind for n in needs] == ["state", "kv", "state", "kv", "state", "kv", "state", "kv"]
    ssm, latent, rglru = needs[0], needs[1], needs[6]
    assert ssm.state_shape == (4 * 24 * 16 + 3 * (64 + 2 * 4 * 24),) and ssm.state_dtype == torch.float32
    assert (latent.planes, latent.n_kv_heads, latent.head_dim, latent.window) == (1, 1, 40 + 16, None)
    assert rglru.state_shape == (64 * 2,)
    emb = model.embedding_cache_need()
    assert emb.kind == "state" and emb.state_shape == (1,) and emb.state_dtype == torch.int32
    assert build_model(config_from_dict(Z2).model_spec(), Runtime(torch.float32, "cpu")).embedding_cache_need().kind == "none"


def test_weights_load_into_fused_layouts(tmp_path):
    W = _write_model(str(tmp_path), Z1, seed=3)
    for dtype in (torch.float32, torch.bfloat16):
        model = build_model(config_from_dict(Z1).model_spec(), Runtime(dtype, "cpu"))
        model.load_from_dir(str(tmp_path))
        ssm, latent, rglru = (model.layers[i].mixer for i in (0, 1, 2))
        f = lambda name: W[name].to(torch.float32)
        assert torch.equal(latent.w_down.float(), torch.cat([f("l1.mix.dq"), f("l1.mix.dkv"), f("l1.mix.g")]))
        assert torch.equal(latent.w_uk_t.float(), f("l1.mix.uk").view(3, 24, 40).transpose(1, 2))
        assert torch.equal(latent.w_uv.float(), f("l1.mix.uv").view(3, 40, 40))
        assert torch.equal(rglru.w_yx.float(), torch.cat([f("l2.mix.y"), f("l2.mix.x")]))
        assert torch.equal(rglru.w_gate.float(), torch.cat([f("l2.mix.ra"), f("l2.mix.ri")], dim=1))
        assert rglru.b_gate.dtype == torch.float32 and torch.equal(rglru.b_gate.view(4, 32), torch.cat([f("l2.mix.ra.b"), f("l2.mix.ri.b")], dim=1))
        assert torch.allclose(rglru.decay.double(), -8 * P.softplus(W["l2.mix.lam"]), atol=1e-6)
        assert torch.allclose(ssm.neg_a.double(), -torch.exp(W["l0.mix.A_log"]), atol=1e-6)
        hc = model.layers[0].hc[2]
        assert all(t.dtype == torch.float32 for t in hc) and torch.equal(hc[2], f("l0.hc2.mix"))
        assert model.embedding.pair_table.shape == (258, 96)


def test_the_plain_implementation_is_causal_and_its_pair_rows_hash_the_neighbours():
    W = P.random_weights(Z1, 1)
    toks = list(range(5, 45))
    full = P.forward(Z1, W, toks)
    assert torch.allclose(P.forward(Z1, W, toks[:17]), full[:17], atol=1e-9)          # what follows changes nothing
    other = P.forward(Z1, W, toks[:16] + [99] + toks[17:])
    assert torch.allclose(other[:16], full[:16], atol=1e-9) and not torch.allclose(other[16:], full[16:], atol=1e-3)
    rows = P.bigram_rows([3, 4, 5], 257, 31, 7)
    assert rows == [257, (3 * 31 + 4 * 7) % 257, (4 * 31 + 5 * 7) % 257]


def test_the_plain_recurrences_against_their_closed_forms():
    g = torch.Generator().manual_seed(0)
    # a convolution is a sum over shifted copies
    x, w, b = torch.randn(9, 3, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64), torch.randn(3, dtype=torch.float64, generator=g)
    pad = torch.cat([torch.zeros(3, 3, dtype=torch.float64), x])
    want = b + sum(w[:, k] * pad[k:k + 9] for k in range(4))
    assert torch.allclose(P.causal_conv(x, w, b), want)
    # rotation keeps lengths, turns a pair by position * frequency, and leaves what lies beyond ``dims``
    v = torch.randn(6, 2, 10, generator=g, dtype=torch.float64)
    r = P.rotate_pairs(v, torch.arange(6), 100.0, 6)
    assert torch.allclose(r[..., :6].norm(dim=-1), v[..., :6].norm(dim=-1)) and torch.equal(r[..., 6:], v[..., 6:])
    ang = 5 * 100.0 ** (-2.0 / 6)
    assert torch.allclose(r[5, 0, 2], v[5, 0, 2] * math.cos(ang) - v[5, 0, 3] * math.sin(ang))
    # streams: with an identity mix and a read of all ones over equal streams the block is the plain residual sum, S times over
    xs = torch.stack([torch.randn(4, 5, generator=g, dtype=torch.float64)] * 3)
    y = torch.randn(4, 5, generator=g, dtype=torch.float64)
    new = P.hyper_write(xs, y, torch.eye(3, dtype=torch.float64), torch.ones(3, dtype=torch.float64))
    assert torch.allclose(P.hyper_read(new, torch.ones(3, dtype=torch.float64)), 3 * (xs[0] + y))
