"""Kamivik without a GPU: its configuration and registry entry, the tensors it declares, what its layers ask of the
cache, the rotation's tables, and the plain model's own mechanisms."""
import copy
import math

import pytest
import torch

import plain_kamivik as P
from kamivik_cases import CONFIGS, layer, config, A1, A2
from synaptix_amd.config import KamivikConfig, ConfigError, resolve_architecture
from synaptix_amd.parts import KvNeed, RotaryInterleaved


def test_configuration_round_trip_and_registry():
    for name, d in CONFIGS.items():
        arch = resolve_architecture(d)
        assert arch.name == "Kamivik"
        cfg = arch.config_cls.from_dict(copy.deepcopy(d))
        assert KamivikConfig.from_dict(cfg.to_dict()) == cfg
        assert cfg.to_dict() == d
        assert len(cfg.layers) == len(d["layers"]) and cfg.vocab_size == d["vocab"]
    cfg = KamivikConfig.from_dict(CONFIGS["P"])
    assert cfg.layers[0].mixer.window == 20 and cfg.layers[1].mixer.window is None and cfg.layers[1].mlp is None
    assert cfg.layers[0].mixer.rot_dims == 4 and cfg.layers[0].mlp.top == 2 and cfg.residual_mult == 0.5
    d = copy.deepcopy(CONFIGS["S"])
    d.pop("residual_mult")
    d["layers"][0]["mixer"].pop("scale")
    cfg = KamivikConfig.from_dict(d)
    assert cfg.residual_mult == 1.0 and cfg.layers[0].mixer.scale == pytest.approx(12 ** -0.5)


@pytest.mark.parametrize("change,match", [
    (lambda d: d["layers"][0].__setitem__("type", "attention"), "layer type"),
    (lambda d: d["layers"][0]["mixer"].pop("mask"), "mask"),
    (lambda d: d["layers"][0]["mixer"]["rot"].__setitem__("dims", 3), "even"),
    (lambda d: d["layers"][0]["mixer"]["rot"].__setitem__("dims", 10), "rot_dim"),
    (lambda d: d["layers"][0]["mlp"].__setitem__("kind", "dense"), "moe"),
    (lambda d: d["layers"][0]["mlp"]["router"].__setitem__("top", 7), "top"),
    (lambda d: d["layers"][0]["mixer"].__setitem__("kv_rank", 0), "kv_rank"),
    (lambda d: d.__setitem__("width", 0), "width"),
    (lambda d: d.__setitem__("layers", []), "layers"),
    (lambda d: d["norm"].__setitem__("eps", "tiny"), "eps"),
])
def test_configuration_names_what_is_wrong(change, match):
    d = copy.deepcopy(CONFIGS["P"])
    change(d)
    with pytest.raises(ConfigError, match=match):
        KamivikConfig.from_dict(d)


def test_declared_tensors_and_cache_needs_of_unlike_layers():
    arch = resolve_architecture(CONFIGS["P"])
    model = arch.build(arch.config_cls.from_dict(CONFIGS["P"]))
    specs = model.tensor_specs()
    assert tuple(specs["l0.mix.q"].shape) == (4 * 24, 64) and tuple(specs["l0.mix.dkv"].shape) == (40, 64)
    assert tuple(specs["l0.mix.uk"].shape) == (64, 32) and tuple(specs["l0.mix.uv"].shape) == (96, 32)
    assert tuple(specs["l0.mix.g"].shape) == (96, 64)                 # the windowed type gates every value
    assert tuple(specs["l1.mix.g"].shape) == (2, 64)                  # the other type gates a head
    assert tuple(specs["l0.mlp.e5.up"].shape) == (48, 64) and tuple(specs["l0.mlp.router.b"].shape) == (6,)
    assert "l1.ls1" in specs and "l1.ls2" not in specs and not any(n.startswith("l1.mlp") for n in specs)
    assert tuple(specs["head"].shape) == (300, 64) and "final.norm" in specs
    # the cache holds one row a token: the latent and the rotated key part, and the latent once more as the value
    assert model.cache_needs() == [KvNeed(1, 40, 20, v_dim=32), KvNeed(1, 64, None, v_dim=48), KvNeed(1, 28, None, v_dim=24)]
    assert model.capturable()


def test_rotation_tables():
    rot = RotaryInterleaved(500.0, 6, 50)
    cos, sin = rot.tables("cpu")
    assert cos.shape == (50, 3) and cos.dtype == torch.float32
    for p in (0, 7, 49):
        for i in range(3):
            a = p * 500.0 ** (-2 * i / 6)
            assert abs(float(cos[p, i]) - math.cos(a)) < 1e-6 and abs(float(sin[p, i]) - math.sin(a)) < 1e-6
    assert RotaryInterleaved(1.0, 0, 4).tables("cpu") == (None, None)
    with pytest.raises(ValueError):
        RotaryInterleaved(10.0, 3, 4)


def test_the_plain_models_own_mechanisms():
    assert P.visible(5, None).tolist() == torch.tril(torch.ones(5, 5)).bool().tolist()
    seen = P.visible(6, 2)
    assert seen[4].tolist() == [False, False, False, True, True, False] and seen[0].tolist() == [True] + [False] * 5
    # a turn keeps lengths, turns by the position, and is the identity at position 0 and behind `dims`
    x = torch.randn(4, 3, 8, dtype=P.F64)
    y = P.turn_pairs(x, torch.arange(4), 100.0, 4)
    assert torch.allclose(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    assert torch.allclose(y[..., :4].pow(2).sum(-1), x[..., :4].pow(2).sum(-1))
    assert torch.allclose(y[2, 1, 0], x[2, 1, 0] * math.cos(2.0) - x[2, 1, 1] * math.sin(2.0))
    # scores depend on the distance of query and key only
    q, k = torch.randn(1, 1, 4, dtype=P.F64), torch.randn(1, 1, 4, dtype=P.F64)
    dots = [float((P.turn_pairs(q, torch.tensor([a + 3]), 50.0, 4) * P.turn_pairs(k, torch.tensor([a]), 50.0, 4)).sum())
            for a in (0, 5, 40)]
    assert max(dots) - min(dots) < 1e-12
    # the router: the largest logits, weights that sum to one over the chosen alone
    ids, w = P.route(torch.eye(3, dtype=P.F64), torch.tensor([[1., 0, 0], [0, 2, 0], [0, 0, 3], [1, 1, 1]], dtype=P.F64),
                     torch.tensor([0., 0, 0, 0.5], dtype=P.F64), 2)
    assert ids.tolist() == [[3, 0], [1, 3], [2, 3]] and torch.allclose(w.sum(-1), torch.ones(3, dtype=P.F64))
    assert float(w[0, 0]) == pytest.approx(1 / (1 + math.exp(-0.5)))
    assert float(P.gelu(torch.tensor(1.0, dtype=P.F64))) == pytest.approx(0.8413447460685429)
    # one key row a token for all heads is attention with that row as every head's key and its front as the value
    rows, qq = torch.randn(9, 6, dtype=P.F64), torch.randn(9, 2, 6, dtype=P.F64)
    a = P.shared_row_attention(qq, rows, 4, 0.7, 3)
    s = 0.7 * qq[8, 1] @ rows[6:9].T
    assert torch.allclose(a[8, 1], torch.softmax(s, -1) @ rows[6:9, :4])
