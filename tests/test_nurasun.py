"""The Nurasun design's configuration, manifest and cache rules, and the plain implementation's pieces, without a GPU."""

from __future__ import annotations

import copy

import pytest
import torch

import nurasun_models as M
import plain_nurasun as P
from pyre_amd.config import ConfigError, NurasunConfig
from pyre_amd.parts.base import PagedCacheSpec
from pyre_amd.parts.model import LayeredModel
from pyre_amd.registry import config_from_dict, get_architecture


def test_config_is_chosen_by_its_name_and_round_trips():
    for raw in (M.SMALL, M.ONES, M.WIDE, M.ODD):
        cfg = config_from_dict(raw)
        assert isinstance(cfg, NurasunConfig) and cfg.to_dict() == raw and config_from_dict(cfg.to_dict()) == cfg
    cfg = config_from_dict(M.SMALL)
    assert cfg.vocab_size == 113 and cfg.hidden_size == 40 and cfg.residual_mult == 0.45 and cfg.logit_softcap == 9.0
    l0, l2 = cfg.layers[0], cfg.layers[2]
    assert l0.mixer.chunk == 20 and l0.mixer.rot_dims == 16 and l0.mixer.rot_base == 500.0
    assert l2.mlp is None and l2.mixer.kv_from == 1 and l2.mixer.kv_rank == 40
    wide = config_from_dict(M.WIDE)
    assert wide.layers[0].mixer.chunk == 0 and wide.layers[0].mixer.rot_dims == 0 and wide.layers[0].mlp.shared_ff == 24


@pytest.mark.parametrize("damage", [
    lambda r: r.pop("width"), lambda r: r["layers"][0].update(type="recurrent"), lambda r: r["layers"][0].pop("mixer"),
    lambda r: r["layers"][0]["mixer"].update(heads=3, kv_heads=2), lambda r: r["layers"][0]["mlp"].update(kind="sparse"),
    lambda r: r["layers"][0]["mixer"].update(vdim=8), lambda r: r["layers"][0]["mixer"]["rot"].update(dims=26),
    lambda r: r["layers"][0]["mixer"]["rot"].update(dims=5), lambda r: r["norm"].update(eps=0),
    lambda r: r["layers"][1]["mlp"]["router"].update(top=6), lambda r: r["layers"][2]["mixer"].update(kv_from=2),
    lambda r: r["layers"][2]["mixer"].update(kv_from=0), lambda r: r["layers"][2]["mixer"].update(kv_rank=24),
    lambda r: r["layers"][4]["mixer"].update(kv_from=2), lambda r: r.update(layers=[])])
def test_a_broken_config_is_refused(damage):
    raw = copy.deepcopy(M.SMALL)
    damage(raw)
    with pytest.raises(ConfigError):
        config_from_dict(raw)


def test_manifest_names_shapes_and_caches():
    cfg = config_from_dict(M.SMALL)
    model = LayeredModel(get_architecture("Nurasun").build(cfg))
    shapes = {s.name: s.shape for s in model.tensor_specs()}
    assert shapes["embed"] == shapes["head"] == (113, 40)
    assert shapes["final.norm"] == shapes["final.norm.b"] == shapes["l3.norm1"] == (40,) and shapes["l3.norm1.alpha"] == ()
    assert shapes["l0.mix.q"] == (96, 40) and shapes["l0.mix.k"] == (48, 40) and shapes["l0.mix.q.b"] == (96,)
    assert shapes["l0.mix.k.b"] == (48,) and shapes["l0.mix.o"] == (40, 96) and "l0.mix.v" not in shapes
    assert shapes["l1.mix.q"] == (48, 40) and shapes["l1.mix.dkv"] == (40, 40) and shapes["l1.mix.dkv.norm"] == (40,)
    assert shapes["l1.mix.uk"] == (48, 40) and shapes["l1.mix.uv"] == (72, 40) and shapes["l1.mix.o"] == (40, 72)
    assert "l2.mix.dkv" not in shapes and "l2.mix.dkv.norm" not in shapes and shapes["l2.mix.uk"] == (16, 40)
    assert shapes["l1.mlp.router"] == (5, 40) and shapes["l1.mlp.e4.up"] == (24, 40) and shapes["l1.mlp.e4.down"] == (40, 24)
    assert shapes["l1.mlp.shared.up"] == (16, 40) and "l3.mlp.shared.up" not in shapes and "l1.mlp.e5.up" not in shapes
    assert shapes["l0.mlp.gate"] == shapes["l0.mlp.up"] == (56, 40) and shapes["l0.mlp.down"] == (40, 56)
    assert not any(n.startswith("l2.mlp") for n in shapes)
    caches = model.cache_specs()
    assert [len(c) for c in caches] == [1, 1, 0, 1, 1] and all(isinstance(c[0], PagedCacheSpec) for c in caches if c)
    assert [t.name for t in caches[0][0].tensors] == ["k", "v"] and caches[0][0].tensors[0].token_shape == (2, 24)
    assert caches[0][0].chunk == 20 and caches[3][0].chunk == 7 and caches[1][0].chunk == 0
    assert [t.token_shape for t in caches[1][0].tensors] == [(1, 40)] and caches[4][0].tensors[0].token_shape == (1, 12)
    assert [c.cache_from for c in model.schedule] == [None, None, 1, None, None]


def test_random_weights_fit_the_manifest(tmp_path):
    from pyre_amd.weights import write_random_model

    write_random_model(tmp_path, config_from_dict(M.ONES), seed=3, std=0.2, gain_std=0.1)
    cfg, w = P.read_folder(tmp_path)
    assert cfg == M.ONES and w["l0.norm1.alpha"].shape == () and w["l1.mix.dkv"].shape == (2, 20)
    z, hidden = P.forward(w, cfg, [3, 1, 4, 1, 5], return_hidden=True)
    assert z.shape == (5, 31) and len(hidden) == 2 and float(z.abs().max()) <= 2.5  # the squashed logits stay under the cap


# ----------------------------------------------------------------------------- the plain pieces say what they should


def test_plain_masks():
    run = P.same_chunk(4)
    assert [j for j in range(10) if run(6, j)] == [4, 5, 6] and [j for j in range(10) if run(4, j)] == [4]
    assert [j for j in range(10) if run(3, j)] == [0, 1, 2, 3] and [j for j in range(5) if P.causal(2, j)] == [0, 1, 2]


def test_plain_rotation_turns_pairs_and_keeps_the_rest():
    x = torch.arange(12, dtype=P.F).view(1, 2, 6) + 1
    y = P.rotate(x.expand(3, 2, 6).clone(), [0, 1, 5], 4, 10.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[:, :, 4:], x.expand(3, 2, 6)[:, :, 4:])
    # element 0 pairs with element 2 at angle p, element 1 with 3 at angle p / sqrt(10); lengths are kept
    c, s = torch.cos(torch.tensor(5.0, dtype=P.F)), torch.sin(torch.tensor(5.0, dtype=P.F))
    assert torch.allclose(y[2, 0, 0], x[0, 0, 0] * c - x[0, 0, 2] * s) and torch.allclose(y[2, 0, 2], x[0, 0, 2] * c + x[0, 0, 0] * s)
    a = torch.tensor(10.0 ** -0.5, dtype=P.F)
    assert torch.allclose(y[1, 1, 1], x[0, 1, 1] * torch.cos(a) - x[0, 1, 3] * torch.sin(a))
    assert torch.allclose((y[:, :, :4] ** 2).sum(-1), (x[:, :, :4] ** 2).sum(-1).expand(3, 2))


def test_plain_routing_takes_the_largest_and_weights_sum_to_one():
    w = {"m.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [-1.0, 0.0], [0.5, 0.5]], dtype=P.F)}
    picks = P.route(torch.tensor([[2.0, 1.0], [-3.0, 0.1]], dtype=P.F), w, "m", 2)
    assert [e for e, _ in picks[0]] == [0, 3] and [e for e, _ in picks[1]] == [2, 1]
    for chosen in picks:
        assert abs(sum(float(x) for _, x in chosen) - 1.0) < 1e-12
    s = torch.sigmoid(torch.tensor([2.0, 1.5], dtype=P.F))
    assert abs(float(picks[0][0][1]) - float(s[0] / s.sum())) < 1e-12


def test_plain_norm_and_activations():
    w = {"n": torch.tensor([2.0, 1.0], dtype=P.F), "n.b": torch.tensor([0.5, -0.5], dtype=P.F), "n.alpha": torch.tensor(0.5, dtype=P.F)}
    y = P.squash_norm(torch.tensor([[2.0, -40.0]], dtype=P.F), w, "n")
    assert torch.allclose(y, torch.tensor([[2 * torch.tanh(torch.tensor(1.0, dtype=P.F)) + 0.5, -1.5]], dtype=P.F))
    z = torch.linspace(-4, 4, 9, dtype=P.F)
    assert torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(P.unit_rms(torch.tensor([[3.0, 4.0]], dtype=P.F), 0.0), torch.tensor([[3.0, 4.0]], dtype=P.F) / (12.5 ** 0.5))
