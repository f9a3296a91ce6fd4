"""The Mafurax design's configuration, manifest and cache rules, without a GPU."""

from __future__ import annotations

import copy

import pytest

import mafurax_models as M
import plain_mafurax as P
from pyre_amd.config import ConfigError, MafuraxConfig
from pyre_amd.parts.base import PagedCacheSpec, PagedTensorSpec, StateCacheSpec
from pyre_amd.parts.capped_attention import distance_rows
from pyre_amd.parts.model import LayeredModel
from pyre_amd.registry import config_from_dict, get_architecture


def test_config_is_chosen_by_its_name_and_round_trips():
    cfg = config_from_dict(M.SMALL)
    assert isinstance(cfg, MafuraxConfig) and cfg.vocab_size == 97 and cfg.hidden_size == 48
    assert cfg.to_dict() == M.SMALL
    assert config_from_dict(cfg.to_dict()) == cfg
    l1 = cfg.layers[1]
    assert l1.mlp is None and l1.mixer.left.window == 0 and l1.mixer.left.softcap == 0.0 and l1.mixer.right.dim == 70


def test_sizes_that_only_the_file_knows_stay_open():
    raw = copy.deepcopy(M.ONES)
    del raw["layers"][0]["mixer"]["left"]["bias_rows"], raw["layers"][0]["mixer"]["right"]["rank"]
    cfg = config_from_dict(raw)
    assert cfg.layers[0].mixer.left.bias_rows is None and cfg.to_dict() == raw
    specs = {s.name: s for s in LayeredModel(get_architecture("Mafurax").build(cfg)).tensor_specs()}
    assert specs["l0.mix.left.rel"].shape == (None, 1) and specs["l0.mix.left.rel"].fits((9, 1))
    assert not specs["l0.mix.left.rel"].fits((9, 2))
    assert specs["l0.mix.right.a1"].shape == (None, 20) and specs["l0.mix.right.a2"].shape == (3, None)


@pytest.mark.parametrize("damage", [
    lambda r: r.pop("vocab"), lambda r: r["layers"][0].update(type="serial"), lambda r: r["layers"][0]["mixer"].pop("left"),
    lambda r: r["layers"][0]["mixer"]["left"].update(heads=3, kv_heads=2), lambda r: r["layers"][0]["mlp"].update(kind="moe"),
    lambda r: r["norm"].update(eps=0), lambda r: r["layers"][0]["mixer"]["right"].update(tau=0),
    lambda r: r.update(layers=[])])
def test_a_broken_config_is_refused(damage):
    raw = copy.deepcopy(M.SMALL)
    damage(raw)
    with pytest.raises(ConfigError):
        config_from_dict(raw)


def test_manifest_names_shapes_and_caches():
    cfg = config_from_dict(M.SMALL)
    model = LayeredModel(get_architecture("Mafurax").build(cfg))
    shapes = {s.name: s.shape for s in model.tensor_specs()}
    assert shapes["embed"] == (97, 48) and shapes["final.norm"] == (48,)
    assert shapes["l0.mix.left.q"] == (96, 48) and shapes["l0.mix.left.k"] == (48, 48) and shapes["l0.mix.left.v"] == (32, 48)
    assert shapes["l0.mix.left.g"] == (4, 48) and shapes["l0.mix.left.o"] == (48, 64) and shapes["l0.mix.left.rel"] == (10, 4)
    assert shapes["l0.mix.right.q"] == (32, 48) and shapes["l0.mix.right.v"] == (48, 48) and shapes["l0.mix.right.o"] == (48, 48)
    assert shapes["l0.mix.right.a1"] == (5, 48) and shapes["l0.mix.right.a2"] == (32, 5) and shapes["l0.mix.right.a2.b"] == (32,)
    assert shapes["l0.mix.right.norm"] == (24,) and shapes["l0.mlp.gate"] == (80, 48) and shapes["l0.mlp.down"] == (48, 80)
    assert shapes["l0.ls1"] == shapes["l0.ls2"] == shapes["l0.norm1b"] == shapes["l0.norm2b"] == (48,)
    # the layer without a feed-forward has none of its matrices; that half's norms and scale may be in a file, unread
    optional = {s.name for s in model.tensor_specs() if s.optional}
    assert "l1.norm1b" in shapes and not any(n.startswith("l1.mlp") for n in shapes)
    assert optional == {"l1.norm2", "l1.norm2b", "l1.ls2"}
    assert "lm_head.weight" not in shapes
    kept = model.cache_specs()
    assert kept[0] == [PagedCacheSpec((PagedTensorSpec("k", (2, 24), 1), PagedTensorSpec("v", (2, 16), 1)), 20, 3),
                       StateCacheSpec((2, 16, 24), "float32")]
    assert kept[1][0].window == 0 and kept[1][0].keep_first == 0 and kept[2][0].window == 7


@pytest.mark.parametrize("rows,far", [(16, 120), (10, 40), (6, 9), (12, 25), (4, 6), (8, 64), (32, 128), (7, 30)])
def test_distance_rows_are_the_plain_buckets(rows, far):
    table = distance_rows(rows, far)
    assert len(table) == far + 1 and table[-1] == rows - 1
    assert table == [P.distance_bucket(n, rows, far) for n in range(far + 1)]
    assert all(P.distance_bucket(n, rows, far) == rows - 1 for n in range(far, far + 300))
    assert all(b >= a for a, b in zip(table, table[1:]))


def test_pages_of_the_kept_first_tokens_are_never_given_back():
    from pyre_amd.cache import CacheManager

    spec = PagedCacheSpec((PagedTensorSpec("k", (1, 4), 1),), window=10, keep_first=9)   # two pages of 8 hold the first 9
    plain_window = PagedCacheSpec((PagedTensorSpec("k", (1, 2), 1),), window=10)
    m = CacheManager([[spec], [plain_window]], page_size=8, num_pages=16, max_num_seqs=2, max_model_len=128)
    m.add_request("a")
    for _ in range(10):
        m.reserve("a", 7)
        m.commit("a", 7)
    kept, free = m.block_table("a", 0), m.block_table("a", 1)
    assert kept[0] >= 0 and kept[1] >= 0 and all(p == -1 for p in kept[2:7]) and all(p >= 0 for p in kept[7:])
    assert all(p == -1 for p in free[:7]) and all(p >= 0 for p in free[7:])
    m.check_invariants()
    m.free_request("a")
    assert all(g.allocator.num_used == 0 for g in m.page_groups)


def test_random_folder_loads_back(tmp_path):
    from pyre_amd.weights import write_random_model
    from pyre_amd.weights.loader import check_against, checkpoint_index

    cfg = config_from_dict(M.ONES)
    write_random_model(tmp_path, cfg, seed=5, std=0.3, gain_std=0.2)
    specs = LayeredModel(get_architecture("Mafurax").build(cfg)).tensor_specs()
    check_against(specs, checkpoint_index(tmp_path), tmp_path)
    raw, w = P.read_folder(tmp_path)
    assert raw == M.ONES and w["l0.mix.left.rel"].shape == (4, 1) and w["l0.mix.right.a2"].shape == (3, 1)
    assert float(w["l0.mix.left.rel"].abs().max()) > 0.2   # the distance table is drawn wide enough to matter
    logits = P.forward(raw, w, [3, 1, 4, 1, 5])
    assert logits.shape == (5, 31) and bool(logits.isfinite().all())


def test_norms_of_a_missing_feed_forward_may_be_in_the_file_or_not(tmp_path):
    import torch
    from safetensors.torch import load_file, save_file

    from pyre_amd.weights import write_random_model
    from pyre_amd.weights.loader import WeightsError, check_against, checkpoint_index

    cfg = config_from_dict(M.SMALL)
    write_random_model(tmp_path, cfg, seed=6)
    specs = LayeredModel(get_architecture("Mafurax").build(cfg)).tensor_specs()
    state = load_file(str(tmp_path / "model.safetensors"))
    assert "l1.norm2" not in state
    check_against(specs, checkpoint_index(tmp_path), tmp_path)
    state.update({n: torch.ones(48, dtype=torch.bfloat16) for n in ("l1.norm2", "l1.norm2b", "l1.ls2")})
    save_file(state, str(tmp_path / "model.safetensors"))
    check_against(specs, checkpoint_index(tmp_path), tmp_path)
    state["l1.mlp.gate"] = torch.ones(4, 48, dtype=torch.bfloat16)      # a matrix that no part names is still refused
    save_file(state, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError):
        check_against(specs, checkpoint_index(tmp_path), tmp_path)
