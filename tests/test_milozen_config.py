"""Milozen without a GPU: the reader of config.json, tensor names, cache groups and page bookkeeping."""

import copy

import pytest
import torch

from milozen_configs import SMALL, SMALL_B, SMALL_C, config_of, moe

from llmserve.cache.manager import CacheManager, group_layers
from llmserve.config.model_config import ConfigError
from llmserve.config.registry import architecture_of, preset
from llmserve.parts.model import Model
from llmserve.parts.registry import BuildContext


def build(config):
    arch = architecture_of(config)
    assert arch.name == "Milozen"
    cfg = arch.config_class.from_dict(config)
    return cfg, Model(arch.build_spec(cfg), BuildContext(torch.float32, torch.device("cpu")))


def test_tensor_names_and_shapes_follow_the_configuration():
    _cfg, model = build(SMALL)
    infos = model.param_infos()
    assert infos["embed"].shape == (151, 72) and infos["final.norm"].shape == (72,)
    assert "head.weight" not in infos  # the output head is the embedding table
    assert infos["l0.mix.dq"].shape == (40, 72) and infos["l0.mix.dq.norm"].shape == (40,)
    assert infos["l0.mix.uq"].shape == (3 * (16 + 8), 40)
    assert infos["l0.mix.dkv"].shape == (32 + 8, 72) and infos["l0.mix.dkv.norm"].shape == (32,)
    assert infos["l0.mix.uk"].shape == (3 * 16, 32) and infos["l0.mix.uv"].shape == (3 * 24, 32)
    assert infos["l0.mix.g"].shape == (3 * 24, 72) and infos["l0.mix.o"].shape == (72, 3 * 24)
    assert infos["l0.mlp.gate"].shape == (56, 72) and infos["l0.mlp.down"].shape == (72, 56)
    assert infos["l1.mlp.router"].shape == (5, 72)
    assert infos["l1.mlp.e4.up"].shape == (24, 72) and infos["l1.mlp.e4.down"].shape == (72, 24)
    assert "l1.mlp.e5.up" not in infos
    assert infos["l0.hc1.in"].shape == (2,) and infos["l0.hc2.mix"].shape == (2, 2)
    # a layer that reads another's cache rows has no key/value projection; a layer without feed-forward no second norm
    assert "l3.mix.dkv" not in infos and "l3.mix.dkv.norm" not in infos and "l3.mix.uk" in infos
    assert infos["l3.mix.uk"].shape == (4 * 12, 48)
    assert "l3.norm2" not in infos and "l3.hc2.in" not in infos and "l3.norm1" in infos
    assert "l3.norm2" in model.spec.unused_tensors


def test_without_streams_there_are_no_connection_tensors():
    _cfg, model = build(SMALL_C)
    assert not [n for n in model.param_infos() if ".hc" in n]
    _cfg, model = build(SMALL_B)  # one stream through connections is not the same thing
    assert model.param_infos()["l0.hc1.mix"].shape == (1, 1)


def test_a_borrowed_cache_is_kept_for_the_widest_window_among_its_readers():
    cfg, model = build(SMALL)
    specs = model.cache_specs()
    assert specs[3] is None and specs[4] is None
    assert specs[0].window == 11 and specs[0].head_dim == 32 + 8  # layer 4 reads it with a window of 5
    assert specs[2].window == 19 and specs[2].head_dim == 48 + 16  # its own 7, layer 3's 19
    assert specs[0].v_heads == 0
    assert model.cache_sources() == [None, None, None, 2, 0]
    assert cfg.cache_window(1) == 11
    _cfg, model = build(SMALL_B)
    assert model.cache_specs()[1].window is None  # its own layer has no mask, whatever the readers have
    groups = group_layers(model.cache_specs())
    assert len(groups) == 3


def test_pages_behind_the_widest_window_come_back_while_a_request_runs():
    _cfg, model = build(SMALL)
    groups = group_layers(model.cache_specs())
    manager = CacheManager(groups, 64, 4, 2)
    manager.add_sequence("a")
    for _ in range(10):
        manager.append(["a"], [10])
        manager.release_passed(["a"])
        manager.check_invariants()
    by_window = {g.spec.window: g.group_id for g in groups}
    for window, gid in by_window.items():
        table = manager.table(gid, "a")
        live = [i for i, page in enumerate(table) if page >= 0]
        assert live[0] == (100 - window + 1) // 4  # the first page a query at position 100 can still reach
    manager.free_sequence("a")
    assert all(a.num_free == 64 for a in manager.allocators.values())


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_from=1), "earlier"),
    (lambda c: c["layers"][1]["mixer"].update(kv_from=0, kv_rank=99), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0].update(type="attention"), "type"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "kind"),
])
def test_what_the_reader_refuses(change, message):
    config = copy.deepcopy(config_of(layers=[{}, {"mlp": moe()}]))
    change(config)
    with pytest.raises(ConfigError, match=message):
        build(config)


def test_a_reader_of_a_reader_is_refused():
    config = config_of(layers=[{}, {"mixer": {"kv_from": 0}}, {"mixer": {"kv_from": 0}}])
    config["layers"][2]["mixer"]["kv_from"] = 1
    with pytest.raises(ConfigError, match="no cache of its own"):
        build(config)


def test_named_sizes():
    for name in ("milozen-tiny", "milozen-1b"):
        cfg, model = build(preset(name))
        assert model.spec.vocab_size == cfg.vocab
        assert cfg.to_dict()["layers"][0]["mixer"]["heads"] == preset(name)["layers"][0]["mixer"]["heads"]
    assert build(preset("milozen-tiny"))[1].cache_sources()[3] == 2
