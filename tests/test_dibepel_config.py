"""Dibepel without a GPU: its configuration reader, the spec it builds, its tensor names, and what
its layers ask of the cache manager (pages behind a window that keeps first tokens, pages of passed
chunks, a state slot beside pages)."""

import pytest
import torch

from dibepel_configs import SMALL, SMALL_B, config_of


def spec_of(config):
    from llmserve.config.registry import architecture_of

    arch = architecture_of(config)
    return arch, arch.build_spec(arch.config_class.from_dict(config))


def test_architecture_is_found_by_its_own_key():
    from llmserve.config import ConfigError
    from llmserve.config.registry import architecture_of

    assert architecture_of(SMALL).name == "Dibepel"
    assert architecture_of({"architectures": ["Dibepel"]}).name == "Dibepel"
    with pytest.raises(ConfigError):
        architecture_of(SMALL).config_class.from_dict({"architecture": "Dibepel", "vocab": 10})


def test_layers_that_borrow_weights_become_second_runs():
    _, spec = spec_of(SMALL)
    # layers 0..3 own tensors; 4 runs on 1's, 5 on 2's
    assert len(spec.layers) == 4 and spec.schedule == (0, 1, 2, 3, 1, 2)
    cfg = config_of(layers=[("attention_2", {}), ("attention", {}), ("attention_2", {"weights_of": 0}),
                            ("attention_2", {"weights_of": 2})])  # a chain ends at the layer with tensors
    _, spec = spec_of(cfg)
    assert spec.schedule == (0, 1, 0, 0)


def test_bad_configurations_are_refused():
    from llmserve.config import ConfigError

    arch, _ = spec_of(SMALL)
    for change in ({"type": "attention_3"}, {"weights_of": 9}, {"mixer": {"heads": 3, "kv_heads": 2, "dim": 8, "vdim": 8}},
                   {"mlp": {"kind": "experts", "ff": 8}}):
        cfg = config_of()
        cfg["layers"][0] = dict(cfg["layers"][0], **change)
        with pytest.raises(ConfigError):
            arch.config_class.from_dict(cfg)
    loop = config_of(layers=[("attention", {}), ("attention", {})])
    loop["layers"][0]["weights_of"], loop["layers"][1]["weights_of"] = 1, 0
    with pytest.raises(ConfigError):
        arch.config_class.from_dict(loop)


def test_tensor_names_and_shapes():
    from llmserve.parts import BuildContext
    from llmserve.parts.model import Model

    _, spec = spec_of(SMALL)
    infos = Model(spec, BuildContext(torch.float32, torch.device("cpu"))).param_infos()
    w = SMALL["width"]
    m0, m1 = SMALL["layers"][0]["mixer"], SMALL["layers"][1]["mixer"]
    assert infos["embed"].shape == (SMALL["vocab"], w) and infos["head"].shape == (SMALL["vocab"], w)
    assert infos["final.norm"].shape == (w,) and infos["l0.norm1"].shape == (w,)
    assert infos["l0.mix.q"].shape == (m0["heads"] * m0["dim"], w)
    assert infos["l0.mix.q.conv"].shape == (m0["heads"] * m0["dim"], m0["conv"])
    assert infos["l0.mix.v.conv"].shape == (m0["kv_heads"] * m0["vdim"], m0["conv"])
    assert infos["l0.mix.talk"].shape == (m0["heads"], m0["heads"])
    assert infos["l0.mix.o"].shape == (w, m0["heads"] * m0["vdim"])
    assert infos["l1.mix.q"].shape == (m1["heads"] * 2 * m1["dim"], w)  # two score maps per head
    assert infos["l1.mix.k"].shape == (m1["kv_heads"] * 2 * m1["dim"], w)
    assert infos["l1.mix.v"].shape == (m1["kv_heads"] * m1["vdim"], w)
    assert infos["l1.mix.lq1"].shape == (m1["dim"],)
    assert infos["l0.rg1"].shape == (w, w) and infos["l0.rg2.b"].shape == (w,)
    assert infos["l0.mlp.gate"].shape == (SMALL["layers"][0]["mlp"]["ff"], w)
    assert not any(name.startswith(("l4.", "l5.")) for name in infos)  # borrowed layers hold nothing
    # layer 3 has no feed-forward: no tensors for it or its gate, and a checkpoint may hold the gate all the same
    assert not any(name.startswith(("l3.mlp", "l3.rg2")) for name in infos)
    assert set(spec.unused_tensors) == {"l3.rg2", "l3.rg2.b"}


def test_cache_groups_hold_pages_and_a_state():
    from llmserve.cache import group_layers
    from llmserve.parts import BuildContext, PagedCacheSpec, StateCacheSpec
    from llmserve.parts.model import Model

    _, spec = spec_of(SMALL)
    model = Model(spec, BuildContext(torch.float32, torch.device("cpu")))
    groups = group_layers(model.cache_specs())
    m0, m1 = SMALL["layers"][0]["mixer"], SMALL["layers"][1]["mixer"]
    channels = (m0["heads"] + m0["kv_heads"]) * m0["dim"] + m0["kv_heads"] * m0["vdim"]
    by_spec = {g.spec: g.layers for g in groups}
    chunked = PagedCacheSpec(m0["kv_heads"], m0["dim"], chunk=m0["mask"]["size"], value_heads=m0["kv_heads"],
                             value_dim=m0["vdim"])
    windowed = PagedCacheSpec(2 * m1["kv_heads"], m1["dim"], window=m1["mask"]["size"],
                              keep_first=m1["mask"]["keep_first"], value_heads=m1["kv_heads"], value_dim=m1["vdim"])
    assert by_spec[chunked] == (0, 2, 5) and by_spec[windowed] == (1, 4)
    assert by_spec[StateCacheSpec((m0["conv"] - 1, channels), "float32")] == (0, 2, 5)
    assert SMALL["layers"][3]["mixer"]["conv"] == 1  # one tap needs no state: schedule entry 3 keeps pages only
    assert all(3 not in g.layers for g in groups if not g.paged)
    assert sum(3 in g.layers for g in groups if g.paged) == 1


def test_reach_of_a_paged_spec():
    from llmserve.parts import PagedCacheSpec

    win = PagedCacheSpec(1, 8, window=10, keep_first=3)
    assert win.bounded and win.live_tokens() == 10
    assert win.dead_before(9) == 0 and win.dead_before(10) == 1 and win.dead_before(25) == 16
    chunk = PagedCacheSpec(1, 8, chunk=6)
    assert chunk.bounded and [chunk.dead_before(n) for n in (0, 5, 6, 11, 12)] == [0, 0, 6, 6, 12]
    assert not PagedCacheSpec(1, 8).bounded


def manager_for(spec, pages, block_size=4, seqs=2):
    from llmserve.cache import CacheManager, group_layers

    return CacheManager(group_layers([spec]), pages, block_size, seqs)


def held(manager, seq):
    return [i for i, page in enumerate(manager.table(0, seq)) if page >= 0]


def test_pages_of_kept_first_tokens_stay_and_the_window_moves_on():
    from llmserve.parts import PagedCacheSpec

    m = manager_for(PagedCacheSpec(1, 8, window=6, keep_first=5), pages=16)
    m.add_sequence("a")
    m.append(["a"], [30])
    m.release_passed(["a"])
    # keys 0..4 are kept (pages 0, 1); the next query sits at 30 and sees 25..: page 6 on
    assert held(m, "a") == [0, 1, 6, 7]
    for _ in range(10):
        m.append(["a"], [1])
        m.release_passed(["a"])
    assert held(m, "a") == [0, 1, 8, 9]  # length 40: keys 35.. are in reach
    m.check_invariants()
    m.free_sequence("a")
    assert m.free_pages() == {0: 16}


def test_pages_of_passed_chunks_come_back():
    from llmserve.parts import PagedCacheSpec

    m = manager_for(PagedCacheSpec(1, 8, chunk=10), pages=8)
    m.add_sequence("a")
    m.append(["a"], [9])
    m.release_passed(["a"])
    assert held(m, "a") == [0, 1, 2]  # position 9 still belongs to the first chunk
    m.append(["a"], [1])
    m.release_passed(["a"])
    assert held(m, "a") == [2]  # the next query opens chunk 10..19: only the page of key 10 (8..11) can matter
    m.append(["a"], [25])  # to length 35, chunk 30..39: pages from 7 on
    m.release_passed(["a"])
    assert held(m, "a") == [7, 8]
    m.check_invariants()
    # a long request never holds more than a chunk and a step: the pool of 8 pages served 35 tokens of 4 a page
    need = m.pages_for(10_000, step_tokens=4)
    assert need[0] == -(-(10 - 1 + 4) // 4) + 1


def test_pool_sizes_count_the_kept_first_pages():
    from llmserve.cache.manager import bounded_pages, window_pages
    from llmserve.parts import PagedCacheSpec

    assert window_pages(6, 4, 4) == 4 and window_pages(6, 4, 4, keep_first=5) == 6
    assert bounded_pages(PagedCacheSpec(1, 8, window=6, keep_first=5), 4, 4) == 6
    assert bounded_pages(PagedCacheSpec(1, 8, window=100, chunk=6), 4, 4) == 4  # the narrower bound counts


def test_page_bytes_with_values_of_another_shape():
    from llmserve.cache import group_layers
    from llmserve.cache.storage import page_bytes_of
    from llmserve.parts import PagedCacheSpec

    (g,) = group_layers([PagedCacheSpec(4, 8, value_heads=2, value_dim=24)] * 3)
    assert page_bytes_of(g, 16, 2) == 3 * 16 * 2 * (4 * 8 + 2 * 24)


def test_random_weights_for_every_tensor(tmp_path):
    from safetensors.torch import load_file

    from llmserve.weights import write_random_model

    write_random_model(tmp_path, SMALL_B, seed=3)
    w = load_file(str(tmp_path / "model.safetensors"))
    assert w["l0.norm1"].abs().max() < 1.0  # stored as a deviation from one
    taps = w["l1.mix.k.conv"]
    assert taps.shape[1] == SMALL_B["layers"][1]["mixer"]["conv"] and float(taps[:, -1].mean()) > 0.5
    talk = w["l1.mix.talk"]
    assert float(talk.diagonal().mean()) > 0.5
