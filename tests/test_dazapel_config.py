"""The Dazapel architecture without a GPU: its reader of config.json, its spec and run list, tensor
names, the frequency ramp, windowed pages that keep the first tokens, the random-weights folder."""

import copy
import math

import pytest
import torch

import dazapel_util as du
import plain_dazapel as plain


def _spec(cfg):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    return build_model(load_config(copy.deepcopy(cfg)), torch.float32, "meta")


@pytest.mark.parametrize("cfg", [du.MIXED, du.ONES, du.ODD])
def test_the_spec_expects_the_files_tensors(cfg):
    model = _spec(cfg)
    got = {model.spec.store_name(k): tuple(v.shape) for k, v in model.expected_tensors().items()}
    got.pop("lm_head")      # tied to the table
    assert got == du.tensor_shapes(cfg)
    for name in du.tensor_shapes(cfg):
        assert model.spec.store_name(model.spec.map_name(name)) == name


def test_run_list_follows_the_loop():
    from qwen25vl_lite_amd.models.dazapel import dazapel_run_list
    run = dazapel_run_list(5, {"start": 1, "stop": 3, "times": 3})
    assert [(e.layer, e.add_vector) for e in run] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None),
                                                      (3, None), (4, None)]
    assert [(i, t) for i, t in plain.run_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}})] == \
        [(e.layer, e.add_vector) for e in run]
    assert [e.layer for e in dazapel_run_list(3, None)] == [0, 1, 2]
    model = _spec(du.MIXED)
    # every pass through a looped layer has a cache layer of its own: 4 layers, two of them three times
    assert sum(g.num_layers for g in model.cache_groups()) == 8
    assert len(model.cache_groups()) == 4   # four different shapes and windows


def test_cache_needs_carry_window_kept_tokens_and_value_size():
    needs = {(g.need.head_dim, g.need.v_dim, g.need.window, g.need.keep_first) for g in _spec(du.MIXED).cache_groups()}
    assert needs == {(16, 24, 9, 3), (20, 12, 21, 0), (32, 32, None, 0), (48, 16, 37, 18)}


@pytest.mark.parametrize("bad, text", [
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 5), "fit together"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].__setitem__("count", 3), "fit together"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), "kind"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("keep_first"), "keep_first"),
])
def test_config_errors_name_the_key(bad, text):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.config.model_config import ConfigError
    cfg = copy.deepcopy(du.MIXED)
    bad(cfg)
    with pytest.raises(ConfigError, match=text):
        load_config(cfg)


def test_optional_blocks_may_be_absent():
    cfg = copy.deepcopy(du.ODD)
    cfg["layers"][0]["mixer"]["rot"]["scaling"] = None
    cfg["layers"][0]["mixer"].pop("mask")
    cfg["layers"][0]["mlp"]["shared"] = None
    cfg["loop"] = None
    model = _spec(cfg)
    assert model.pass_vectors is None and "l0.mlp.shared.gate.weight" not in model.expected_tensors()


@pytest.mark.parametrize("dims, base, sc", [(8, 500.0, du.RAMP), (16, 80.0, {"factor": 2.0, "original": 16, "fast": 2.0, "slow": 1.0}),
                                            (64, 250000.0, {"factor": 6.0, "original": 256, "fast": 16.0, "slow": 2.0}),
                                            (6, 77.0, du.RAMP)])
def test_frequency_ramp(dims, base, sc):
    from qwen25vl_lite_amd.parts.base import PartSpec, build_part
    rope = build_part("position", PartSpec("rope", {"theta": base, "rotary_dim": dims, "scaling": dict(sc, kind="ramp")}),
                      torch.float32, torch.device("cpu"))
    freqs, _ = rope.rotary_tables(dims + 2)
    want, mult = plain.yarn_frequencies(dims, base, sc)
    assert torch.allclose(freqs.double(), want, rtol=1e-6, atol=0)
    assert rope.amplitude == pytest.approx(mult) == pytest.approx(0.1 * math.log(sc["factor"]) + 1.0)
    plain_f, one = plain.yarn_frequencies(dims, base, None)
    assert one == 1.0 and plain_f[0] == 1.0 and (want <= plain_f + 1e-12).all()


def test_a_windowed_group_keeps_the_pages_of_the_first_tokens():
    from qwen25vl_lite_amd.cache.manager import CacheGroupSpec, CacheManager
    from qwen25vl_lite_amd.parts.base import CacheNeed
    groups = [CacheGroupSpec(CacheNeed(2, 16, window=10, keep_first=5), 1), CacheGroupSpec(CacheNeed(2, 16, window=10), 1),
              CacheGroupSpec(CacheNeed(2, 16, window=6, keep_first=9), 1)]
    cm = CacheManager(groups, 16, 4, 2, enable_prefix_cache=False)
    cm.admit("a")
    for upto in (3, 11, 12, 30, 31, 47):
        cm.reserve("a", upto)
        cm.commit("a", upto)
        for g, (window, keep) in enumerate(((10, 5), (10, 0), (6, 9))):
            table = cm.table("a", g)
            for page, held in enumerate(table):
                tokens = range(page * 4, page * 4 + 4)
                seen_later = any(t < keep or t >= upto - window + 1 for t in tokens)
                assert (held >= 0) == seen_later, (upto, g, page)
    cm.check()
    before = cm.free_pages()
    cm.release("a")
    cm.check()
    assert cm.free_pages() == [16, 16, 16] and before[0] < 16


def test_random_weights_folder_loads_back(tmp_path):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.weights import write_random_model
    from qwen25vl_lite_amd.weights.safetensors_io import SafetensorsFile
    folder = write_random_model(load_config(copy.deepcopy(du.ODD)), str(tmp_path / "m"), seed=3)
    with SafetensorsFile(folder + "/model.safetensors") as f:
        assert {n: tuple(f.shape(n)) for n in f.keys()} == du.tensor_shapes(du.ODD)
    cfg, tensors = plain.dazapel_read(folder)
    logits = plain.dazapel_forward(cfg, tensors, [1, 2, 3, 4, 5, 6, 7])
    assert logits.shape == (7, 101) and torch.isfinite(logits).all()


def test_plain_router_limits_the_choice_to_the_best_groups():
    z = torch.tensor([[3.0, 2.9, -5.0, -5.0, 2.0, 1.9, 2.95, -9.0]], dtype=torch.float64)
    chosen, w = plain.route(z, top=3, groups=4, keep=2, scale=2.0)
    # group scores: (0,1) highest, then (4,5); expert 6 is the third largest score but its group (6,7) is out
    assert sorted(chosen[0].tolist()) == [0, 1, 4]
    assert w.sum().item() == pytest.approx(2.0)


def test_plain_mask():
    see = plain.visible(12, 4, 2)
    assert see[11].nonzero().flatten().tolist() == [0, 1, 8, 9, 10, 11]
    assert see[3].nonzero().flatten().tolist() == [0, 1, 2, 3]
    assert plain.visible(5, None, 0)[4].all()
