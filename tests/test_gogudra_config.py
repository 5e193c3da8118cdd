"""The Gogudra architecture without a GPU: its configuration reader, the spec it builds, tensor
names and shapes, frequency scaling, and a model folder written by the random-weights mode."""

import copy
import json
import os

import pytest
import torch

import gogudra_util as gu
from plain_gogudra import scaled_frequencies


def _folder(tmp_path, cfg, seed=0, rank=6):
    return gu.write_model(str(tmp_path / "m"), cfg, seed, rank)


def test_registered_and_chosen_by_config_json(tmp_path):
    from qwen25vl_lite_amd.config import known_architectures, load_config
    from qwen25vl_lite_amd.models.gogudra import GogudraConfig
    assert "Gogudra" in known_architectures()
    cfg = load_config(_folder(tmp_path, gu.MIXED))
    assert isinstance(cfg, GogudraConfig) and cfg.width == 80 and cfg.vocab == 211 and cfg.eps == 1e-5
    assert cfg.to_dict() == gu.MIXED


def test_expected_tensors_are_the_files(tmp_path):
    """Names and shapes come out as the file has them; the decay projection's inner size is read from
    a tensor's shape; the head is the embedding table."""
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    for cfg, rank in ((gu.MIXED, 6), (gu.ONES, 3), (gu.NO_PAGES, 10)):
        d = gu.write_model(str(tmp_path / f"m{rank}"), cfg, 1, rank)
        model = build_model(load_config(d), torch.float32, "meta")
        mine = {model.spec.store_name(k): tuple(v.shape) for k, v in model.expected_tensors().items()}
        assert mine.pop("lm_head") == (cfg["vocab"], cfg["width"]) and model.spec.tie_word_embeddings
        assert mine == gu.tensor_shapes(cfg, rank)
        for name in mine:
            assert model.spec.store_name(model.spec.map_name(name)) == name


def test_cache_groups_and_states(tmp_path):
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    model = build_model(load_config(_folder(tmp_path, gu.MIXED)), torch.float32, "meta")
    groups = model.cache_groups()
    assert [(g.need.num_kv_heads, g.need.head_dim, g.need.window, g.num_layers) for g in groups] == \
        [(2, 24, None, 1), (4, 32, None, 1)]
    assert [None if s is None else s.shape for s in model.entry_state] == \
        [(2, 12, 24), None, (3, 20, 40), None, (1, 64, 8)]
    assert model.graph_safe


def test_a_model_without_attention_has_no_pages(tmp_path):
    from qwen25vl_lite_amd.cache import CacheManager
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.models import build_model
    model = build_model(load_config(_folder(tmp_path, gu.NO_PAGES, rank=10)), torch.float32, "meta")
    assert model.cache_groups() == []
    cache = CacheManager([], 4, 16, 2, enable_prefix_cache=False)
    cache.admit("a")
    cache.reserve("a", 100)
    cache.commit("a", 100)
    assert cache.num_tokens("a") == 100
    cache.release("a")


@pytest.mark.parametrize("broken, word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("tau"), "tau"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 8), "vdim"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 4), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("decay", [0.5]), "decay"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "kind"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
])
def test_config_errors_name_the_key(broken, word):
    from qwen25vl_lite_amd.config import ConfigError, load_config
    cfg = copy.deepcopy(gu.MIXED)
    broken(cfg)
    with pytest.raises(ConfigError, match=word):
        load_config(cfg)


def test_frequency_scaling_matches_the_plain_rule():
    from qwen25vl_lite_amd.parts.rope import rescale_frequencies
    for rot in ({"base": 50000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}},
                {"base": 10000.0, "dims": 64, "scaling": {"factor": 3.0, "low": 2.0, "high": 5.0, "original": 512}},
                {"base": 100.0, "dims": 6, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}):
        plain = torch.tensor(scaled_frequencies(rot), dtype=torch.float64)
        base = torch.tensor([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)], dtype=torch.float64)
        sc = rot["scaling"]
        got = rescale_frequencies(base, sc["factor"], sc["low"], sc["high"], sc["original"])
        assert torch.allclose(got, plain, rtol=1e-12, atol=0)
        # all three regimes occur in the first two
        if rot["dims"] > 6:
            ratio = plain / base
            assert (ratio == 1).any() and torch.isclose(ratio, torch.tensor(1 / sc["factor"], dtype=torch.float64)).any()
            assert ((ratio < 0.999) & (ratio > 1 / sc["factor"] + 1e-3)).any()


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    """The random-weights mode works from the configuration alone when it names the decay
    projection's inner size; the folder has the file names of the design."""
    from qwen25vl_lite_amd import write_random_model
    from qwen25vl_lite_amd.weights import SafetensorsFile
    cfg = copy.deepcopy(gu.MIXED)
    for layer in cfg["layers"]:
        if layer["type"] == "gla":
            layer["mixer"]["rank"] = 5
    d = write_random_model(cfg, str(tmp_path / "w"), seed=3)
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        shapes = {k: tuple(f.shape(k)) for k in f.keys()}
    assert shapes == gu.tensor_shapes(cfg, 5)
    with open(os.path.join(d, "config.json")) as fh:
        assert json.load(fh) == cfg
    # without the size and without a folder there is nothing to read it from
    from qwen25vl_lite_amd.config import ConfigError
    with pytest.raises(ConfigError, match="rank"):
        write_random_model(copy.deepcopy(gu.MIXED), str(tmp_path / "x"), seed=3)
