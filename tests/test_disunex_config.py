"""The Disunex configuration: what its config.json turns into, and what is refused."""
import copy
import json
import os

import pytest
import torch

from disunex_models import DISUNEX_CONFIGS, DX_P, DX_R, make_disunex_dir
from tffinfer_amd.config.base import ConfigError, LayerCall
from tffinfer_amd.models import build_model_skeleton, config_from_dict, load_config
from tffinfer_amd.parts import GeluMLP, LatentAttention, NoFeedForward, PostNormBlock, RoutedExperts
from tffinfer_amd.weights.loader import WeightError, check_weights
from tffinfer_amd.weights.safetensors_io import load_model_dir


def test_layers_that_borrow_tensors_are_calls_of_their_owner_with_a_cache_of_their_own():
    cfg = config_from_dict(copy.deepcopy(DX_P))
    assert cfg.owners() == [0, 1, 3]
    assert cfg.layer_schedule() == [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(2, 3), LayerCall(1, 4)]
    model = build_model_skeleton(cfg)
    assert len(model.blocks) == 3 and all(isinstance(b, PostNormBlock) and b.alpha == 2.0 for b in model.blocks)
    assert [type(b.feed_forward) for b in model.blocks] == [GeluMLP, RoutedExperts, NoFeedForward]
    caches = [c for c, _, _, _ in model.call_requirements()]
    assert caches == [0, 1, 2, 3, 4]
    specs = [kv for _, _, kv, _ in model.call_requirements()]
    assert specs[0] == specs[2] and specs[1] == specs[4] and specs[0] != specs[1]
    assert specs[0].num_kv_heads == 1 and specs[0].window == 12 and specs[3].window == 0


def test_a_layer_may_borrow_from_a_later_one_and_a_large_key_is_padded_to_a_multiple_of_8():
    from disunex_models import DX_T
    cfg = config_from_dict(copy.deepcopy(DX_T))
    assert cfg.owners() == [1] and cfg.layer_schedule() == [LayerCall(0, 0), LayerCall(0, 1)]
    model = build_model_skeleton(cfg)
    assert sorted(n for n in model.expected_tensors() if n.endswith("norm1")) == ["l1.norm1"]
    assert model.blocks[0].mixer.cache_spec().head_dim == 288


def test_every_size_comes_from_the_file():
    cfg = config_from_dict(copy.deepcopy(DX_R))
    m = build_model_skeleton(cfg).blocks[0].mixer
    assert isinstance(m, LatentAttention)
    assert (m.num_heads, m.head_dim, m.rot_dim, m.value_dim, m.kv_rank, m.window, m.scale) == (20, 8, 10, 8, 150, 33, 0.25)
    assert m.position.rotary_dim == 6 and m.position.pairing == "interleaved"
    assert m.key_dim == 160 and m.cache_spec().head_dim == 192      # padded to a size the matrix-core kernels take
    ff = build_model_skeleton(cfg).blocks[0].feed_forward
    assert (ff.num_experts, ff.top, ff.intermediate_size, ff.limit) == (6, 3, 16, 0.5)


def test_tensor_names_follow_the_files():
    cfg = config_from_dict(copy.deepcopy(DX_P))
    names = build_model_skeleton(cfg).expected_tensors()
    for n in ("embed", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk",
              "l0.mix.uv", "l0.mix.sink", "l0.mix.g", "l0.mix.o", "l0.mlp.up", "l0.mlp.down", "l1.mlp.router",
              "l1.mlp.correction", "l1.mlp.e4.gate", "l1.mlp.e0.down", "l3.mix.q", "l3.norm1"):
        assert n in names, n
    assert not any(n.startswith(("l2.", "l4.", "head")) for n in names)       # borrowed layers and the head have none
    assert names["l3.norm2"].optional and not names["l0.norm2"].optional
    assert names["l0.mix.q"].shape == (4 * (16 + 8), 64) and names["l0.mix.dkv"].shape == (48, 64)
    assert names["l1.mlp.e0.gate"].shape == (40, 64) and names["l1.mlp.e0.down"].shape == (64, 40)


def test_round_trip_and_refusals(tmp_path):
    d = make_disunex_dir(str(tmp_path / "m"), DX_P, 1, sharp=False)
    cfg = load_config(d)
    assert cfg.to_dict() == json.load(open(os.path.join(d, "config.json"))) or cfg.to_dict()["layers"] == DX_P["layers"]
    found = load_model_dir(d)
    check_weights(build_model_skeleton(cfg).expected_tensors(), found, set(), d)
    assert "l3.norm2" not in found                       # a tensor a file may leave out is not written
    del found["l1.mlp.correction"]
    with pytest.raises(WeightError) as e:
        check_weights(build_model_skeleton(cfg).expected_tensors(), found, set(), d)
    assert e.value.missing == ["l1.mlp.correction"]
    for breaker, text in (
            (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
            (lambda c: c["layers"][2].update(weights_of=4), "weights_of"),
            (lambda c: c["layers"][0].update(type="other"), "mixer"),
            (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "feed-forward"),
            (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
            (lambda c: c.pop("postln_alpha"), "postln_alpha"),
            (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top")):
        bad = copy.deepcopy(DX_P)
        breaker(bad)
        with pytest.raises(ConfigError) as e:
            build_model_skeleton(config_from_dict(bad))
        assert text in str(e.value)


def test_the_test_configurations_differ_from_each_other_in_every_size():
    seen = {}
    for name, (cfg, _) in DISUNEX_CONFIGS.items():
        for L in cfg["layers"]:
            m = L["mixer"]
            assert len({m["dim"], m["rot_dim"], m["vdim"]}) >= 2         # never all three alike
        seen[name] = (cfg["width"], cfg["vocab"], cfg["postln_alpha"])
    assert len(set(seen.values())) == len(seen)
