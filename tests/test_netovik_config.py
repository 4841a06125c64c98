"""The Netovik configuration: what its config.json turns into, what is refused, and what its
cache asks of the cache manager (all on the CPU)."""
import copy
import json
import os

import pytest
import torch

import plain_netovik as plain
from netovik_models import NETOVIK_CONFIGS, NV_A, NV_B, NV_C, NV_D, make_netovik_dir
from tffinfer_amd.cache.manager import CacheManager
from tffinfer_amd.cache.sizing import min_window_pages, window_pool_pages
from tffinfer_amd.config.base import ConfigError, LayerCall
from tffinfer_amd.models import build_model_skeleton, config_from_dict, load_config
from tffinfer_amd.parts import (GroupRMSNorm, KVCacheSpec, MixedHeadAttention, NoFeedForward, OutputNormBlock,
                                RoutedExperts, SwiGLU, WKVMixer)
from tffinfer_amd.parts.mixed_attention import distance_buckets
from tffinfer_amd.weights.loader import WeightError, check_weights
from tffinfer_amd.weights.safetensors_io import load_model_dir


def test_every_size_and_constant_comes_from_the_file():
    cfg = config_from_dict(copy.deepcopy(NV_A))
    model = build_model_skeleton(cfg)
    assert cfg.layer_schedule() == [LayerCall(i, i) for i in range(4)]
    assert [type(b.mixer) for b in model.blocks] == [MixedHeadAttention, WKVMixer, WKVMixer, MixedHeadAttention]
    assert [type(b.feed_forward) for b in model.blocks] == [SwiGLU, RoutedExperts, NoFeedForward, RoutedExperts]
    assert all(isinstance(b, OutputNormBlock) and b.depth == i and b.depths == 5 for i, b in enumerate(model.blocks))
    assert model.embedding.scale == 0.7
    a = model.blocks[0].mixer
    assert (a.num_heads, a.num_kv_heads, a.head_dim, a.scale, a.softcap, a.bias_max, a.window, a.keep_first) == \
        (4, 2, 16, 0.3, 8.0, 40, 13, 3)
    assert a.cache_spec() == KVCacheSpec(2, 16, 13, 3) and model.blocks[3].mixer.cache_spec() == KVCacheSpec(3, 8, 5, 0)
    w = model.blocks[2].mixer
    assert (w.num_heads, w.head_dim, w.decay_rank) == (2, 24, 8)
    assert w.cache_spec() is None and w.state_spec().shape == (2 * 24 * 24 + 64,) and w.state_spec().dtype == torch.float32
    ff = model.blocks[1].feed_forward
    assert (ff.num_experts, ff.top, ff.intermediate_size, ff.router_softmax, ff.up_offset, ff.act_alpha) == (5, 2, 24, True, 0.0, 1.0)
    assert ff.limit == float("inf") and not ff.has_correction
    n = model.final_norm
    assert isinstance(n, GroupRMSNorm) and (n.groups, n.eps, n.size) == (2, 1e-6, 64)
    # a layer without a window keeps every key; kv heads default to the heads
    c = build_model_skeleton(config_from_dict(copy.deepcopy(NV_C)))
    assert c.blocks[1].mixer.cache_spec() == KVCacheSpec(2, 32, 0, 0)
    m = copy.deepcopy(NV_C)
    del m["layers"][0]["mixer"]["kv_heads"]
    assert build_model_skeleton(config_from_dict(m)).blocks[0].mixer.num_kv_heads == 12


def test_tensor_names_follow_the_files():
    names = build_model_skeleton(config_from_dict(copy.deepcopy(NV_A))).expected_tensors()
    for n in ("embed", "final.norm", "l0.norm1", "l0.norm2", "l0.dwa", "l3.dwa", "l0.mix.q", "l0.mix.q.b", "l0.mix.k",
              "l0.mix.k.b", "l0.mix.rel", "l0.mix.talk", "l0.mix.o", "l0.mlp.gate", "l0.mlp.up", "l0.mlp.down",
              "l1.mix.mu.r", "l1.mix.mu.w", "l1.mix.r", "l1.mix.g", "l1.mix.w1", "l1.mix.w2", "l1.mix.w0", "l1.mix.u",
              "l1.mix.norm", "l1.mix.o", "l1.mlp.router", "l1.mlp.e4.gate", "l1.mlp.e0.down", "l2.norm1"):
        assert n in names, n
    assert not any(n.startswith("head") or n.endswith(("mix.v.b", "correction", "sink")) for n in names)
    assert "l0.mix.v" not in names                      # the values are the keys: no value matrix
    assert names["l2.norm2"].optional and not names["l0.norm2"].optional
    assert names["l0.dwa"].shape == (2,) and names["l3.dwa"].shape == (5,)
    assert names["l0.mix.k"].shape == (32, 64) and names["l0.mix.rel"].shape == (12, 4) and names["l0.mix.talk"].shape == (4, 4)
    assert names["l1.mix.u"].shape == (4, 16) and names["l2.mix.w1"].shape == (8, 64) and names["l2.mix.w2"].shape == (48, 8)


def test_sizes_that_the_tensors_give_are_left_open(tmp_path):
    """A file that does not say how many rows its bias table has, or how wide its decay's inner product is,
    loads: the tensors' shapes say it."""
    d = make_netovik_dir(str(tmp_path / "m"), NV_A, 1, sharp=False)
    raw = json.load(open(os.path.join(d, "config.json")))
    for L in raw["layers"]:
        L["mixer"].pop("bias_buckets", None)
        L["mixer"].pop("decay_rank", None)
    cfg = config_from_dict(raw)
    names = build_model_skeleton(cfg).expected_tensors()
    assert names["l0.mix.rel"].shape == (None, 4) and names["l1.mix.w1"].shape == (None, 64)
    found = load_model_dir(d)
    check_weights(names, found, set(), d)
    model = build_model_skeleton(cfg)
    model.load_tensors(found, torch.float32, "cpu")
    assert model.blocks[0].mixer.bias_by_distance.shape == (41, 4)      # distances 0 .. bias_max, the last for all beyond
    found["l0.mix.rel"] = found["l0.mix.rel"][:, :3]
    with pytest.raises(WeightError):
        check_weights(names, found, set(), d)


def test_round_trip_and_refusals(tmp_path):
    d = make_netovik_dir(str(tmp_path / "m"), NV_A, 1, sharp=False)
    cfg = load_config(d)
    assert cfg.to_dict()["layers"] == NV_A["layers"] and cfg.to_dict()["embedding"] == {"scale": 0.7}
    found = load_model_dir(d)
    check_weights(build_model_skeleton(cfg).expected_tensors(), found, set(), d)
    assert "l2.norm2" not in found                       # a tensor a file may leave out is not written
    del found["l1.mix.mu.g"]
    with pytest.raises(WeightError) as e:
        check_weights(build_model_skeleton(cfg).expected_tensors(), found, set(), d)
    assert e.value.missing == ["l1.mix.mu.g"]
    for breaker, text in (
            (lambda c: c["layers"][0].update(type="other"), "mixer"),
            (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "feed-forward"),
            (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
            (lambda c: c["layers"][0]["mixer"].update(vdim=24), "values are the keys"),
            (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv heads"),
            (lambda c: c["layers"][1]["mixer"].update(dim=300), "128"),
            (lambda c: c["norm"].update(groups=5), "groups"),
            (lambda c: c.update(embedding=3), "embedding"),
            (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top")):
        bad = copy.deepcopy(NV_A)
        breaker(bad)
        with pytest.raises(ConfigError) as e:
            build_model_skeleton(config_from_dict(bad))
        assert text in str(e.value), text


def test_the_buckets_of_distances():
    for B, Dmax in ((32, 120), (6, 25), (16, 64), (8, 33), (12, 40), (10, 50)):
        got = distance_buckets(B, Dmax).tolist()
        assert got == [plain.distance_bucket(n, B, Dmax) for n in range(Dmax + 1)]
        assert got[:B // 2] == list(range(B // 2)) and got[-1] == B - 1 and sorted(got) == got
    with pytest.raises(ConfigError):
        distance_buckets(16, 8)


def test_a_window_gives_pages_back_but_keeps_those_of_the_first_tokens():
    spec = KVCacheSpec(2, 16, 20, 9)
    cache = CacheManager([(0, True, spec, None)], page_size=8, num_pages=12, max_seqs=2)
    cache.add_request("a")
    for n in (5, 30, 1, 1, 40, 3):
        cache.reserve("a", n)
        cache.commit("a", n)
        cache.check()
        count = cache.num_tokens("a")
        table = cache.block_table(0, "a")
        held = [b for b, p in enumerate(table) if p >= 0]
        first_needed = max(0, count - 20 + 1) // 8
        assert held == sorted(set(range(min(2, len(table)))) | set(range(first_needed, len(table))))
    cache.release("a")
    assert cache.groups[0].pool.num_used == 0
    assert min_window_pages(20, 8, 9) == min_window_pages(20, 8) + 2
    assert window_pool_pages(20, 8, 4, 64, 9) == window_pool_pages(20, 8, 4, 64) + 4 * 2


def test_the_test_configurations_differ_from_each_other():
    seen = set()
    for name, (cfg, _) in NETOVIK_CONFIGS.items():
        key = (cfg["width"], cfg["vocab"], cfg["norm"]["groups"], cfg["embedding"]["scale"], len(cfg["layers"]))
        assert key not in seen
        seen.add(key)
    assert {L["type"] for L in NV_D["layers"]} == {"wkv"} and NV_B["layers"][1]["mixer"]["mask"]["keep_first"] > 8
