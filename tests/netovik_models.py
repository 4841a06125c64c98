"""Tiny Netovik configurations for the tests, and their model folders.

Sizes differ from layer to layer and between the configurations: head sizes of 8 to 64 that
are no multiples of each other, one to twelve heads, grouped and ungrouped kv heads, windows
of 5 to 70 with 0 to 9 kept first tokens and one layer without a window, one to three norm
groups, embedding scales other than a power of two, one or two experts a token, or all of
them, layers without a feed-forward, bias tables of 6 to 32 rows, attention first, last, twice
in a row or absent.  The random weights are made *sharp* after they are drawn (queries, keys
and routers scaled up, biases and mixing matrices of size one) so that a wrong window edge, a
lost state or a left-out sink moves the logits by far more than bfloat16 rounding.
"""
from __future__ import annotations

import functools
import json
import os

import torch


def wkv(heads, dim, rank=4):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}}


def att(heads, kv_heads, dim, scale, softcap, bias_max, buckets, window=None, keep=0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "softcap": softcap,
         "bias_max": bias_max, "bias_buckets": buckets}
    if window:
        m["mask"] = {"size": window, "keep_first": keep}
    return {"type": "attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(mix, mlp):
    return dict(mix, mlp=mlp)


def model(width, vocab, groups, eps, scale, layers):
    return {"architecture": "Netovik", "width": width, "vocab": vocab, "norm": {"eps": eps, "groups": groups},
            "embedding": {"scale": scale}, "layers": layers}


# attention first and last, a layer without a feed-forward, windows that are no multiple of anything
NV_A = model(64, 300, 2, 1e-6, 0.7, [
    layer(att(4, 2, 16, 0.3, 8.0, 40, 12, window=13, keep=3), dense(72)),
    layer(wkv(4, 16), moe(5, 2, 24)),
    layer(wkv(2, 24, rank=8), None),
    layer(att(3, 3, 8, 0.5, 30.0, 25, 6, window=5, keep=0), moe(5, 2, 24)),
])
# one norm group, one head, every expert chosen (so a long request is compared to its end in bfloat16 too), a window of
# one page and more kept tokens than a page holds
NV_B = model(96, 257, 1, 1e-5, 1.0, [
    layer(wkv(1, 64), moe(3, 3, 16)),
    layer(att(1, 1, 40, 0.2, 5.0, 100, 32, window=8, keep=9), dense(40)),
    layer(wkv(12, 8, rank=16), dense(104)),
])
# two attention layers in a row with different caches, one without a window and with heads of 32 (in bfloat16 its
# prompts run on the matrix cores); both experts chosen; three groups
NV_C = model(72, 128, 3, 1e-4, 1.9, [
    layer(att(12, 4, 8, 0.4, 50.0, 64, 16, window=70, keep=2), moe(2, 2, 16)),
    layer(att(6, 2, 32, 0.18, 12.0, 33, 8), dense(40)),
    layer(wkv(3, 24), dense(48)),
])
# recurrence only; one expert a token
NV_D = model(48, 90, 2, 1e-6, 0.5, [
    layer(wkv(6, 8), dense(56)),
    layer(wkv(2, 32, rank=2), moe(4, 1, 8)),
])
NETOVIK_CONFIGS = {"nvA": (NV_A, 3), "nvB": (NV_B, 5), "nvC": (NV_C, 7), "nvD": (NV_D, 9)}
NETOVIK_PAGE = {"nvA": 16, "nvB": 8, "nvC": 32, "nvD": 16}
NETOVIK_LENGTHS = {"nvA": [1, 2, 12, 13, 14, 40, 61], "nvB": [3, 8, 9, 17, 75, 130], "nvC": [5, 69, 70, 71, 100],
                   "nvD": [1, 2, 33, 80]}

#: factors on the drawn weights by the tensor's last name
SHARP = {"q": 12.0, "k": 12.0, "r": 8.0, "v": 8.0, "g": 8.0, "o": 5.0, "w1": 5.0, "w2": 10.0, "up": 6.0, "down": 6.0,
         "gate": 10.0, "router": 10.0, "embed": 40.0, "rel": 2.0, "talk": 1.0}


def make_netovik_dir(path: str, cfg: dict, seed: int, sharp: bool = True) -> str:
    from safetensors import safe_open
    from safetensors.torch import save_file
    from tffinfer_amd.weights import write_random_model
    write_random_model(path, json.loads(json.dumps(cfg)), seed, dtype="bfloat16")
    if sharp:
        f = os.path.join(path, "model.safetensors")
        W = {}
        with safe_open(f, "pt") as fh:
            for k in fh.keys():
                W[k] = fh.get_tensor(k)
        for k in list(W):
            last = k.split(".")[-1]
            if last in SHARP and W[k].dim() == 2 and ".mu." not in k:
                W[k] = (W[k].float() * SHARP[last]).to(W[k].dtype)
            if last == "talk":
                W[k] = (W[k].float() + torch.eye(W[k].shape[0])).to(W[k].dtype)
        save_file(W, f)
    return path


#: a choice of experts that hangs on less than this much of a router's logit is a close call that bfloat16
#: rounding may turn (the stream that the router reads has drifted by a percent by then, its logits are of
#: size one to five): what follows it in that request is compared in float32 only
CLOSE_CALL = 0.08


@functools.lru_cache(maxsize=None)
def comparable_tokens(model_dir: str, tokens: tuple, dtype: str = "bfloat16") -> int:
    """How many of the tokens come before the sequence's first close call.  In float32 only a first token whose
    recurrence output all but cancels counts as one (the norm over the head then blows rounding up a thousandfold)."""
    import plain_netovik as plain
    cfg, W = plain.load(model_dir)
    if dtype == "float32":
        return plain.first_close_call(cfg, W, list(tokens), 1e-5, sign_share=0.003)
    return plain.first_close_call(cfg, W, list(tokens), CLOSE_CALL)
