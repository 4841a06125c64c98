"""Tiny Disunex configurations for the tests, and their model folders.

The sizes differ from layer to layer and from each other (head size, rotated size and value
size all different; one, two and three experts a token; an alpha of 1 and others; a layer
without a window, one without a feed-forward; heads that fill more than one column tile of
the matrix-core attention; sizes that are no multiples of 8).  The random weights are made
*sharp* after they are drawn: queries, keys and routers are scaled up so that attention
weights and expert choices are far from uniform and the sinks carry weight; with the plain
N(0, 0.02) matrices a wrong window edge or a missing sink would move the logits by less than
the bfloat16 rounding does.
"""
from __future__ import annotations

import functools
import json
import os

import torch


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, window=None, base=10000.0, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        m["mask"] = {"size": window}
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def layer(mix, mlp, weights_of=None):
    L = {"type": "latent_attention", "mixer": mix, "mlp": mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


_P = mixer(4, 16, 8, 24, 40, 0.2, window=12)
_Q = mixer(2, 24, 16, 8, 24, 0.15, window=20, base=500.0)
DX_P = {"architecture": "Disunex", "width": 64, "vocab": 300, "postln_alpha": 2.0, "norm": {"eps": 1e-6}, "layers": [
    layer(_P, dense(136)),
    layer(_Q, moe(5, 2, 40, 0.7)),
    layer(_P, dense(136), weights_of=0),
    layer(mixer(4, 8, 8, 16, 56, 0.3), None),                   # no window, no feed-forward
    layer(_Q, moe(5, 2, 40, 0.7), weights_of=1),
]}
# alpha 1, one expert a token, an odd vocabulary, a window that is no multiple of anything
DX_Q = {"architecture": "Disunex", "width": 96, "vocab": 257, "postln_alpha": 1.0, "norm": {"eps": 1e-5}, "layers": [
    layer(mixer(5, 8, 4, 12, 100, 0.35, window=37, base=20000.0), moe(3, 1, 24, 1.5)),
    layer(mixer(3, 32, 24, 40, 16, 0.1, window=64), dense(72)),
    layer(mixer(3, 32, 24, 40, 16, 0.1, window=64), dense(72), weights_of=1),
]}
# twenty heads (two column tiles), a key of 160 elements (a cache padded to 192 in bfloat16), three experts
# a token, a rotation of part of the rotated size only
DX_R = {"architecture": "Disunex", "width": 72, "vocab": 128, "postln_alpha": 3.5, "norm": {"eps": 1e-6}, "layers": [
    layer(mixer(20, 8, 10, 8, 150, 0.25, window=33, dims=6), moe(6, 3, 16, 0.5)),
    layer(mixer(1, 40, 2, 48, 30, 0.2, window=5), dense(40)),
]}
# sizes that are no multiples of 8
DX_S = {"architecture": "Disunex", "width": 60, "vocab": 101, "postln_alpha": 0.5, "norm": {"eps": 1e-4}, "layers": [
    layer(mixer(3, 10, 6, 14, 20, 0.3, window=9), dense(50)),
    layer(mixer(3, 10, 6, 14, 20, 0.3, window=9), dense(50), weights_of=0),
    layer(mixer(2, 6, 2, 5, 11, 0.4), moe(4, 2, 12, 2.0)),
]}
# a key of 288 elements, beyond what the matrix-core attention takes (the general kernel in both types),
# and a mixture in which every expert is chosen
DX_T = {"architecture": "Disunex", "width": 48, "vocab": 90, "postln_alpha": 1.5, "norm": {"eps": 1e-5}, "layers": [
    layer(mixer(2, 8, 8, 16, 280, 0.3, window=10), moe(2, 2, 16, 1.0), weights_of=1),
    layer(mixer(2, 8, 8, 16, 280, 0.3, window=10), moe(2, 2, 16, 1.0)),
]}
DISUNEX_CONFIGS = {"dxP": (DX_P, 3), "dxQ": (DX_Q, 5), "dxR": (DX_R, 7), "dxS": (DX_S, 9), "dxT": (DX_T, 13)}
DISUNEX_PAGE = {"dxP": 16, "dxQ": 8, "dxR": 16, "dxS": 32, "dxT": 16}
DISUNEX_LENGTHS = {"dxP": [1, 2, 11, 12, 13, 40, 61], "dxQ": [3, 36, 37, 38, 75, 130], "dxR": [5, 33, 34, 70],
                   "dxS": [2, 9, 10, 33, 80], "dxT": [1, 10, 11, 50]}

#: factors on the drawn weights by the tensor's last name
SHARP = {"q": 10.0, "uk": 10.0, "dkv": 6.0, "g": 10.0, "uv": 5.0, "o": 5.0, "up": 6.0, "down": 6.0, "gate": 10.0,
         "router": 8.0}


def make_disunex_dir(path: str, cfg: dict, seed: int, sharp: bool = True) -> str:
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
        g = torch.Generator().manual_seed(seed)
        for k in list(W):
            last = k.split(".")[-1]
            if last in SHARP and W[k].dim() == 2:
                W[k] = (W[k].float() * SHARP[last]).to(W[k].dtype)
            elif last == "sink":
                W[k] = (1.5 + torch.randn(W[k].shape, generator=g)).to(W[k].dtype)
        save_file(W, f)
    return path


#: a choice of experts that hangs on less than this is a close call that bfloat16 rounding may
#: turn (the router's scores move by some 1e-3 when its input is rounded): no test rests on one
MIN_MARGIN = 0.004


@functools.lru_cache(maxsize=None)
def clear_tokens(model_dir: str, n: int, vocab: int, seed: int) -> tuple:
    """``n`` random tokens whose sequence makes no close call in any mixture of experts: the
    first of the seeds seed, seed + 1000, ... that does."""
    import plain_disunex as plain
    from helpers import random_tokens
    cfg, W = plain.load(model_dir)
    for k in range(100):
        toks = random_tokens(n, vocab, seed + 1000 * k)
        if plain.smallest_margin(cfg, W, toks) >= MIN_MARGIN:
            return tuple(toks)
    raise AssertionError(f"no sequence of {n} tokens without a close call among 100 seeds")
