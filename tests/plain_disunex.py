"""Plain, slow implementation of the Disunex decoder, used only by tests.

Whole sequences, no cache, no batching, one function per mechanism, float64.  It shares no
code with the package: config.json is read with ``json``, the weights with the
``safetensors`` library.  The attention is written the long way round (every head's keys and
values are expanded from the latent vectors), where the package keeps the latent vectors and
moves the expansion to the query's side.
"""
from __future__ import annotations

import json
import math
import os

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight lies around zero: unit(x) * (1 + w)."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def rotate_pairs(x: torch.Tensor, positions, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., n]: the first ``dims`` elements are rotated in pairs (2i, 2i+1) by the angle
    p * base^(-2i/dims); the rest pass."""
    out = x.clone()
    for t, p in enumerate(positions):
        for i in range(dims // 2):
            a = float(p) * base ** (-2.0 * i / dims)
            u, v = x[t, ..., 2 * i].clone(), x[t, ..., 2 * i + 1].clone()
            out[t, ..., 2 * i] = u * math.cos(a) - v * math.sin(a)
            out[t, ..., 2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def softmax_with_sink(scores: torch.Tensor, visible: torch.Tensor, sink) -> torch.Tensor:
    """scores [T, S], visible [T, S] bool; weights e^s / (sum over the visible e^s + e^sink):
    the sink has no key and no value and counts once (sink None: a plain softmax)."""
    s = scores.masked_fill(~visible, float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.as_tensor(sink, dtype=scores.dtype).reshape(1, 1))
    e = torch.exp(s - m)                       # 0 where nothing is seen
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - m)
    w = e / den
    return w


def visibility(T: int, window) -> torch.Tensor:
    """Position i sees j iff 0 <= i - j, and i - j < window if there is one."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = (i - j) >= 0
    if window:
        vis = vis & ((i - j) < window)
    return vis


def latent_attention(h: torch.Tensor, m: dict, W: dict, eps: float, positions=None) -> torch.Tensor:
    """h [T, width]; m: the mixer's entry of the configuration; W: its tensors by short name."""
    T = h.shape[0]
    H, dim, rd, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = list(range(T)) if positions is None else positions
    q = (h @ W["q"].T).view(T, H, dim + rd)
    dkv = h @ W["dkv"].T
    c = norm_plain(dkv[:, :R], W["dkv.norm"], eps)
    kr = dkv[:, R:]
    if rd:
        base, dims = m["rot"]["base"], m["rot"].get("dims", rd)
        qr = rotate_pairs(q[:, :, dim:], positions, base, dims)
        kr = rotate_pairs(kr, positions, base, dims)
    else:
        qr = q[:, :, dim:]
    kn = (c @ W["uk"].T).view(T, H, dim)
    v = (c @ W["uv"].T).view(T, H, vd)
    window = (m.get("mask") or {}).get("size")
    vis = visibility(T, window)
    heads = []
    for hh in range(H):
        s = (q[:, hh, :dim] @ kn[:, hh].T + qr[:, hh] @ kr.T) * m["scale"]
        p = softmax_with_sink(s, vis, W["sink"][hh] if "sink" in W else None)
        heads.append(p @ v[:, hh])
    o = torch.cat(heads, -1)
    if "g" in W:
        o = o * torch.sigmoid(h @ W["g"].T)
    return o @ W["o"].T


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def dense_ff(h, W):
    return gelu_erf(h @ W["up"].T) @ W["down"].T


def route(h, router, correction, top):
    """(chosen experts [T, top], weights [T, top]): scores s = sigmoid(router h); the choice
    goes by s + correction, the weights by s alone, divided by their sum (+ 1e-20)."""
    s = torch.sigmoid(h @ router.T)
    choice = s + (correction if correction is not None else 0.0)
    idx = torch.zeros(h.shape[0], top, dtype=torch.long)
    wts = torch.zeros(h.shape[0], top, dtype=h.dtype)
    for t in range(h.shape[0]):
        order = sorted(range(s.shape[1]), key=lambda e: (-float(choice[t, e]), e))[:top]
        tot = sum(float(s[t, e]) for e in order) + 1e-20
        for k, e in enumerate(order):
            idx[t, k] = e
            wts[t, k] = s[t, e] / tot
    return idx, wts


def expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def choice_margins(h, router, correction, top) -> torch.Tensor:
    """Per token: by how much the last chosen expert's corrected score exceeds the first one
    left out (inf where all are chosen).  A small margin is a close call: rounding may turn it."""
    c = torch.sigmoid(h @ router.T) + (correction if correction is not None else 0.0)
    srt = c.sort(-1, descending=True).values
    if top >= srt.shape[1]:
        return torch.full((h.shape[0],), float("inf"), dtype=h.dtype)
    return srt[:, top - 1] - srt[:, top]


def moe_ff(h, m, W, margins: list | None = None):
    if margins is not None:
        margins.append(choice_margins(h, W["router"], W.get("correction"), m["router"]["top"]))
    idx, wts = route(h, W["router"], W.get("correction"), m["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            out[t] += wts[t, k] * expert(h[t], W[f"e{e}.gate"], W[f"e{e}.up"], W[f"e{e}.down"], m["expert"]["limit"])
    return out


def sub(W: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def load(model_dir: str):
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    W = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), "pt") as f:
        for k in f.keys():
            W[k] = f.get_tensor(k).to(torch.float64)
    return cfg, W


def forward(cfg: dict, W: dict, tokens, stream_after_layers: list | None = None,
            margins: list | None = None) -> torch.Tensor:
    """float64 logits [T, vocab] of a whole sequence.  ``margins`` collects, per call of a
    mixture of experts, the tokens' choice margins."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = W["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % L.get("weights_of", i)
        x = norm_around_zero(alpha * x + latent_attention(x, L["mixer"], sub(W, p + "mix."), eps), W[p + "norm1"], eps)
        mlp = L.get("mlp")
        if mlp is not None:
            f = dense_ff(x, sub(W, p + "mlp.")) if mlp["kind"] == "dense" else moe_ff(x, mlp, sub(W, p + "mlp."), margins)
            x = norm_around_zero(alpha * x + f, W[p + "norm2"], eps)
        elif p + "norm2" in W:
            x = norm_around_zero(alpha * x, W[p + "norm2"], eps)
        if stream_after_layers is not None:
            stream_after_layers.append(x.clone())
    return norm_around_zero(x, W["final.norm"], eps) @ W["embed"].T


def greedy(cfg, W, prompt, n_new: int) -> list[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(cfg, W, toks)[-1])))
    return toks[len(prompt):]


def smallest_margin(cfg, W, tokens) -> float:
    """The closest call any token of the sequence makes in any mixture of experts."""
    margins = []
    forward(cfg, W, tokens, margins=margins)
    return min((float(m.min()) for m in margins), default=float("inf"))
