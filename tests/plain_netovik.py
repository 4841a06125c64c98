"""Plain, slow implementation of the Netovik decoder, used only by tests.

Whole sequences, no cache, no state slots, no batching, one function per mechanism, float64.
It shares no code with the package: config.json is read with ``json``, the weights with the
``safetensors`` library, and the recurrence is the loop over tokens that its definition is.
"""
from __future__ import annotations

import json
import math
import os

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Rows cut into ``groups`` consecutive parts, each brought to unit root mean square; times w."""
    T, W = x.shape
    return unit_rms(x.reshape(T, groups, W // groups), eps).reshape(T, W) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def shifted(x: torch.Tensor, before=None) -> torch.Tensor:
    """Row t-1 for every row t; zeros (or ``before``) for the first."""
    first = torch.zeros_like(x[:1]) if before is None else before.reshape(1, -1)
    return torch.cat([first, x[:-1]], 0)


def wkv_recurrence(r, k, v, w, u, S=None):
    """r, k, v, w [T, H, D], u [H, D].  o_t[j] = sum_i r_t[i] (S[i, j] + u[i] k_t[i] v_t[j]);
    then S[i, j] <- w_t[i] S[i, j] + k_t[i] v_t[j].  Returns (o [T, H, D], S [H, D, D])."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype) if S is None else S.clone()
    o = torch.zeros(T, H, D, dtype=r.dtype)
    for t in range(T):
        for h in range(H):
            outer = torch.outer(k[t, h], v[t, h])
            o[t, h] = r[t, h] @ (S[h] + u[h].unsqueeze(1) * outer)
            S[h] = w[t, h].unsqueeze(1) * S[h] + outer
    return o, S


def wkv_mixer(m: dict, P: dict, x: torch.Tensor, eps: float, fragile: list | None = None) -> torch.Tensor:
    T, W = x.shape
    H, D = m["heads"], m["dim"]
    xp = shifted(x)
    mix = {s: x + (xp - x) * P[f"mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ P["r"].T).reshape(T, H, D)
    k = (mix["k"] @ P["k"].T).reshape(T, H, D)
    v = (mix["v"] @ P["v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ P["g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mix["w"] @ P["w1"].T) @ P["w2"].T + P["w0"])).reshape(T, H, D)
    o, _ = wkv_recurrence(r, k, v, w, P["u"])
    if fragile is not None:
        # A sequence's first token meets an empty state: o_0 = c v_0 with c = sum_i r_i u_i k_i, and the
        # norm over the head makes of it sign(c) times the unit vector of v_0.  How far c is from zero,
        # as a share of the sum of its terms' magnitudes (the smallest over the heads):
        terms = r[0] * P["u"] * k[0]
        share = torch.full((T,), float("inf"), dtype=x.dtype)
        share[0] = (terms.sum(-1).abs() / terms.abs().sum(-1)).min()
        fragile.append(share)
    y = unit_rms(o, eps).reshape(T, H * D) * P["norm"] * gate
    return y @ P["o"].T


def distance_bucket(n: int, B: int, Dmax: int) -> int:
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(Dmax / half) * (B - half))))


def sees(i: int, j: int, window, keep_first: int) -> bool:
    return j <= i and (window is None or i - j < window or j < keep_first)


def softmax_plus_one(s: torch.Tensor) -> torch.Tensor:
    """exp(s_j) / (1 + sum_j exp(s_j)) over the last dimension; -inf entries get 0."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attend(qn, kn, vals, scale, cap, rel, bias_max, talk, window, keep, sink=True, first_pos=0):
    """qn [Tq, H, D] (the queries are the last Tq positions), kn, vals [T, G, D].  Scores are capped,
    get the bias of their distance's bucket, are mixed between heads, masked, and weighed by a
    softmax with 1 in the denominator.  Returns [Tq, H, D]."""
    Tq, H, D = qn.shape
    T, G, _ = kn.shape
    off = T - Tq
    raw = torch.zeros(H, Tq, T, dtype=qn.dtype)
    for g in range(H):
        dots = (qn[:, g] @ kn[:, g // (H // G)].T) * scale
        raw[g] = cap * torch.tanh(dots / cap) if cap else dots
    if rel is not None:
        for i in range(Tq):
            for j in range(off + i + 1):
                raw[:, i, j] += rel[distance_bucket(off + i - j, rel.shape[0], bias_max)]
    mixed = torch.einsum("hg,gij->hij", talk, raw) if talk is not None else raw
    s = torch.full((H, Tq, T), float("-inf"), dtype=qn.dtype)
    for i in range(Tq):
        for j in range(T):
            if sees(off + i, j, window, keep):
                s[:, i, j] = mixed[:, i, j]
    if sink:
        p = softmax_plus_one(s)
    else:
        p = torch.softmax(s, -1)
    out = torch.zeros(Tq, H, D, dtype=qn.dtype)
    for h in range(H):
        out[:, h] = p[h] @ vals[:, h // (H // G)]
    return out


def mixed_attention(m: dict, P: dict, x: torch.Tensor, eps: float) -> torch.Tensor:
    T, W = x.shape
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    q = (x @ P["q"].T + P["q.b"]).reshape(T, H, D)
    k = (x @ P["k"].T + P["k.b"]).reshape(T, G, D)
    mask = m.get("mask")
    out = attend(unit_rms(q, eps), unit_rms(k, eps), k, m["scale"], m["softcap"], P["rel"], m["bias_max"], P["talk"],
                 mask["size"] if mask else None, mask.get("keep_first", 0) if mask else 0)      # the values are the keys as projected
    return out.reshape(T, H * D) @ P["o"].T


def dense_ff(P: dict, x: torch.Tensor) -> torch.Tensor:
    return (silu(x @ P["gate"].T) * (x @ P["up"].T)) @ P["down"].T


def router_scores(P: dict, x: torch.Tensor) -> torch.Tensor:
    return torch.softmax(x @ P["router"].T, -1)


def moe_ff(mlp: dict, P: dict, x: torch.Tensor, margins: list | None = None) -> torch.Tensor:
    top = mlp["router"]["top"]
    s = router_scores(P, x)
    order = torch.argsort(s, dim=-1, descending=True, stable=True)
    if margins is not None and top < s.shape[1]:
        srt = torch.log(torch.gather(s, 1, order))       # (differences of these are differences of the router's logits)
        margins.append(srt[:, top - 1] - srt[:, top])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in order[t, :top].tolist():
            y = silu(P[f"e{e}.gate"] @ x[t]) * (P[f"e{e}.up"] @ x[t])
            out[t] += s[t, e] * (P[f"e{e}.down"] @ y)
    return out


def load(model_dir: str):
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    W = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), "pt") as fh:
        for k in fh.keys():
            t = fh.get_tensor(k)
            W[k] = t.double() if t.is_floating_point() else t
    return cfg, W


def layer_tensors(W: dict, i: int, part: str) -> dict:
    pre = f"l{i}.{part}."
    return {k[len(pre):]: v for k, v in W.items() if k.startswith(pre)}


def forward(cfg: dict, W: dict, tokens, streams: list | None = None, margins: list | None = None,
            fragile: list | None = None) -> torch.Tensor:
    """float64 logits [T, vocab]; ``streams`` gets the stream after every layer (after the sum over
    depth), ``margins`` per mixture and token the gap between the router's logits of the last chosen and the
    first left-out expert, ``fragile`` per recurrence layer and token how far the output is from
    changing its sign (the first token's: see ``wkv_mixer``)."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    outputs = [x]
    for i, L in enumerate(cfg["layers"]):
        P = layer_tensors(W, i, "mix")
        a = wkv_mixer(L["mixer"], P, x, eps, fragile) if L["type"] == "wkv" else mixed_attention(L["mixer"], P, x, eps)
        x = x + group_norm(a, W[f"l{i}.norm1"], groups, eps)
        if L.get("mlp") is not None:
            F = layer_tensors(W, i, "mlp")
            f = dense_ff(F, x) if L["mlp"]["kind"] == "dense" else moe_ff(L["mlp"], F, x, margins)
            x = x + group_norm(f, W[f"l{i}.norm2"], groups, eps)
        outputs.append(x)
        x = sum(W[f"l{i}.dwa"][j] * outputs[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x.clone())
    return group_norm(x, W["final.norm"], groups, eps) @ W["embed"].T


def first_close_call(cfg, W, tokens, gap: float, sign_share: float = 0.03) -> int:
    """The first position at which some mixture's choice hangs on less than ``gap`` of a logit
    (len(tokens) if none does): from there on a run in fewer bits may have chosen otherwise.
    Also the first token, if a recurrence layer's output for it is within ``sign_share`` of changing its sign."""
    margins, fragile = [], []
    forward(cfg, W, tokens, margins=margins, fragile=fragile)
    close = torch.zeros(len(tokens), dtype=torch.bool)
    if margins:
        close |= torch.stack(margins).min(0).values < gap
    if fragile:
        close |= torch.stack(fragile).min(0).values < sign_share
    close = close.nonzero()
    return int(close[0]) if len(close) else len(tokens)


def greedy(cfg, W, prompt, n: int) -> list:
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, W, toks)[-1])))
    return toks[len(prompt):]
