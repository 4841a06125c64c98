"""Attention whose heads exchange their scores before the softmax, with a learned bias by
distance, a soft cap, a window that keeps a request's first tokens, and keys that serve as values."""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError
from .base import KVCacheSpec, Mixer, WeightSpec, register_mixer, to_device


def distance_buckets(num_buckets: int, max_distance: int) -> torch.Tensor:
    """The bucket of every distance 0 .. max_distance (int64 [max_distance + 1]); larger distances
    fall into the last bucket.  The first half of the buckets holds one distance each; the
    second half divides the distances up to ``max_distance`` evenly by their logarithm:

        bucket(n) = n                                                        n < B/2
                  = min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) * (B - B/2)))   otherwise
    """
    B, D = int(num_buckets), int(max_distance)
    half = B // 2
    if half < 1 or D <= half:
        raise ConfigError(f"distance bias: {B} buckets up to a distance of {D}: the largest distance "
                          "must lie beyond the first half of the buckets")
    n = torch.arange(D + 1, dtype=torch.float32)
    far = half + torch.floor(torch.log(n.clamp(min=1) / half) / math.log(D / half) * (B - half)).to(torch.int64)
    return torch.where(n < half, n.to(torch.int64), far.clamp(max=B - 1))


@register_mixer("mixed_head_attention")
class MixedHeadAttention(Mixer):
    """q = Wq x + bq, k = Wk x + bk per head; the values are the keys as projected (there is no
    value matrix); q and k are divided by their root mean square over the head (no weight).

        s_g(i, j) = cap * tanh(scale * q_g(i) . k_g(j) / cap) + rel[bucket(i - j), g]
        s'_h = sum_g talk[h, g] * s_g
        visible: j <= i and (i - j < window or j < keep_first)
        p_h(i, j) = exp(s'_h(i, j)) / (1 + sum over the visible j' of exp(s'_h(i, j')))
        out = Wo [ sum_j p_h(i, j) k_kv(h)(j) ]_h

    Query head h reads kv head h // (heads / kv_heads).  Positions enter through the bias alone.
    Every term is an argument: ``softcap`` 0 or None leaves the cap out, ``bias_max`` None the bias,
    ``talk`` False the exchange between heads, ``sink`` False the 1 in the denominator, ``window``
    0 the window, ``qk_bias`` False the biases.  ``bias_buckets`` (the rows of the bias table) may
    be left open: the tensor gives it.
    """

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 value_dim: int | None = None, softcap: float | None = None, bias_max: int | None = None,
                 bias_buckets: int | None = None, talk: bool = True, window: int = 0, keep_first: int = 0,
                 sink: bool = True, qk_bias: bool = True, qk_norm_eps: float = 1e-6):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.scale = float(scale)
        self.softcap = float(softcap or 0.0)
        self.bias_max = None if bias_max is None else int(bias_max)
        self.bias_buckets = None if bias_buckets is None else int(bias_buckets)
        self.has_talk = bool(talk)
        self.window = int(window or 0)
        self.keep_first = int(keep_first or 0) if self.window > 0 else 0
        self.has_sink = bool(sink)
        self.has_qk_bias = bool(qk_bias)
        self.qk_norm_eps = float(qk_norm_eps)
        if min(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim) <= 0:
            raise ConfigError("mixed-head attention: sizes must be positive")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"mixed-head attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if value_dim is not None and int(value_dim) != self.head_dim:
            raise ConfigError(f"mixed-head attention: the values are the keys, so a value size of {value_dim} "
                              f"must equal the key size of {self.head_dim}")
        if self.window < 0 or self.keep_first < 0 or self.softcap < 0:
            raise ConfigError("mixed-head attention: window, kept tokens and soft cap must not be negative")
        self.w_qk = self.w_o = self.q_bias = self.k_bias = self.bias_by_distance = self.talk = None

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window, self.keep_first)

    def flops_per_query_key_pair(self):
        return 4 * self.num_heads * self.head_dim + (2 * self.num_heads * self.num_heads if self.has_talk else 0)

    def weight_specs(self):
        W, H, G, D = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        specs = {"q": WeightSpec((H * D, W)), "k": WeightSpec((G * D, W)), "o": WeightSpec((W, H * D))}
        if self.has_qk_bias:
            specs["q.b"] = WeightSpec((H * D,), "vector")
            specs["k.b"] = WeightSpec((G * D,), "vector")
        if self.bias_max is not None:
            specs["rel"] = WeightSpec((self.bias_buckets, H), "vector")
        if self.has_talk:
            specs["talk"] = WeightSpec((H, H), "vector")
        return specs

    def load_weights(self, weights, dtype, device):
        f32 = lambda t: t.to(torch.float32).contiguous().to(device)      # noqa: E731
        self.w_qk = to_device(torch.cat([weights["q"], weights["k"].to(weights["q"].dtype)], 0), dtype, device)
        self.w_o = to_device(weights["o"], dtype, device)
        if self.has_qk_bias:
            self.q_bias, self.k_bias = f32(weights["q.b"]), f32(weights["k.b"])
        if self.bias_max is not None:
            rel = weights["rel"].to(torch.float32)
            # the table by distance, its last row for every larger distance
            self.bias_by_distance = f32(rel[distance_buckets(rel.shape[0], self.bias_max)])
        if self.has_talk:
            self.talk = f32(weights["talk"])

    def forward(self, ctx, x):
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        H, G, D = self.num_heads, self.num_kv_heads, self.head_dim
        qk = ops.linear(x, self.w_qk, out_dtype=torch.float32)
        q = ops.qk_bias_norm_store(qk, self.q_bias, self.k_bias, self.qk_norm_eps, H, G, D, kv)
        o = ops.mixed_attention(q, H, G, D, kv, b, self.scale, self.softcap, self.bias_by_distance, self.talk,
                                self.window, self.keep_first, self.has_sink)
        return ops.linear(o, self.w_o, out_dtype=torch.float32, partials=True)
