"""A mixer that carries a matrix of state per head instead of keys and values (time mixing in
the manner of RWKV)."""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from .base import Mixer, StateSpec, WeightSpec, register_mixer, to_device


@register_mixer("wkv")
class WKVMixer(Mixer):
    """With x the token's row of the stream and x' the row of the token before it (zeros before
    a request's first token), every projection reads a mix of the two of its own:

        m_s = x + (x' - x) * mu_s                          s in r, k, v, g, w
        r, k, v = Wr m_r, Wk m_k, Wv m_v                   (heads x dim)
        w = exp(-exp(Ww2 tanh(Ww1 m_w) + w0))              (a decay per head and key channel)
        o = (S + diag(u) k v^T)^T r;   S <- diag(w) S + k v^T      (per head, S starts at zero)
        out = Wo [ o / rms_head(o) * norm * silu(Wg m_g) ]

    S and the last token's x are the request's state (float32), one row of the state tensor:
    [heads * dim * dim | hidden].  Mixes, decay, recurrence and the norm over each head are
    float32; the projections run in the activation type with float32 sums.

    The mixer reads the float32 stream itself (``reads_stream``), not a copy in the
    activation type.  ``decay_rank`` (the inner size of the decay's two matrices) may be left
    open: the tensors then give it.
    """

    graph_safe = True
    #: the block hands this mixer the float32 residual stream
    reads_stream = True

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float = 1e-6,
                 decay_rank: int | None = None):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.norm_eps = float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        if self.hidden_size <= 0 or self.num_heads <= 0 or not 0 < self.head_dim <= 128:
            raise ConfigError(f"wkv: {num_heads} heads of {head_dim} on rows of {hidden_size} "
                              "(a head has up to 128 channels)")
        self.mu = self.w0 = self.u = self.norm = None
        self.w_r = self.w_k = self.w_v = self.w_g = self.w_w1 = self.w_w2 = self.w_o = None

    @property
    def inner(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def prev_offset(self) -> int:
        """Where the last token's row lies in a request's state row, behind the heads' matrices."""
        return self.inner * self.head_dim

    def state_spec(self):
        return StateSpec((self.prev_offset + self.hidden_size,), torch.float32)

    def weight_specs(self):
        W, N = self.hidden_size, self.inner
        specs = {f"mu.{s}": WeightSpec((W,), "unit_interval") for s in self.MIXES}
        for s in ("r", "k", "v", "g"):
            specs[s] = WeightSpec((N, W))
        specs["w1"] = WeightSpec((self.decay_rank, W))
        specs["w2"] = WeightSpec((N, self.decay_rank))
        specs["w0"] = WeightSpec((N,), "decay_log")
        specs["u"] = WeightSpec((self.num_heads, self.head_dim), "vector")
        specs["norm"] = WeightSpec((N,), "norm")
        specs["o"] = WeightSpec((W, N))
        return specs

    def load_weights(self, weights, dtype, device):
        f32 = lambda t: t.to(torch.float32).contiguous().to(device)      # noqa: E731
        self.mu = f32(torch.stack([weights[f"mu.{s}"].to(torch.float32) for s in self.MIXES], 0))
        self.w_r, self.w_k, self.w_v, self.w_g = (to_device(weights[s], dtype, device) for s in ("r", "k", "v", "g"))
        if weights["w1"].shape[0] != weights["w2"].shape[1]:
            raise ConfigError(f"wkv: the decay's matrices {tuple(weights['w1'].shape)} and "
                              f"{tuple(weights['w2'].shape)} do not fit each other")
        self.w_w1 = to_device(weights["w1"], dtype, device)
        self.w_w2 = to_device(weights["w2"], dtype, device)
        self.w0 = f32(weights["w0"])
        self.u = f32(weights["u"].reshape(-1))
        self.norm = f32(weights["norm"])
        self.w_o = to_device(weights["o"], dtype, device)

    def forward(self, ctx, x):
        ops, b = ctx.ops, ctx.batch
        H, D = self.num_heads, self.head_dim
        f32 = torch.float32
        m = ops.token_shift_mix(x, ctx.state, self.prev_offset, self.mu, b, ctx.act_dtype)
        r = ops.linear(m[0], self.w_r, out_dtype=f32)
        k = ops.linear(m[1], self.w_k, out_dtype=f32)
        v = ops.linear(m[2], self.w_v, out_dtype=f32)
        g = ops.linear(m[3], self.w_g, out_dtype=f32)
        z = ops.linear(ops.tanh(ops.linear(m[4], self.w_w1, out_dtype=f32), ctx.act_dtype), self.w_w2, out_dtype=f32)
        o = ops.wkv_recurrence(r, k, v, z, self.w0, self.u, ctx.state, b, H, D, x=x, prev_off=self.prev_offset)
        y = ops.head_norm_gate(o, g, self.norm, self.norm_eps, H, D, ctx.act_dtype)
        return ops.linear(y, self.w_o, out_dtype=f32, partials=True)
