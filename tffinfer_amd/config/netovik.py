"""Typed configuration of the Netovik decoder, read from its config.json.

The file lists its layers one by one (``layers``): each entry names its mixer (``type``: a
recurrence with a matrix of state per head, ``wkv``, or ``attention`` with scores mixed between
heads) with the mixer's sizes (``mixer``) and its feed-forward (``mlp``: a dense gated one, a
mixture of experts, or null for none).  Norms stand on the sublayers' outputs (``norm.groups``
groups, ``norm.eps``), the embedding is scaled (``embedding.scale``), and after every layer
the stream is a weighted sum of the outputs of all layers so far.  Sizes and constants all come
from the file; nothing is assumed equal between layers.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .base import ConfigError, LayerSpec, ModelConfig, PartSpec, optional, require

ARCHITECTURE = "Netovik"

#: a length limit for callers that give none (the file names none; no table grows with it)
DEFAULT_MAX_POSITIONS = 1 << 20


def _mixer_spec(i: int, width: int, eps: float, kind: str, m) -> PartSpec:
    where = f"config.json: layers[{i}].mixer"
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object")
    if kind == "wkv":
        return PartSpec("wkv", {
            "hidden_size": width,
            "num_heads": require(m, "heads", int, where),
            "head_dim": require(m, "dim", int, where),
            "norm_eps": eps,
            "decay_rank": optional(m, "decay_rank", int, None, where),
        })
    if kind == "attention":
        mask = m.get("mask")
        window = keep = 0
        if mask is not None:
            if not isinstance(mask, dict):
                raise ConfigError(f"{where}.mask must be an object")
            window = require(mask, "size", int, where + ".mask")
            keep = optional(mask, "keep_first", int, 0, where + ".mask")
            if window <= 0 or keep < 0:
                raise ConfigError(f"{where}.mask: size must be positive and keep_first not negative")
        heads = require(m, "heads", int, where)
        return PartSpec("mixed_head_attention", {
            "hidden_size": width,
            "num_heads": heads,
            "num_kv_heads": optional(m, "kv_heads", int, heads, where),
            "head_dim": require(m, "dim", int, where),
            "value_dim": optional(m, "vdim", int, None, where),
            "scale": require(m, "scale", float, where),
            "softcap": optional(m, "softcap", float, None, where),      # (none: the scores as they are)
            "bias_max": require(m, "bias_max", int, where),
            "bias_buckets": optional(m, "bias_buckets", int, None, where),
            "window": window,
            "keep_first": keep,
            "qk_norm_eps": eps,
        })
    raise ConfigError(f"config.json: layers[{i}].type '{kind}' is not a mixer of this architecture (wkv, attention)")


def _mlp_spec(i: int, width: int, m) -> PartSpec:
    where = f"config.json: layers[{i}].mlp"
    if m is None:
        return PartSpec("none", {"hidden_size": width})
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object or null")
    kind = require(m, "kind", str, where)
    if kind == "dense":
        return PartSpec("swiglu", {"hidden_size": width, "intermediate_size": require(m, "ff", int, where),
                                   "names": ("gate", "up", "down")})
    if kind == "moe":
        ex, ro = m.get("expert"), m.get("router")
        if not isinstance(ex, dict) or not isinstance(ro, dict):
            raise ConfigError(f"{where}: a mixture of experts needs 'expert' and 'router' objects")
        return PartSpec("routed_experts", {
            "hidden_size": width,
            "intermediate_size": require(ex, "ff", int, where + ".expert"),
            "num_experts": require(ro, "experts", int, where + ".router"),
            "top": require(ro, "top", int, where + ".router"),
            # softmax over all experts, the chosen scores as weights; experts silu(g) * u without a clamp
            "limit": None, "act_alpha": 1.0, "up_offset": 0.0, "correction": False, "router_softmax": True,
        })
    raise ConfigError(f"{where}.kind '{kind}' is not a feed-forward of this architecture (dense, moe)")


@dataclass
class NetovikConfig(ModelConfig):
    hidden_size: int
    vocab_size: int
    layers: list
    norm_eps: float
    norm_groups: int
    embedding_scale: float
    max_position_embeddings: int = DEFAULT_MAX_POSITIONS
    eos_token_id: int | None = None
    extra: dict = field(default_factory=dict, repr=False)

    architecture = ARCHITECTURE
    tie_word_embeddings = True      # the logits are products with the embedding table, without its scale
    caller_options = {}

    @classmethod
    def from_dict(cls, d: dict) -> "NetovikConfig":
        if d.get("architecture") != ARCHITECTURE:
            raise ConfigError(f"config.json: 'architecture' must be '{ARCHITECTURE}', found {d.get('architecture')!r}")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        norm, emb = d.get("norm"), d.get("embedding")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: required object 'norm' is missing")
        if emb is None:
            emb = {}            # (no scale: the rows as they are)
        if not isinstance(emb, dict):
            raise ConfigError("config.json: 'embedding' must be an object")
        eos = d.get("eos_token_id")
        known = {"architecture", "architectures", "layers", "norm", "embedding", "vocab", "width",
                 "max_position_embeddings", "eos_token_id"}
        cfg = cls(
            hidden_size=require(d, "width", int),
            vocab_size=require(d, "vocab", int),
            layers=copy.deepcopy(layers),
            norm_eps=require(norm, "eps", float, "config.json: norm"),
            norm_groups=optional(norm, "groups", int, 1, "config.json: norm"),
            embedding_scale=optional(emb, "scale", float, 1.0, "config.json: embedding"),
            max_position_embeddings=optional(d, "max_position_embeddings", int, DEFAULT_MAX_POSITIONS),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for k in ("hidden_size", "vocab_size", "max_position_embeddings", "norm_groups"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, found {getattr(self, k)}")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps={self.norm_eps} must be positive")
        if self.hidden_size % self.norm_groups:
            raise ConfigError(f"config.json: width {self.hidden_size} does not divide into norm.groups={self.norm_groups}")
        for i, L in enumerate(self.layers):
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        self.layer_specs()      # every entry is read once, so that a bad one is reported at load

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
             "layers": copy.deepcopy(self.layers), "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.max_position_embeddings != DEFAULT_MAX_POSITIONS:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        for k, v in self.extra.items():
            d.setdefault(k, v)
        return d

    def layer_specs(self) -> list[LayerSpec]:
        norm = self.final_norm_spec()
        depths = len(self.layers) + 1
        specs = []
        for i, L in enumerate(self.layers):
            specs.append(LayerSpec(PartSpec("outnorm", {"depth": i, "depths": depths}),
                                   _mixer_spec(i, self.hidden_size, self.norm_eps,
                                               require(L, "type", str, f"config.json: layers[{i}]"), L.get("mixer")),
                                   _mlp_spec(i, self.hidden_size, L.get("mlp")), norm))
        return specs

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("group_rmsnorm", {"size": self.hidden_size, "eps": self.norm_eps, "groups": self.norm_groups})
