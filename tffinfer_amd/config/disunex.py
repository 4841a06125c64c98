"""Typed configuration of the Disunex decoder, read from its config.json.

The file lists its layers one by one (``layers``): each entry names its mixer
(``type``) with the mixer's sizes (``mixer``) and its feed-forward (``mlp``: a
dense one, a routed mixture of experts, or null for none).  An entry with
``weights_of: j`` has no tensors of its own: it runs layer j's parts on a cache
of its own, which here is one more call of layer j in the run order.  Sizes and
constants all come from the file; nothing is assumed equal between layers.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .base import ConfigError, LayerCall, LayerSpec, ModelConfig, PartSpec, coerce, optional, require

ARCHITECTURE = "Disunex"

#: positions the rotation tables are made for when the caller gives no shorter limit
#: (the file names none)
DEFAULT_MAX_POSITIONS = 131072


def _mixer_spec(i: int, width: int, eps: float, kind: str, m: dict) -> PartSpec:
    where = f"config.json: layers[{i}].mixer"
    if kind != "latent_attention":
        raise ConfigError(f"config.json: layers[{i}].type '{kind}' is not a mixer of this architecture "
                          "(latent_attention)")
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object")
    rot_dim = require(m, "rot_dim", int, where)
    rot = m.get("rot") or {}
    position = None
    if rot_dim > 0:
        if not isinstance(rot, dict):
            raise ConfigError(f"{where}.rot must be an object")
        dims = optional(rot, "dims", int, rot_dim, where + ".rot")
        position = PartSpec("rope", {"head_dim": rot_dim, "theta": require(rot, "base", float, where + ".rot"),
                                     "pairing": "interleaved", "rotary_dim": dims})
    mask = m.get("mask")
    window = 0
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"{where}.mask must be an object")
        window = require(mask, "size", int, where + ".mask")
        if window <= 0:
            raise ConfigError(f"{where}.mask.size must be positive, found {window}")
    return PartSpec("latent_attention", {
        "hidden_size": width,
        "num_heads": require(m, "heads", int, where),
        "head_dim": require(m, "dim", int, where),
        "rot_dim": rot_dim,
        "value_dim": require(m, "vdim", int, where),
        "kv_rank": require(m, "kv_rank", int, where),
        "scale": require(m, "scale", float, where),
        "window": window,
        "latent_norm_eps": eps,
        "position": position,
    })


def _mlp_spec(i: int, width: int, m) -> PartSpec:
    where = f"config.json: layers[{i}].mlp"
    if m is None:
        return PartSpec("none", {"hidden_size": width})
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object or null")
    kind = require(m, "kind", str, where)
    if kind == "dense":
        return PartSpec("gelu_mlp", {"hidden_size": width, "intermediate_size": require(m, "ff", int, where)})
    if kind == "moe":
        ex, ro = m.get("expert"), m.get("router")
        if not isinstance(ex, dict) or not isinstance(ro, dict):
            raise ConfigError(f"{where}: a mixture of experts needs 'expert' and 'router' objects")
        return PartSpec("routed_experts", {
            "hidden_size": width,
            "intermediate_size": require(ex, "ff", int, where + ".expert"),
            "limit": require(ex, "limit", float, where + ".expert"),
            "num_experts": require(ro, "experts", int, where + ".router"),
            "top": require(ro, "top", int, where + ".router"),
        })
    raise ConfigError(f"{where}.kind '{kind}' is not a feed-forward of this architecture (dense, moe)")


@dataclass
class DisunexConfig(ModelConfig):
    hidden_size: int
    vocab_size: int
    layers: list
    norm_eps: float
    postln_alpha: float
    max_position_embeddings: int = DEFAULT_MAX_POSITIONS
    eos_token_id: int | None = None
    extra: dict = field(default_factory=dict, repr=False)

    architecture = ARCHITECTURE
    tie_word_embeddings = True      # the logits are products with the embedding table
    caller_options = {}

    @classmethod
    def from_dict(cls, d: dict) -> "DisunexConfig":
        if d.get("architecture") != ARCHITECTURE:
            raise ConfigError(f"config.json: 'architecture' must be '{ARCHITECTURE}', found {d.get('architecture')!r}")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        norm = d.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: required object 'norm' is missing")
        eos = d.get("eos_token_id")
        known = {"architecture", "architectures", "layers", "norm", "postln_alpha", "vocab", "width",
                 "max_position_embeddings", "eos_token_id"}
        cfg = cls(
            hidden_size=require(d, "width", int),
            vocab_size=require(d, "vocab", int),
            layers=copy.deepcopy(layers),
            norm_eps=require(norm, "eps", float, "config.json: norm"),
            postln_alpha=require(d, "postln_alpha", float),
            max_position_embeddings=optional(d, "max_position_embeddings", int, DEFAULT_MAX_POSITIONS),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for k in ("hidden_size", "vocab_size", "max_position_embeddings"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, found {getattr(self, k)}")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps={self.norm_eps} must be positive")
        for i, L in enumerate(self.layers):
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            j = L.get("weights_of")
            if j is not None:
                j = coerce(j, "weights_of", int, f"config.json: layers[{i}]")
                if not 0 <= j < len(self.layers) or j == i or self.layers[j].get("weights_of") is not None:
                    raise ConfigError(f"config.json: layers[{i}].weights_of={j} must name another layer "
                                      "that has tensors of its own")
        self.layer_specs()      # every entry is read once, so that a bad one is reported at load

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "layers": copy.deepcopy(self.layers), "norm": {"eps": self.norm_eps},
             "postln_alpha": self.postln_alpha, "vocab": self.vocab_size, "width": self.hidden_size}
        if self.max_position_embeddings != DEFAULT_MAX_POSITIONS:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        for k, v in self.extra.items():
            d.setdefault(k, v)
        return d

    # ---- what the layers are made of -------------------------------------
    def owners(self) -> list[int]:
        """Indices of the layers that have tensors of their own, in the file's numbering."""
        return [i for i, L in enumerate(self.layers) if L.get("weights_of") is None]

    def layer_numbers(self) -> list[int]:
        return self.owners()

    def layer_specs(self) -> list[LayerSpec]:
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.norm_eps, "weight_offset": 1.0})
        specs = []
        for i in self.owners():
            L = self.layers[i]
            specs.append(LayerSpec(PartSpec("postnorm", {"alpha": self.postln_alpha}),
                                   _mixer_spec(i, self.hidden_size, self.norm_eps, require(L, "type", str, f"config.json: layers[{i}]"),
                                               L.get("mixer")),
                                   _mlp_spec(i, self.hidden_size, L.get("mlp")), norm))
        return specs

    def layer_schedule(self) -> list[LayerCall]:
        index = {i: n for n, i in enumerate(self.owners())}
        out = []
        for i, L in enumerate(self.layers):
            j = L.get("weights_of")
            out.append(LayerCall(index[i if j is None else int(j)], i))
        return out

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.norm_eps, "weight_offset": 1.0})
