"""Netovik decoder: registration of its configuration and tensor names.

The file names its tensors ``embed``, ``final.norm`` and ``l<i>.{norm1, norm2, mix.*, mlp.*, dwa}``:
a part's single weight carries the part's own name, and the logits are products with the
embedding table (no head tensor)."""
from ..config.netovik import ARCHITECTURE, NetovikConfig
from .decoder import TensorNames
from .registry import register_architecture

NETOVIK_NAMES = TensorNames(
    embedding="embed",
    layer="l{i}",
    final_norm="final.norm",
    head="head",
    children={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
    bare_weights=True,
)

register_architecture(ARCHITECTURE, NetovikConfig, NETOVIK_NAMES)
