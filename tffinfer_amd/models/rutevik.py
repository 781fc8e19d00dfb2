"""Rutevik decoder: registration of its configuration and tensor names.

The file names its tensors ``embed``, ``final.norm``, ``head`` and ``l<i>.{norm1, norm2, mix.*, mlp.*}``:
a part's single weight carries the part's own name, its other tensors follow it (``l0.norm1.alpha``)."""
from ..config.rutevik import ARCHITECTURE, RutevikConfig
from .decoder import TensorNames
from .registry import register_architecture

RUTEVIK_NAMES = TensorNames(
    embedding="embed",
    layer="l{i}",
    final_norm="final.norm",
    head="head",
    children={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
    bare_weights=True,
)

register_architecture(ARCHITECTURE, RutevikConfig, RUTEVIK_NAMES)
