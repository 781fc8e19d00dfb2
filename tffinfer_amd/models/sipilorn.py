"""Sipilorn decoder: registration of its configuration and tensor names.

The file names its tensors ``embed``, ``embed.norm``, ``loop.step``, ``final.norm``, ``head`` and
``l<i>.{norm1, norm2, mix.*, mlp.*}``: a part's single weight carries the part's own name."""
from ..config.sipilorn import ARCHITECTURE, SipilornConfig
from .decoder import TensorNames
from .registry import register_architecture

SIPILORN_NAMES = TensorNames(
    embedding="embed",
    layer="l{i}",
    final_norm="final.norm",
    head="head",
    stream_offsets="loop.step",
    children={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
    bare_weights=True,
)

register_architecture(ARCHITECTURE, SipilornConfig, SIPILORN_NAMES)
