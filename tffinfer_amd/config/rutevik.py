"""Typed configuration of the Rutevik decoder, read from its config.json.

The file lists its layers one by one (``layers``): each entry names its mixer (``type``:
``latent_attention``, whose queries pass a latent vector as its keys and values do, or ``attention``, a
differential attention with two score maps a head) with the mixer's sizes (``mixer``) and its
feed-forward (``mlp``: a dense one with the square of relu, a mixture of experts whose scores
weigh the experts' inputs, or null for none).  A latent attention with ``kv_from: j`` has no
down-projection of keys and values: it reads what layer j's call left in its cache.  Layers are
pre-norm blocks whose norm computes no statistics; the logits are scaled.  Sizes and constants all
come from the file; nothing is assumed equal between layers.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .base import ConfigError, LayerCall, LayerSpec, ModelConfig, PartSpec, coerce, optional, require

ARCHITECTURE = "Rutevik"

#: a length limit for callers that give none (the file names none)
DEFAULT_MAX_POSITIONS = 1 << 20


def _rotation(m: dict, size: int, where: str) -> PartSpec | None:
    """The position encoding of a part of ``size`` elements from the mixer's ``rot`` object."""
    rot = m.get("rot")
    if rot is None:
        return None
    if not isinstance(rot, dict):
        raise ConfigError(f"{where}.rot must be an object")
    dims = optional(rot, "dims", int, size, where + ".rot")
    if dims == 0:
        return None
    if dims < 0 or dims % 2 or dims > size:
        raise ConfigError(f"{where}.rot.dims={dims} must be even and at most {size}")
    args = {"head_dim": size, "theta": require(rot, "base", float, where + ".rot"), "pairing": "half", "rotary_dim": dims}
    sc = rot.get("scaling")
    if sc is None:
        return PartSpec("rope", args)
    if not isinstance(sc, dict):
        raise ConfigError(f"{where}.rot.scaling must be an object")
    for k in ("factor", "low", "high", "original"):
        args[k] = require(sc, k, float, where + ".rot.scaling")
    return PartSpec("rope_scaled", args)


def _latent_spec(i: int, width: int, eps: float, m: dict, where: str) -> PartSpec:
    rot_dim = require(m, "rot_dim", int, where)
    if rot_dim < 0:
        raise ConfigError(f"{where}.rot_dim must not be negative")
    return PartSpec("latent_attention", {
        "hidden_size": width,
        "num_heads": require(m, "heads", int, where),
        "head_dim": require(m, "dim", int, where),
        "rot_dim": rot_dim,
        "value_dim": require(m, "vdim", int, where),
        "kv_rank": require(m, "kv_rank", int, where),
        "q_rank": require(m, "q_rank", int, where),
        "scale": require(m, "scale", float, where),
        "latent_norm_eps": eps,
        "position": _rotation(m, rot_dim, where) if rot_dim > 0 else None,
        "sink": False,
        "output_gate": False,
        "shared_cache": m.get("kv_from") is not None,
    })


def _attention_spec(i: int, width: int, eps: float, m: dict, where: str) -> PartSpec:
    heads = require(m, "heads", int, where)
    dim = require(m, "dim", int, where)
    return PartSpec("differential_attention", {
        "hidden_size": width,
        "num_heads": heads,
        "num_kv_heads": optional(m, "kv_heads", int, heads, where),
        "head_dim": dim,
        "value_dim": optional(m, "vdim", int, dim, where),
        "position": _rotation(m, dim, where),
        "scale": require(m, "scale", float, where),
        "softcap": optional(m, "softcap", float, None, where),
        "diff": require(m, "diff", float, where),
        "norm_eps": eps,
    })


def _mixer_spec(i: int, width: int, eps: float, kind: str, m) -> PartSpec:
    where = f"config.json: layers[{i}].mixer"
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object")
    if kind == "latent_attention":
        return _latent_spec(i, width, eps, m, where)
    if kind == "attention":
        return _attention_spec(i, width, eps, m, where)
    raise ConfigError(f"config.json: layers[{i}].type '{kind}' is not a mixer of this architecture "
                      "(latent_attention, attention)")


def _mlp_spec(i: int, width: int, m) -> PartSpec:
    where = f"config.json: layers[{i}].mlp"
    if m is None:
        return PartSpec("none", {"hidden_size": width})
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object or null")
    kind = require(m, "kind", str, where)
    if kind == "dense":
        return PartSpec("gelu_mlp", {"hidden_size": width, "intermediate_size": require(m, "ff", int, where),
                                     "activation": "relu2"})
    if kind == "moe":
        ex, ro = m.get("expert"), m.get("router")
        if not isinstance(ex, dict) or not isinstance(ro, dict):
            raise ConfigError(f"{where}: a mixture of experts needs 'expert' and 'router' objects")
        return PartSpec("routed_experts", {
            "hidden_size": width,
            "intermediate_size": require(ex, "ff", int, where + ".expert"),
            "num_experts": require(ro, "experts", int, where + ".router"),
            "top": require(ro, "top", int, where + ".router"),
            "limit": None, "act_alpha": 1.0, "up_offset": 0.0,          # silu(gate) * up, no clamp
            "correction": False, "normalize": False, "weight_input": True,
        })
    raise ConfigError(f"{where}.kind '{kind}' is not a feed-forward of this architecture (dense, moe)")


@dataclass
class RutevikConfig(ModelConfig):
    hidden_size: int
    vocab_size: int
    layers: list
    norm_eps: float
    logit_scale: float = 1.0
    max_position_embeddings: int = DEFAULT_MAX_POSITIONS
    eos_token_id: int | None = None
    extra: dict = field(default_factory=dict, repr=False)

    architecture = ARCHITECTURE
    tie_word_embeddings = False
    caller_options = {}

    @classmethod
    def from_dict(cls, d: dict) -> "RutevikConfig":
        if d.get("architecture") != ARCHITECTURE:
            raise ConfigError(f"config.json: 'architecture' must be '{ARCHITECTURE}', found {d.get('architecture')!r}")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        norm = d.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: required object 'norm' is missing")
        eos = d.get("eos_token_id")
        known = {"architecture", "architectures", "layers", "norm", "logit_scale", "vocab", "width",
                 "max_position_embeddings", "eos_token_id"}
        cfg = cls(
            hidden_size=require(d, "width", int),
            vocab_size=require(d, "vocab", int),
            layers=copy.deepcopy(layers),
            norm_eps=require(norm, "eps", float, "config.json: norm"),
            logit_scale=optional(d, "logit_scale", float, 1.0),
            max_position_embeddings=optional(d, "max_position_embeddings", int, DEFAULT_MAX_POSITIONS),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    def kv_source(self, i: int) -> int | None:
        """The layer whose cache layer i reads, or None if it fills its own."""
        m = self.layers[i].get("mixer")
        j = m.get("kv_from") if isinstance(m, dict) else None
        return None if j is None else coerce(j, "kv_from", int, f"config.json: layers[{i}].mixer")

    def validate(self) -> None:
        for k in ("hidden_size", "vocab_size", "max_position_embeddings"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, found {getattr(self, k)}")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps={self.norm_eps} must be positive")
        for i, L in enumerate(self.layers):
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        specs = self.layer_specs()      # every entry is read once, so that a bad one is reported at load
        for i, L in enumerate(self.layers):
            j = self.kv_source(i)
            if j is None:
                continue
            where = f"config.json: layers[{i}].mixer.kv_from={j}"
            if L.get("type") != "latent_attention":
                raise ConfigError(f"{where}: only a latent attention reads another layer's cache")
            if not 0 <= j < len(self.layers) or j == i or self.layers[j].get("type") != "latent_attention" \
                    or self.kv_source(j) is not None:
                raise ConfigError(f"{where} must name another latent attention layer that fills a cache of its own")
            if j > i:
                raise ConfigError(f"{where}: the layer whose cache is read must run before the reader")
            a, b = specs[i].mixer.args, specs[j].mixer.args
            if any(a[k] != b[k] for k in ("kv_rank", "rot_dim", "position")):
                raise ConfigError(f"{where}: rank, rotated size and rotation of the two layers must be equal")

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "layers": copy.deepcopy(self.layers), "logit_scale": self.logit_scale,
             "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.hidden_size}
        if self.max_position_embeddings != DEFAULT_MAX_POSITIONS:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        for k, v in self.extra.items():
            d.setdefault(k, v)
        return d

    def layer_specs(self) -> list[LayerSpec]:
        norm = self.final_norm_spec()
        specs = []
        for i, L in enumerate(self.layers):
            specs.append(LayerSpec(PartSpec("prenorm"),
                                   _mixer_spec(i, self.hidden_size, self.norm_eps,
                                               require(L, "type", str, f"config.json: layers[{i}]"), L.get("mixer")),
                                   _mlp_spec(i, self.hidden_size, L.get("mlp")), norm))
        return specs

    def layer_schedule(self) -> list[LayerCall]:
        """Every layer once, in order; a layer with ``kv_from`` works on the cache of the layer it names and
        writes nothing there."""
        out = []
        for i in range(len(self.layers)):
            j = self.kv_source(i)
            out.append(LayerCall(i, i, True) if j is None else LayerCall(i, j, False))
        return out

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("dyt", {"size": self.hidden_size})
