"""Typed configuration of the Sipilorn decoder, read from its config.json.

The file lists its layers one by one (``layers``): each entry names its mixer (``type``: ``delta``, a
recurrence written by the gated delta rule, or ``parallel``, a windowed attention with an output
gate and such a recurrence side by side) with the mixer's sizes (``mixer``) and its feed-forward
(``mlp``: a dense gated one, experts chosen by a table over the token ids, or null for none).  A
layer's mixer and feed-forward read the same stream, each through a norm of its own.  ``loop`` runs
a span of the layers several times in a row with the same weights and a cache and state per pass,
adding a learned vector to the stream before each pass; the embedding has a norm, the logits a cap.
Sizes and constants all come from the file; nothing is assumed equal between layers.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

from .base import ConfigError, LayerCall, LayerSpec, ModelConfig, PartSpec, optional, require

ARCHITECTURE = "Sipilorn"

#: a length limit for callers that give none (the file names none)
DEFAULT_MAX_POSITIONS = 1 << 20


def _delta_args(width: int, eps: float, m, where: str) -> dict:
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object")
    heads = require(m, "heads", int, where)
    return {
        "hidden_size": width,
        "num_heads": heads,
        "num_kv_heads": optional(m, "kv_heads", int, heads, where),
        "head_dim": require(m, "dim", int, where),
        "value_dim": require(m, "vdim", int, where),
        "conv_taps": require(m, "conv", int, where),
        "norm_eps": eps,
    }


def _attention_args(width: int, eps: float, m, where: str) -> dict:
    if not isinstance(m, dict):
        raise ConfigError(f"{where} must be an object")
    heads = require(m, "heads", int, where)
    dim = require(m, "dim", int, where)
    window = 0
    mask = m.get("mask")
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"{where}.mask must be an object")
        window = require(mask, "size", int, where + ".mask")
        if window <= 0:
            raise ConfigError(f"{where}.mask: size must be positive")
    position = None
    rot = m.get("rot")
    if rot is not None:
        if not isinstance(rot, dict):
            raise ConfigError(f"{where}.rot must be an object")
        dims = require(rot, "dims", int, where + ".rot")
        if dims:
            position = PartSpec("rope", {"head_dim": dim, "theta": require(rot, "base", float, where + ".rot"),
                                         "pairing": "half", "rotary_dim": dims})
    return {
        "hidden_size": width,
        "num_heads": heads,
        "num_kv_heads": optional(m, "kv_heads", int, heads, where),
        "head_dim": dim,
        "value_dim": optional(m, "vdim", int, dim, where),
        "position": position,
        "scale": require(m, "scale", float, where),
        "qk_norm_eps": eps,
        "window": window,
    }


def _mixer_spec(i: int, width: int, eps: float, kind: str, m) -> PartSpec:
    where = f"config.json: layers[{i}].mixer"
    if kind == "delta":
        return PartSpec("gated_delta", _delta_args(width, eps, m, where))
    if kind == "parallel":
        if not isinstance(m, dict):
            raise ConfigError(f"{where} must be an object")
        return PartSpec("mixer_pair", {
            "hidden_size": width,
            "left": PartSpec("gated_gqa_attention", _attention_args(width, eps, m.get("left"), where + ".left")),
            "right": PartSpec("gated_delta", _delta_args(width, eps, m.get("right"), where + ".right")),
            "left_scale": optional(m, "left_scale", float, 1.0, where),
            "right_scale": optional(m, "right_scale", float, 1.0, where),
        })
    raise ConfigError(f"config.json: layers[{i}].type '{kind}' is not a mixer of this architecture (delta, parallel)")


def _mlp_spec(i: int, width: int, vocab: int, m) -> PartSpec:
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
        return PartSpec("table_experts", {
            "hidden_size": width,
            "intermediate_size": require(ex, "ff", int, where + ".expert"),
            "num_experts": require(ro, "experts", int, where + ".router"),
            "top": require(ro, "top", int, where + ".router"),
            "vocab_size": vocab,
        })
    raise ConfigError(f"{where}.kind '{kind}' is not a feed-forward of this architecture (dense, moe)")


@dataclass
class SipilornConfig(ModelConfig):
    hidden_size: int
    vocab_size: int
    layers: list
    norm_eps: float
    logit_softcap: float | None = None
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_position_embeddings: int = DEFAULT_MAX_POSITIONS
    eos_token_id: int | None = None
    extra: dict = field(default_factory=dict, repr=False)

    architecture = ARCHITECTURE
    tie_word_embeddings = False
    caller_options = {}

    @classmethod
    def from_dict(cls, d: dict) -> "SipilornConfig":
        if d.get("architecture") != ARCHITECTURE:
            raise ConfigError(f"config.json: 'architecture' must be '{ARCHITECTURE}', found {d.get('architecture')!r}")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        norm = d.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: required object 'norm' is missing")
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json: 'loop' must be an object")
            start = require(loop, "start", int, "config.json: loop")
            stop = require(loop, "stop", int, "config.json: loop")
            times = require(loop, "times", int, "config.json: loop")
        eos = d.get("eos_token_id")
        known = {"architecture", "architectures", "layers", "norm", "loop", "logit_softcap", "vocab", "width",
                 "max_position_embeddings", "eos_token_id"}
        cfg = cls(
            hidden_size=require(d, "width", int),
            vocab_size=require(d, "vocab", int),
            layers=copy.deepcopy(layers),
            norm_eps=require(norm, "eps", float, "config.json: norm"),
            logit_softcap=optional(d, "logit_softcap", float, None),
            loop_start=start, loop_stop=stop, loop_times=times,
            max_position_embeddings=optional(d, "max_position_embeddings", int, DEFAULT_MAX_POSITIONS),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None,
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def validate(self) -> None:
        for k in ("hidden_size", "vocab_size", "max_position_embeddings"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, found {getattr(self, k)}")
        if not (self.norm_eps > 0):
            raise ConfigError(f"config.json: norm.eps={self.norm_eps} must be positive")
        if self.logit_softcap is not None and not (self.logit_softcap > 0):
            raise ConfigError(f"config.json: logit_softcap={self.logit_softcap} must be positive")
        n = len(self.layers)
        if not (0 <= self.loop_start <= self.loop_stop <= n) or self.loop_times < 1:
            raise ConfigError(f"config.json: loop {self.loop_start} .. {self.loop_stop} x {self.loop_times} "
                              f"does not fit {n} layers")
        for i, L in enumerate(self.layers):
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        self.layer_specs()      # every entry is read once, so that a bad one is reported at load

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "layers": copy.deepcopy(self.layers), "norm": {"eps": self.norm_eps},
             "vocab": self.vocab_size, "width": self.hidden_size}
        if self.has_loop:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
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
            specs.append(LayerSpec(PartSpec("parallel"),
                                   _mixer_spec(i, self.hidden_size, self.norm_eps,
                                               require(L, "type", str, f"config.json: layers[{i}]"), L.get("mixer")),
                                   _mlp_spec(i, self.hidden_size, self.vocab_size, L.get("mlp")), norm))
        return specs

    def layer_schedule(self) -> list[LayerCall]:
        """The layers before the looped span, the span ``times`` times in a row (the pass's vector added
        before its first layer), the layers after it.  Every call has a cache and state of its own."""
        n = len(self.layers)
        order = [(i, -1) for i in range(self.loop_start)] if self.has_loop else [(i, -1) for i in range(n)]
        if self.has_loop:
            for t in range(self.loop_times):
                order += [(i, t if i == self.loop_start else -1) for i in range(self.loop_start, self.loop_stop)]
            order += [(i, -1) for i in range(self.loop_stop, n)]
        return [LayerCall(layer, call, True, offset) for call, (layer, offset) in enumerate(order)]

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.norm_eps})

    def embedding_norm_spec(self) -> PartSpec:
        return self.final_norm_spec()

    def stream_offset_rows(self) -> int:
        return self.loop_times if self.has_loop else 0
