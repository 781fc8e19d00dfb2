"""Token embedding and output head."""
from __future__ import annotations

import torch

from .base import Part, WeightSpec, to_device


class Embedding(Part):
    """x[t, :] = scale * E[token[t], :] into the float32 residual stream (scale 1: the rows
    as they are), then through ``norm`` (an RMS norm part, named ``norm`` under the table's name)
    if there is one.  Reference: src/kernel/cpu/embedding.cpp:34-49 (a CPU lookup there)."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, norm=None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.scale = float(scale)
        self.norm = norm
        self.weight = None

    def children(self):
        return {"norm": self.norm} if self.norm is not None else {}

    def weight_specs(self):
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), "embedding")}

    def load_weights(self, weights, dtype, device):
        self.weight = to_device(weights["weight"], dtype, device)

    def forward(self, ctx, token_ids):
        x = ctx.ops.embed(self.weight, token_ids)
        if self.scale != 1.0:
            ctx.ops.scale_rows(x, self.scale)       # (in float32; the table itself also serves a tied head)
        if self.norm is not None:
            x = ctx.ops.rmsnorm(x, self.norm.weight, self.norm.eps)
        return x


class OutputHead(Part):
    """logits = y . Wout^T in float32, no bias, no scale
    (src/core/model/qwen3/QWen3Creator.cpp:161-165, :324-329).  With tied
    embeddings the head has no tensor of its own and uses the embedding's.
    ``softcap`` c: the logits leave as c * tanh(logits / c).  ``scale``: the logits are multiplied by it
    (in float32, before a cap)."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Embedding | None, softcap: float | None = None,
                 scale: float | None = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.tied_to = tied_to
        self.softcap = float(softcap) if softcap else 0.0
        self.scale = float(scale) if scale is not None else 1.0
        self._weight = None

    def weight_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), "matrix")}

    def load_weights(self, weights, dtype, device):
        if self.tied_to is None:
            self._weight = to_device(weights["weight"], dtype, device)

    @property
    def weight(self):
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def forward(self, ctx, y):
        logits = ctx.ops.linear(y, self.weight, out_dtype=torch.float32)
        if self.scale != 1.0:
            ctx.ops.scale_rows(logits, self.scale)
        return ctx.ops.softcap_(logits, self.softcap) if self.softcap else logits
