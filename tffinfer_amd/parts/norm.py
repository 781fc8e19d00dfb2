"""Norms on the residual stream: RMS norms, and a norm without statistics."""
from __future__ import annotations

import torch

from .base import Norm, WeightSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """y = v * rsqrt(mean(v^2) + eps) * w over rows of ``size`` elements, where
    v is the residual stream plus the term still pending; sum, mean, rsqrt and
    products in float32.  Reference: src/kernel/cuda/norm.cu:31-48 (the weight
    product fused as in src/core/runtime/GraphOptimizer.cpp:197-229).

    ``weight_offset``: the stored weight lies around zero and the factor is
    ``weight_offset + w`` (formed once, in float32, at load).  ``optional``: a
    file may leave the weight out; the norm then has none and its block skips it."""

    graph_safe = True

    def __init__(self, size: int, eps: float, weight_offset: float = 0.0, optional: bool = False):
        self.size = int(size)
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.optional = bool(optional)
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), "norm_offset" if self.weight_offset else "norm",
                                     optional=self.optional)}

    def load_weights(self, weights, dtype, device):
        if "weight" not in weights:
            self.weight = None
            return
        # norm weights stay in float32 whatever the activation type is
        w = weights["weight"].to(torch.float32)
        if self.weight_offset:
            w = w + self.weight_offset
        self.weight = w.contiguous().to(device)

    def forward_post(self, ctx, resid, delta, alpha: float):
        """The norm of a block that norms after the sum: ``resid <- norm(alpha * resid + delta)``
        in place; returns the rows in the activation type (the stream itself where that is
        float32)."""
        out = ctx.ops.scale_add_rmsnorm(resid, delta, self.weight, self.eps, alpha,
                                        None if ctx.act_dtype == torch.float32 else ctx.act_dtype)
        return resid if out is None else out

    #: ``forward`` takes ``for_linear``: its result may then be rows that lack the norm's factor,
    #: which only ``ops.linear`` understands
    for_linear_aware = True

    def forward(self, ctx, resid, delta, rows=None, for_linear=False):
        return ctx.ops.add_rmsnorm(resid, delta, self.weight, self.eps, ctx.act_dtype, rows=rows,
                                   for_linear=for_linear)


@register_norm("group_rmsnorm")
class GroupRMSNorm(Norm):
    """A row is cut into ``groups`` equal consecutive parts; each part is divided by its own
    sqrt(mean(part^2) + eps); the whole is multiplied by w.  Sums, roots and products in float32.

    ``forward_add`` is the norm of a block that norms a sublayer's *output* before the sum:
    ``resid <- resid + norm(delta)``.  ``forward`` norms the stream itself (the model's last norm)."""

    graph_safe = True

    def __init__(self, size: int, eps: float, groups: int = 1, optional: bool = False):
        self.size = int(size)
        self.eps = float(eps)
        self.groups = int(groups)
        self.optional = bool(optional)
        if self.groups <= 0 or self.size % self.groups:
            from ..config.base import ConfigError
            raise ConfigError(f"group norm: rows of {self.size} do not divide into {self.groups} groups")
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), "norm", optional=self.optional)}

    def load_weights(self, weights, dtype, device):
        self.weight = (weights["weight"].to(torch.float32).contiguous().to(device)
                       if "weight" in weights else None)

    def forward_add(self, ctx, resid, delta):
        """``resid <- resid + norm(delta)`` in place; returns the new rows in the activation type
        (the stream itself where that is float32)."""
        out = ctx.ops.group_rmsnorm_add(resid, delta, self.weight, self.groups, self.eps,
                                        None if ctx.act_dtype == torch.float32 else ctx.act_dtype)
        return resid if out is None else out

    def forward(self, ctx, resid, delta, rows=None, for_linear=False):
        if delta is not None:
            resid += ctx.ops.as_tensor(delta)
        return ctx.ops.group_rmsnorm_add(None, resid, self.weight, self.groups, self.eps, ctx.act_dtype, rows=rows)


@register_norm("dyt")
class DynamicTanh(Norm):
    """A norm that computes no mean and no variance: y = tanh(alpha * v) * w + b element by element,
    with one learned scalar ``alpha`` and vectors ``w`` and ``b`` of the row's size; v is the residual
    stream plus the term still pending.  float32 throughout.  The tensors are called ``weight``, ``b``
    and ``alpha`` (a tensor without dimensions).  ``optional``: a file may leave them out (the norm of
    a sublayer that a layer does not have); the norm then has no weight and is not to be run."""

    graph_safe = True

    def __init__(self, size: int, optional: bool = False):
        self.size = int(size)
        self.optional = bool(optional)
        self.weight = self.bias = None
        self.alpha = 1.0

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), "norm", optional=self.optional),
                "b": WeightSpec((self.size,), "norm_offset", optional=self.optional),
                "alpha": WeightSpec((), "unit_interval", optional=self.optional)}

    def load_weights(self, weights, dtype, device):
        if not all(k in weights for k in ("weight", "b", "alpha")):
            self.weight = self.bias = None
            return
        self.weight = weights["weight"].to(torch.float32).contiguous().to(device)
        self.bias = weights["b"].to(torch.float32).contiguous().to(device)
        self.alpha = float(weights["alpha"].to(torch.float32))      # (a kernel argument: read once, at load)

    def forward(self, ctx, resid, delta, rows=None, for_linear=False):
        return ctx.ops.add_dyt(resid, delta, self.alpha, self.weight, self.bias, ctx.act_dtype, rows=rows)
