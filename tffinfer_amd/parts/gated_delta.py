"""A mixer that carries a matrix of state per head, written by the delta rule with a decay, and a
mixer made of two that read the same rows."""
from __future__ import annotations

import torch

from ..config.base import ConfigError, PartSpec
from .base import MIXERS, Mixer, StateSpec, WeightSpec, register_mixer, to_device


@register_mixer("gated_delta")
class GatedDeltaMixer(Mixer):
    """With x the token's row, ``kv_heads`` heads of queries and keys of ``head_dim`` and ``num_heads``
    heads of values of ``value_dim`` (head h reads the queries and keys of head h // (heads / kv_heads)):

        q, k, v = silu(conv(Wq x)), silu(conv(Wk x)), silu(conv(Wv x))   conv: over time, per channel, ``conv_taps``
                                                                         taps ending at the token, zeros before the start
        q <- q / sqrt(|q|^2 + 1e-6) * head_dim^(-1/2),  k <- k / sqrt(|k|^2 + 1e-6)        per head
        beta = sigmoid(Wb x),  decay = exp(-exp(A_log) * softplus(Wa x + dt_bias))         per head
        S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                   per head, S [head_dim, value_dim]
        out = Wo [ o / rms_head(o) * norm * silu(Wg x) ]

    S (zero at a request's start) and the convolution's last ``conv_taps - 1`` inputs are the request's
    state, float32, one row of the state tensor.  The six projections are one product whose results
    stay in float32; convolution, unit vectors, beta, decay, recurrence and the norm over each head are
    float32.  ``external_output``: the mixer stops before Wo (``forward_inner``) and leaves the matrix
    to whoever combines it with another mixer's (``w_o_host``).
    """

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 conv_taps: int = 4, norm_eps: float = 1e-6, external_output: bool = False):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.conv_taps = int(conv_taps)
        self.norm_eps = float(norm_eps)
        self.external_output = bool(external_output)
        if min(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim) <= 0:
            raise ConfigError("gated delta: sizes must be positive")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"gated delta: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if self.head_dim > 256:
            raise ConfigError(f"gated delta: heads of {head_dim} key channels (up to 256)")
        if not 1 <= self.conv_taps <= 8:
            raise ConfigError(f"gated delta: a convolution of {conv_taps} taps (1 to 8)")
        self.w_in = self.w_o = self.w_o_host = self.conv = self.a_log = self.dt_bias = self.norm = None

    # ---- sizes -----------------------------------------------------------
    @property
    def channels(self) -> int:
        """Channels that pass the convolution: q, k and v."""
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.value_dim

    @property
    def inner_size(self) -> int:
        return self.num_heads * self.value_dim

    def state_spec(self):
        return StateSpec((self.num_heads * self.value_dim * self.head_dim + (self.conv_taps - 1) * self.channels,),
                         torch.float32)

    def weight_specs(self):
        W, H, G, D, E, K = (self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                            self.conv_taps)
        return {
            "q": WeightSpec((G * D, W)), "q.conv": WeightSpec((G * D, K), "vector"),
            "k": WeightSpec((G * D, W)), "k.conv": WeightSpec((G * D, K), "vector"),
            "v": WeightSpec((H * E, W)), "v.conv": WeightSpec((H * E, K), "vector"),
            "b": WeightSpec((H, W)), "a": WeightSpec((H, W)),
            "A_log": WeightSpec((H,), "decay_log"), "dt_bias": WeightSpec((H,), "vector"),
            "norm": WeightSpec((E,), "norm"),
            "g": WeightSpec((H * E, W)), "o": WeightSpec((W, H * E)),
        }

    def load_weights(self, weights, dtype, device):
        f32 = lambda t: t.to(torch.float32).contiguous().to(device)      # noqa: E731
        kind = weights["q"].dtype
        self.w_in = to_device(torch.cat([weights[s].to(kind) for s in ("q", "k", "v", "b", "a", "g")], 0), dtype, device)
        self.conv = f32(torch.cat([weights[s].to(torch.float32) for s in ("q.conv", "k.conv", "v.conv")], 0))
        self.a_log, self.dt_bias, self.norm = f32(weights["A_log"]), f32(weights["dt_bias"]), f32(weights["norm"])
        if self.external_output:
            self.w_o_host = weights["o"]
        else:
            self.w_o = to_device(weights["o"], dtype, device)

    def forward_inner(self, ctx, x, out=None, out_scale: float = 1.0):
        """Everything before Wo: [T, heads * value_dim] in the activation type, into ``out`` if given
        (a matrix whose rows may be strided), times ``out_scale``."""
        ops = ctx.ops
        H, G, D, E = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
        o = ops.gated_delta(proj, self.conv, self.a_log, self.dt_bias, ctx.state, ctx.batch, H, G, D, E)
        if out is None:
            out = torch.empty(o.shape[0], H * E, dtype=ctx.act_dtype, device=o.device)
        return ops.head_norm_silu_gate(o, proj[:, self.channels + 2 * H:], self.norm, self.norm_eps, H, E, out, out_scale)

    def forward(self, ctx, x):
        if self.external_output:
            raise RuntimeError("gated delta: its output matrix was left to a combining mixer")
        return ctx.ops.linear(self.forward_inner(ctx, x), self.w_o, out_dtype=torch.float32, partials=True)


@register_mixer("mixer_pair")
class MixerPair(Mixer):
    """Two mixers side by side that read the same rows: out = left_scale * left(x) + right_scale * right(x).

    Both must be able to stop before their output matrix (``external_output`` / ``forward_inner``): each
    writes its part of one matrix [T, left inner + right inner], scaled by its factor, and the two output
    matrices, put side by side, make the sum one product.  One of them may keep keys and values
    (``cache_spec``) and one a state (``state_spec``); the layer call's cache and state go to both.
    Their tensors are named ``left.*`` and ``right.*``."""

    graph_safe = True

    def __init__(self, hidden_size: int, left, right, left_scale: float = 1.0, right_scale: float = 1.0):
        self.hidden_size = int(hidden_size)
        self.left_scale = float(left_scale)
        self.right_scale = float(right_scale)
        self.left = self._build(left)
        self.right = self._build(right)
        if sum(m.cache_spec() is not None for m in (self.left, self.right)) > 1 or \
                sum(m.state_spec() is not None for m in (self.left, self.right)) > 1:
            raise ConfigError("mixer pair: both mixers ask for a cache, or both for a state; a layer call has one of each")
        self.w_o = None

    @staticmethod
    def _build(spec):
        if not isinstance(spec, PartSpec):
            raise ConfigError("mixer pair: 'left' and 'right' are the specs of two mixers")
        m = MIXERS.build(PartSpec(spec.kind, dict(spec.args, external_output=True)))
        if not hasattr(m, "forward_inner"):
            raise ConfigError(f"mixer pair: a '{spec.kind}' cannot stop before its output matrix")
        return m

    def cache_spec(self):
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self):
        return self.left.state_spec() or self.right.state_spec()

    def flops_per_query_key_pair(self):
        return self.left.flops_per_query_key_pair() + self.right.flops_per_query_key_pair()

    def weight_specs(self):
        specs = {f"left.{k}": v for k, v in self.left.weight_specs().items()}
        specs.update({f"right.{k}": v for k, v in self.right.weight_specs().items()})
        return specs

    def load_weights(self, weights, dtype, device):
        for name, m in (("left.", self.left), ("right.", self.right)):
            m.load_weights({k[len(name):]: v for k, v in weights.items() if k.startswith(name)}, dtype, device)
        lo, ro = self.left.w_o_host, self.right.w_o_host
        self.w_o = to_device(torch.cat([lo, ro.to(lo.dtype)], 1), dtype, device)
        self.left.w_o_host = self.right.w_o_host = None

    def forward(self, ctx, x):
        nl, nr = self.left.inner_size, self.right.inner_size
        y = torch.empty(x.shape[0], nl + nr, dtype=ctx.act_dtype, device=x.device)
        self.left.forward_inner(ctx, x, y[:, :nl], self.left_scale)
        self.right.forward_inner(ctx, x, y[:, nl:], self.right_scale)
        return ctx.ops.linear(y, self.w_o, out_dtype=torch.float32, partials=True)
