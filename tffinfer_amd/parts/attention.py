"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError, PartSpec
from .base import (POSITION_ENCODINGS, KVCacheSpec, Mixer, PositionEncoding, WeightSpec,
                   register_mixer, to_device)


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    """q, k, v projections (no bias); per-head RMS norm of q and k over the
    head size with one [d] weight each, before the rotation; the rotation; the
    keys and values of the step's tokens written to the request's pages;
    causal softmax attention with scale 1/sqrt(d) in which q head h reads kv
    head h // (nq / nkv), restricted to the last ``window`` keys if window > 0;
    output projection.

    Reference: src/core/model/qwen3/QWen3Creator.cpp:66-131 (wiring),
    src/core/model/base/ModelCreatorBase.cpp:242-283 (attention and output
    projection), src/kernel/cuda/paged_flash_attention.cu:855-1055 (kernel).
    The three projections are stacked into one [(nq + 2 nkv) d, H] matrix at
    load; the reference keeps three products (QWen3Creator.cpp:66-75).
    """

    graph_safe = True
    #: the input is used by ``ops.linear`` and by nothing else
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position, qk_norm_eps: float | None = 1e-6, window: int = 0,
                 scale: float | None = None):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if isinstance(position, PartSpec):
            position = POSITION_ENCODINGS.build(position)
        if position is not None and not isinstance(position, PositionEncoding):
            raise ConfigError("attention: 'position' must be a position encoding or its spec")
        self.position = position
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = None

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def flops_per_query_key_pair(self):
        return 4 * self.num_heads * self.head_dim      # q.k and p.v, a multiply and an add each

    def weight_specs(self):
        H, nq, nkv, d = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        specs = {
            "q_proj.weight": WeightSpec((nq * d, H)),
            "k_proj.weight": WeightSpec((nkv * d, H)),
            "v_proj.weight": WeightSpec((nkv * d, H)),
            "o_proj.weight": WeightSpec((H, nq * d)),
        }
        if self.qk_norm_eps is not None:
            specs["q_norm.weight"] = WeightSpec((d,), "norm")
            specs["k_norm.weight"] = WeightSpec((d,), "norm")
        return specs

    def load_weights(self, weights, dtype, device):
        qkv = torch.cat([weights["q_proj.weight"], weights["k_proj.weight"], weights["v_proj.weight"]], 0)
        self.w_qkv = to_device(qkv, dtype, device)
        self.w_o = to_device(weights["o_proj.weight"], dtype, device)
        if self.qk_norm_eps is not None:
            self.q_norm = weights["q_norm.weight"].to(torch.float32).contiguous().to(device)
            self.k_norm = weights["k_norm.weight"].to(torch.float32).contiguous().to(device)

    def forward(self, ctx, x):
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        qkv = ops.linear(x, self.w_qkv)
        table = self.position.cached_table(ctx.max_positions, x.device) if self.position is not None else None
        pairing = 1 if (self.position is not None and self.position.pairing == "interleaved") else 0
        o = ops.qkv_attention(qkv, nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0,
                              table, pairing, kv, b, self.window, self.scale)
        return ops.linear(o, self.w_o, out_dtype=torch.float32, partials=True)


@register_mixer("gated_gqa_attention")
class GatedGQAttention(Mixer):
    """Grouped-query attention whose keys and values have sizes of their own and whose heads pass
    a gate before the output projection:

        q_h = rot(norm_q(Wq x)_h),  k_g = rot(norm_k(Wk x)_g)      (heads of ``head_dim``)
        v_g = (Wv x)_g                                              (heads of ``value_dim``)
        p_h(i, .) = softmax over the visible j of scale * q_h(i) . k_g(j),   g = h // (heads / kv_heads)
        y_h = (sum_j p_h(i, j) v_g(j)) * sigmoid(Wg x)_h * out_scale;   out = Wo [y_h]_h

    norm: RMS norm over the head with one [head_dim] weight for all heads (``qk_norm_eps`` None: none);
    rot: the position encoding (``position``), on as many elements of the head as it rotates;
    visible: j <= i, and i - j < window if there is one.  ``output_gate`` False leaves the gate out.

    The attention proper runs on the paged kernels of ``GQAttention`` with one head size for keys
    and values: the larger of the two, brought up to a size those kernels take.  The projections'
    rows are padded with zero rows accordingly (a padded key element adds nothing to a score, a
    padded value element is not read back), and the norm over the padded head is made the norm
    over the head itself by its constants: with P the padded size, x / sqrt(sum / P + eps d / P)
    times w sqrt(d / P) is x / sqrt(sum / d + eps) times w.

    ``external_output``: the mixer stops before Wo (``forward_inner``) and leaves the matrix to
    whoever combines it with another mixer's (``w_o_host``).
    """

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 position, scale: float | None = None, qk_norm_eps: float | None = 1e-6, window: int = 0,
                 output_gate: bool = True, external_output: bool = False):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        if min(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim) <= 0:
            raise ConfigError("gated attention: sizes must be positive")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"gated attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.window = int(window or 0)
        if self.window < 0:
            raise ConfigError("gated attention: the window must not be negative")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if isinstance(position, PartSpec):
            position = POSITION_ENCODINGS.build(position)
        if position is not None and not isinstance(position, PositionEncoding):
            raise ConfigError("gated attention: 'position' must be a position encoding or its spec")
        if position is not None and position.rotary_dim > self.head_dim:
            raise ConfigError(f"gated attention: {position.rotary_dim} rotated elements of a head of {self.head_dim}")
        self.position = position
        self.has_gate = bool(output_gate)
        self.external_output = bool(external_output)
        self._dtype = torch.bfloat16
        self.w_qkv = self.w_g = self.w_o = self.w_o_host = self.q_norm = self.k_norm = None

    # ---- sizes -----------------------------------------------------------
    def padded_head_dim(self) -> int:
        from ..kernels.ops import padded_head_size
        return padded_head_size(max(self.head_dim, self.value_dim), self._dtype)

    @property
    def inner_size(self) -> int:
        """Columns of what ``forward_inner`` leaves: the input size of Wo."""
        return self.num_heads * self.value_dim

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.padded_head_dim(), self.window)

    def flops_per_query_key_pair(self):
        return 4 * self.num_heads * self.padded_head_dim()

    def weight_specs(self):
        W, H, G, D, E = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        specs = {"q": WeightSpec((H * D, W)), "k": WeightSpec((G * D, W)), "v": WeightSpec((G * E, W)),
                 "o": WeightSpec((W, H * E))}
        if self.qk_norm_eps is not None:
            specs["q.norm"] = WeightSpec((D,), "norm")
            specs["k.norm"] = WeightSpec((D,), "norm")
        if self.has_gate:
            specs["g"] = WeightSpec((H * E, W))
        return specs

    def load_weights(self, weights, dtype, device):
        self._dtype = dtype
        H, G, D, E, W = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, self.hidden_size
        P = self.padded_head_dim()

        def padded(w, heads, size):
            w = w.view(heads, size, W)
            return torch.nn.functional.pad(w, (0, 0, 0, P - size)).reshape(heads * P, W) if P > size else w.reshape(heads * size, W)

        kind = weights["q"].dtype
        qkv = torch.cat([padded(weights["q"], H, D), padded(weights["k"].to(kind), G, D),
                         padded(weights["v"].to(kind), G, E)], 0)
        self.w_qkv = to_device(qkv, dtype, device)
        self.w_g = to_device(weights["g"], dtype, device) if self.has_gate else None
        if self.external_output:
            self.w_o_host = weights["o"]
        else:
            self.w_o = to_device(weights["o"], dtype, device)
        if self.qk_norm_eps is not None:
            f = math.sqrt(D / P)
            pad = lambda w: torch.nn.functional.pad(w.to(torch.float32) * f, (0, P - D)).contiguous().to(device)  # noqa: E731
            self.q_norm, self.k_norm = pad(weights["q.norm"]), pad(weights["k.norm"])
            self._eps = self.qk_norm_eps * D / P
        else:
            self._eps = 0.0

    def forward_inner(self, ctx, x, out=None, out_scale: float = 1.0):
        """Everything before Wo: [T, heads * value_dim] in the activation type, into ``out`` if given
        (a matrix whose rows may be strided), times ``out_scale``."""
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        H, G, E = self.num_heads, self.num_kv_heads, self.value_dim
        P = kv.k_cache.shape[3]
        qkv = ops.linear(x, self.w_qkv)
        gate = ops.linear(x, self.w_g) if self.has_gate else None
        table = self.position.cached_table(ctx.max_positions, qkv.device) if self.position is not None else None
        pairing = 1 if (self.position is not None and self.position.pairing == "interleaved") else 0
        o = ops.qkv_attention(qkv, H, G, P, self.q_norm, self.k_norm, self._eps, table, pairing, kv, b,
                              self.window, self.scale)
        if out is None:
            out = torch.empty(o.shape[0], H * E, dtype=o.dtype, device=o.device)
        if gate is None:
            out.copy_(o.view(-1, H, P)[:, :, :E].reshape(-1, H * E))
            return out.mul_(out_scale) if out_scale != 1.0 else out
        return ops.sigmoid_gate_heads(o, P, gate, H, E, out, out_scale)

    def forward(self, ctx, x):
        if self.external_output:
            raise RuntimeError("gated attention: its output matrix was left to a combining mixer")
        return ctx.ops.linear(self.forward_inner(ctx, x), self.w_o, out_dtype=torch.float32, partials=True)


@register_mixer("differential_attention")
class DifferentialAttention(Mixer):
    """Grouped-query attention in which every head has two score maps over the same values, and the
    second map's output is subtracted from the first's:

        q_hm = rot((Wq x + bq)_hm),  k_gm = rot((Wk x + bk)_gm)    (m = 0, 1; maps of ``head_dim``)
        v_g  = (Wv x + bv)_g                                        (heads of ``value_dim``)
        s_hm(i, j) = scale * q_hm(i) . k_gm(j),  capped to softcap * tanh(s / softcap) where there is a cap
        a_hm(i) = sum over j <= i of softmax_j(s_hm(i, .)) v_g(j),   g = h // (heads / kv_heads)
        lambda  = exp(lq1 . lk1) - exp(lq2 . lk2) + diff            (one number for the layer)
        o_h = a_h0 - lambda a_h1;   o_h <- o_h / sqrt(mean(o_h^2) + eps) * (1 - diff)
        out = Wo [o_h * sigmoid(Wg x)_h]_h

    q and k are laid out head by head as [map 0 | map 1]; rot: the position encoding, on as many
    elements of every map as it rotates.  ``bias`` False: no bq, bk, bv; ``output_gate`` False: no gate.

    The attention proper runs on the paged kernels of ``GQAttention`` as 2 heads a head on ``kv_heads``
    kv heads: a key row holds both maps' keys side by side, a query is zero outside its own map's part,
    so the two maps share one stored key row and one stored value row.  The cache's head size is the
    larger of 2 ``head_dim`` and ``value_dim``, brought up to a size those kernels take.  All four
    projections are one product whose result stays float32 until biases and rotation are done.
    """

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 position, scale: float | None = None, softcap: float | None = None, diff: float = 0.0,
                 norm_eps: float = 1e-6, bias: bool = True, output_gate: bool = True):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        if min(self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim) <= 0:
            raise ConfigError("differential attention: sizes must be positive")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"differential attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.softcap = float(softcap) if softcap else 0.0
        if self.softcap < 0:
            raise ConfigError("differential attention: the cap on the scores must not be negative")
        self.diff = float(diff)
        self.norm_eps = float(norm_eps)
        self.has_bias = bool(bias)
        self.has_gate = bool(output_gate)
        if isinstance(position, PartSpec):
            position = POSITION_ENCODINGS.build(position)
        if position is not None and not isinstance(position, PositionEncoding):
            raise ConfigError("differential attention: 'position' must be a position encoding or its spec")
        if position is not None and position.rotary_dim > self.head_dim:
            raise ConfigError(f"differential attention: {position.rotary_dim} rotated elements of a map of {self.head_dim}")
        self.position = position
        self._dtype = torch.bfloat16
        self.w_in = self.w_o = self.q_bias = self.k_bias = self.v_bias = None
        self.lam = 0.0

    # ---- sizes -----------------------------------------------------------
    def padded_head_dim(self) -> int:
        from ..kernels.ops import padded_head_size
        return padded_head_size(max(2 * self.head_dim, self.value_dim), self._dtype)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.padded_head_dim())

    def flops_per_query_key_pair(self):
        return 4 * 2 * self.num_heads * self.padded_head_dim()

    def weight_specs(self):
        W, H, G, D, E = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        specs = {"q": WeightSpec((H * 2 * D, W)), "k": WeightSpec((G * 2 * D, W)), "v": WeightSpec((G * E, W)),
                 "o": WeightSpec((W, H * E))}
        if self.has_bias:
            specs |= {"q.b": WeightSpec((H * 2 * D,), "norm_offset"), "k.b": WeightSpec((G * 2 * D,), "norm_offset"),
                      "v.b": WeightSpec((G * E,), "norm_offset")}
        for n in ("lq1", "lk1", "lq2", "lk2"):
            specs[n] = WeightSpec((D,), "norm_offset")
        if self.has_gate:
            specs["g"] = WeightSpec((H * E, W))
        return specs

    def load_weights(self, weights, dtype, device):
        self._dtype = dtype
        kind = weights["q"].dtype
        stacked = [weights["q"], weights["k"], weights["v"]] + ([weights["g"]] if self.has_gate else [])
        self.w_in = to_device(torch.cat([w.to(kind) for w in stacked], 0), dtype, device)
        self.w_o = to_device(weights["o"], dtype, device)
        f32 = lambda n: weights[n].to(torch.float32).contiguous().to(device)  # noqa: E731
        if self.has_bias:
            self.q_bias, self.k_bias, self.v_bias = f32("q.b"), f32("k.b"), f32("v.b")
        # one number for the layer, formed once, in float32
        l = {n: weights[n].to(torch.float32) for n in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = float(torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum())
                         + torch.tensor(self.diff, dtype=torch.float32))

    def forward(self, ctx, x):
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        H, G, D, E = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        P = kv.k_cache.shape[3]
        proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
        table = self.position.cached_table(ctx.max_positions, proj.device) if self.position is not None else None
        pairing = 1 if (self.position is not None and self.position.pairing == "interleaved") else 0
        q = ops.diff_qkv_store(proj, H, G, D, E, self.q_bias, self.k_bias, self.v_bias, table, pairing, b.positions, kv)
        a = ops.paged_attention(q, 2 * H, G, P, kv, b, 0, self.scale, softcap=self.softcap)
        gate = proj[:, 2 * H * D + 2 * G * D + G * E:] if self.has_gate else None
        o = ops.diff_combine(a, P, gate, self.lam, self.norm_eps, 1.0 - self.diff, H, E)
        return ops.linear(o, self.w_o, out_dtype=torch.float32, partials=True)
