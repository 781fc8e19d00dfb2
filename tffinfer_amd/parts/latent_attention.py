"""Attention whose keys and values are kept as one low-rank latent vector per token."""
from __future__ import annotations

import torch

from ..config.base import ConfigError, PartSpec
from .base import (POSITION_ENCODINGS, KVCacheSpec, Mixer, PositionEncoding, WeightSpec,
                   register_mixer, to_device)


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Per token t with input h:

        q_h   = (Wq h)[head h] = [q_h^n (head_dim) | q_h^r (rot_dim)]
        [a|b] = Wdkv h,  c = rmsnorm(a) * w_c  (kv_rank),  kr = b (rot_dim; shared by all heads)
        k_h^n = Wuk_h c,  v_h = Wuv_h c
        s_h(i, j) = (q_h^n(i) . k_h^n(j) + R_i q_h^r(i) . R_j kr(j)) * scale,  0 <= i - j < window
        p_h(i, .) = softmax over the visible j and one sink term e^(sink_h) in the denominator
        out = Wo [ (sum_j p_h(i, j) v_h(j)) * sigmoid(Wg h)[head h] ]_h

    R_p rotates pairs of the rotated part by the position's angles, (2i, 2i+1) or (i, i + dims/2) as the
    position encoding says.  With ``q_rank`` the queries pass a latent vector too: c_q = rmsnorm(Wdq h) * w_q,
    q = Wuq c_q (tensors ``dq``, ``dq.norm``, ``uq`` in place of ``q``).  ``shared_cache``: the layer has no
    Wdkv; it reads c and R kr from the cache that another layer call fills (the run order names it), with
    its own Wuk, Wuv and queries.  Only c and R kr are cached.  The
    up-projections are taken to the query's side (q_h^n . Wuk_h c = (Wuk_h^T q_h^n) . c, and
    sum_j p v_h(j) = Wuv_h sum_j p c(j)), so the attention proper is attention with one key
    head of size kv_rank + rot_dim whose values are the first kv_rank elements of its keys; it
    runs on the paged attention kernels, padded to a head size they take.  Wq (or Wdq), Wdkv and Wg are
    one product; with a latent vector on the queries' side its result stays float32 for the two norms,
    which are one launch with the rotation and the cache writes.
    """

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int,
                 kv_rank: int, scale: float, position=None, window: int = 0,
                 latent_norm_eps: float = 1e-6, sink: bool = True, output_gate: bool = True,
                 q_rank: int | None = None, shared_cache: bool = False):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.rot_dim = int(rot_dim)
        self.value_dim = int(value_dim)
        self.kv_rank = int(kv_rank)
        self.scale = float(scale)
        self.window = int(window or 0)
        self.latent_norm_eps = float(latent_norm_eps)
        self.has_sink = bool(sink)
        self.has_gate = bool(output_gate)
        self.q_rank = int(q_rank) if q_rank else 0
        self.shared_cache = bool(shared_cache)
        if q_rank is not None and self.q_rank <= 0:
            raise ConfigError(f"latent attention: 'q_rank' must be positive, found {q_rank}")
        if self.shared_cache and not self.q_rank:
            raise ConfigError("latent attention: a layer that reads another layer's cache forms its queries "
                              "through a latent vector")
        for k in ("hidden_size", "num_heads", "head_dim", "value_dim", "kv_rank"):
            if getattr(self, k) <= 0:
                raise ConfigError(f"latent attention: '{k}' must be positive, found {getattr(self, k)}")
        if self.rot_dim < 0:
            raise ConfigError(f"latent attention: 'rot_dim' must not be negative, found {self.rot_dim}")
        if isinstance(position, PartSpec):
            position = POSITION_ENCODINGS.build(position)
        if position is not None and not isinstance(position, PositionEncoding):
            raise ConfigError("latent attention: 'position' must be a position encoding or its spec")
        if position is not None and position.rotary_dim:
            if position.rotary_dim > self.rot_dim:
                raise ConfigError(f"latent attention: {position.rotary_dim} rotated dimensions of a part of {self.rot_dim}")
        self.position = position
        self._dtype = torch.bfloat16
        self.w_in = self.w_uk_t = self.w_uv_t = self.w_o = self.latent_norm = self.sink = None
        self.w_uq = self.w_g = self.q_latent_norm = None

    # ---- sizes -----------------------------------------------------------
    @property
    def key_dim(self) -> int:
        return self.kv_rank + self.rot_dim

    def padded_key_dim(self) -> int:
        from ..kernels.ops import padded_head_size
        return padded_head_size(self.key_dim, self._dtype)

    def cache_spec(self):
        return KVCacheSpec(1, self.padded_key_dim(), self.window)

    def flops_per_query_key_pair(self):
        return 4 * self.num_heads * self.padded_key_dim()

    def weight_specs(self):
        W, H = self.hidden_size, self.num_heads
        specs = {}
        if self.q_rank:
            specs["dq"] = WeightSpec((self.q_rank, W))
            specs["dq.norm"] = WeightSpec((self.q_rank,), "norm")
            specs["uq"] = WeightSpec((H * (self.head_dim + self.rot_dim), self.q_rank))
        else:
            specs["q"] = WeightSpec((H * (self.head_dim + self.rot_dim), W))
        if not self.shared_cache:
            specs["dkv"] = WeightSpec((self.key_dim, W))
            specs["dkv.norm"] = WeightSpec((self.kv_rank,), "norm")
        specs |= {
            "uk": WeightSpec((H * self.head_dim, self.kv_rank)),
            "uv": WeightSpec((H * self.value_dim, self.kv_rank)),
            "o": WeightSpec((W, H * self.value_dim)),
        }
        if self.has_sink:
            specs["sink"] = WeightSpec((H,), "vector")
        if self.has_gate:
            specs["g"] = WeightSpec((H * self.value_dim, W))
        return specs

    def load_weights(self, weights, dtype, device):
        H = self.num_heads
        self._dtype = dtype
        if self.q_rank:
            # (the joint product's result stays float32 for the norms; a gate is a product of its own then)
            stacked = [weights["dq"]] + ([] if self.shared_cache else [weights["dkv"]])
            self.w_uq = to_device(weights["uq"], dtype, device)
            self.q_latent_norm = weights["dq.norm"].to(torch.float32).contiguous().to(device)
            self.w_g = to_device(weights["g"], dtype, device) if self.has_gate else None
        else:
            stacked = [weights["q"], weights["dkv"]] + ([weights["g"]] if self.has_gate else [])
        self.w_in = to_device(torch.cat([w.to(stacked[0].dtype) for w in stacked], 0), dtype, device)
        self.w_o = to_device(weights["o"], dtype, device)
        # per head [outputs, inputs]: k_h^n = Wuk_h c, so (Wuk_h^T q)[r] = sum_d Wuk[h, d, r] q[d]: [H, rank, head_dim]
        self.w_uk_t = weights["uk"].to(dtype).view(H, self.head_dim, self.kv_rank).transpose(1, 2).contiguous().to(device)
        # v_h[e] = sum_r Wuv[h, e, r] c[r]: [H, value_dim, rank], as stored
        self.w_uv_t = weights["uv"].to(dtype).view(H, self.value_dim, self.kv_rank).contiguous().to(device)
        self.latent_norm = (None if self.shared_cache else
                            weights["dkv.norm"].to(torch.float32).contiguous().to(device))
        self.sink = weights["sink"].to(torch.float32).contiguous().to(device) if self.has_sink else None

    def forward(self, ctx, x):
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        H, rank, rot = self.num_heads, self.kv_rank, self.rot_dim
        nq = H * (self.head_dim + rot)
        Dp = kv.k_cache.shape[3]
        table, pairing = None, 1
        if self.position is not None and self.position.rotary_dim:
            table = self.position.cached_table(ctx.max_positions, x.device)
            pairing = 1 if self.position.pairing == "interleaved" else 0
        if self.q_rank:
            qr = self.q_rank
            proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
            cq = ops.latent_kv_store(None if self.shared_cache else proj[:, qr:qr + rank + rot], rank, rot,
                                     self.latent_norm, self.latent_norm_eps, table, b.positions, kv.slot_mapping,
                                     kv.k_cache, kv.v_cache, pairing=pairing, q_latent=proj[:, :qr],
                                     q_norm_w=self.q_latent_norm)
            q_in = ops.linear(cq, self.w_uq)
            gate = ops.linear(x, self.w_g) if self.has_gate else None
        else:
            proj = ops.linear(x, self.w_in)
            ops.latent_kv_store(proj[:, nq:nq + rank + rot], rank, rot, self.latent_norm, self.latent_norm_eps, table,
                                b.positions, kv.slot_mapping, kv.k_cache, kv.v_cache, pairing=pairing)
            q_in = proj[:, :nq]
            gate = proj[:, nq + rank + rot:] if self.has_gate else None
        q = ops.head_linear(q_in, self.head_dim + rot, self.w_uk_t, out_head=Dp, tail=rot, cos_sin=table,
                            positions=b.positions, pairing=pairing)
        o = ops.paged_attention(q, H, 1, Dp, kv, b, self.window, self.scale, sinks=self.sink)
        o = ops.head_linear(o, Dp, self.w_uv_t, gate=gate)
        return ops.linear(o, self.w_o, out_dtype=torch.float32, partials=True)
