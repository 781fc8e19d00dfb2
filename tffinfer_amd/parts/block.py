"""Arrangements of mixer, feed-forward and norms in a layer."""
from __future__ import annotations

from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """r = x + mixer(norm1(x));  out = r + ffn(norm2(r)).

    Reference: src/core/model/qwen3/QWen3Creator.cpp:62-65 (norm before the
    mixer), :140 (first residual sum), :142-148 (norm, feed-forward), :150-151
    (second sum).  Each sum is folded into the norm that follows it: the block
    hands the feed-forward's output on as a pending term, which the next
    block's first norm (or the model's final norm) adds.
    """

    graph_safe = True

    def __init__(self, mixer, feed_forward, make_norm):
        self.norm1 = make_norm()
        self.mixer = mixer
        self.feed_forward = feed_forward
        # (a layer without a feed-forward has no second sum; a second norm that a file holds all the same is
        # not run)
        self.has_ffn = not getattr(feed_forward, "is_none", False)
        self.norm2 = make_norm()
        if not self.has_ffn:
            self.norm2.optional = True

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    @staticmethod
    def _norm(norm, consumer, ctx, resid, pending):
        # a norm and a consumer that both say so may pass rows that still lack the norm's factor
        if getattr(norm, "for_linear_aware", False) and getattr(consumer, "input_goes_to_linear", False):
            return norm.forward(ctx, resid, pending, for_linear=True)
        return norm.forward(ctx, resid, pending)

    def forward(self, ctx, resid, pending):
        h = self._norm(self.norm1, self.mixer, ctx, resid, pending)
        a = self.mixer.forward(ctx, h)
        if not self.has_ffn:
            return a
        z = self._norm(self.norm2, self.feed_forward, ctx, resid, a)
        return self.feed_forward.forward(ctx, z)


@register_block("postnorm")
class PostNormBlock(Block):
    """x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ffn(x)): the norms stand after the
    sums, on the stream itself, and the sublayers read the stream as it is.  The float32
    residual stream therefore holds normed rows; each norm also leaves them in the activation
    type for the products that read them next, and the block hands that copy to the block
    after it through the step's batch.  A layer without a feed-forward has no second sum; its
    second norm runs only if the file holds a weight for it."""

    graph_safe = True

    def __init__(self, mixer, feed_forward, make_norm, alpha: float = 1.0):
        self.alpha = float(alpha)
        self.norm1 = make_norm()
        self.mixer = mixer
        self.norm2 = make_norm()
        self.feed_forward = feed_forward
        self.has_ffn = not getattr(feed_forward, "is_none", False)
        if not self.has_ffn:
            self.norm2.optional = True

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    def _rows(self, ctx, resid):
        """The stream in the activation type: what the block before left, or a cast."""
        if ctx.act_dtype == resid.dtype:
            return resid
        left = getattr(ctx.batch, "_normed_rows", None)
        if left is not None and left[0] is resid and left[1] == ctx.call_index - 1:
            return left[2]
        return ctx.ops.cast(resid, ctx.act_dtype)

    def forward(self, ctx, resid, pending):
        if pending is not None:
            resid += ctx.ops.as_tensor(pending)
        h = self._rows(ctx, resid)
        h = self.norm1.forward_post(ctx, resid, self.mixer.forward(ctx, h), self.alpha)
        if self.has_ffn:
            h = self.norm2.forward_post(ctx, resid, self.feed_forward.forward(ctx, h), self.alpha)
        elif self.norm2.weight is not None:
            h = self.norm2.forward_post(ctx, resid, None, self.alpha)
        ctx.batch._normed_rows = (resid, ctx.call_index, h)
        return None


@register_block("outnorm")
class OutputNormBlock(Block):
    """x <- x + norm1(mixer(x));  x <- x + norm2(ffn(x)): the sublayers read the stream itself and
    the norms stand on their *outputs*.  With ``depths`` (the number of layers plus one) the block
    also averages over the depth of the model: with X_0 the embedding's output and X_(i+1) what
    layer i leaves, the stream that goes on after layer ``depth`` is sum_{j <= depth + 1} dwa[j] * X_j
    (``dwa``: a tensor of the block, depth + 2 long).  The X_j of a step live in one tensor that
    the first layer makes and the step's batch carries.  A mixer that says ``reads_stream`` gets
    the float32 stream; every other sublayer a copy in the activation type, which the kernel
    before it leaves.  A layer without a feed-forward has no second sum and no second norm."""

    graph_safe = True

    def __init__(self, mixer, feed_forward, make_norm, depth: int = 0, depths: int = 0):
        self.depth = int(depth)
        self.depths = int(depths)
        if self.depths and not 0 <= self.depth < self.depths - 1:
            from ..config.base import ConfigError
            raise ConfigError(f"outnorm block: depth {self.depth} of a model of {self.depths - 1} layers")
        self.norm1 = make_norm()
        self.mixer = mixer
        self.norm2 = make_norm()
        self.feed_forward = feed_forward
        self.has_ffn = not getattr(feed_forward, "is_none", False)
        if not self.has_ffn:
            self.norm2.optional = True
        self.dwa = None
        self._one = None

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    def weight_specs(self):
        from .base import WeightSpec
        return {"dwa": WeightSpec((self.depth + 2,), "depth_coef")} if self.depths else {}

    def load_weights(self, weights, dtype, device):
        import torch
        if self.depths:
            self.dwa = weights["dwa"].to(torch.float32).contiguous().to(device)
            self._one = torch.ones(1, dtype=torch.float32, device=device)

    def _rows(self, ctx, resid):
        """The stream in the activation type: what the kernel before left, or a cast."""
        if ctx.act_dtype == resid.dtype:
            return resid
        left = getattr(ctx.batch, "_normed_rows", None)
        if left is not None and left[0] is resid and left[1] == ctx.call_index - 1:
            return left[2]
        return ctx.ops.cast(resid, ctx.act_dtype)

    def forward(self, ctx, resid, pending):
        import torch
        ops = ctx.ops
        if pending is not None:
            resid += ops.as_tensor(pending)
        act = None if ctx.act_dtype == torch.float32 else ctx.act_dtype
        hist = None
        if self.depths:
            kept = getattr(ctx.batch, "_depth_history", None)
            if self.depth == 0 or kept is None or kept[0] is not resid:
                if self.depth != 0:
                    raise RuntimeError("outnorm block: the step's earlier layers left no history of the stream")
                hist = torch.empty(self.depths, *resid.shape, dtype=torch.float32, device=resid.device)
                ctx.batch._depth_history = (resid, hist)
                h = ops.depth_average(hist, 1, self._one, resid, act)       # X_0 is kept; the stream stays
                h = resid if h is None else h
            else:
                hist = kept[1]
                h = self._rows(ctx, resid)
        else:
            h = self._rows(ctx, resid)
        a = self.mixer.forward(ctx, resid if getattr(self.mixer, "reads_stream", False) else h)
        h = self.norm1.forward_add(ctx, resid, a)
        if self.has_ffn:
            h = self.norm2.forward_add(ctx, resid, self.feed_forward.forward(ctx, h))
        if hist is not None:
            h = ops.depth_average(hist, self.depth + 2, self.dwa, resid, act)
            h = resid if h is None else h
        ctx.batch._normed_rows = (resid, ctx.call_index, h)
        return None


@register_block("parallel")
class ParallelBlock(Block):
    """x <- x + (mixer(norm1(x)) + ffn(norm2(x))): both sublayers read the same x, each through a norm
    of its own.  The two outputs stay pending for the block after it (or the model's last norm), whose
    first kernel adds them to the stream and forms its two norms in one pass; a row the run order asks to
    be added to the stream before this call (``ctx.stream_offset``) rides in the same pass.  A layer
    without a feed-forward has no second norm."""

    graph_safe = True
    #: the block adds ``ctx.stream_offset`` to the stream itself
    takes_stream_offset = True

    def __init__(self, mixer, feed_forward, make_norm):
        self.norm1 = make_norm()
        self.mixer = mixer
        self.norm2 = make_norm()
        self.feed_forward = feed_forward
        self.has_ffn = not getattr(feed_forward, "is_none", False)
        if not self.has_ffn:
            self.norm2.optional = True
        for n in (self.norm1, self.norm2):
            if not hasattr(n, "weight") or not hasattr(n, "eps") or getattr(n, "groups", 1) != 1:
                from ..config.base import ConfigError
                raise ConfigError("parallel block: its norms are RMS norms over the whole row")

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    def forward(self, ctx, resid, pending):
        ops = ctx.ops
        h1, h2 = ops.add_rmsnorm_pair(resid, pending, getattr(ctx, "stream_offset", None), self.norm1.weight,
                                      self.norm2.weight if self.has_ffn else None, self.norm1.eps, ctx.act_dtype)
        a = self.mixer.forward(ctx, h1)
        if not self.has_ffn:
            return a
        return ops.PendingTerms([a, self.feed_forward.forward(ctx, h2)])
