"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import FeedForward, WeightSpec, register_feed_forward, to_device


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """f = (silu(z Wgate^T) * (z Wup^T)) Wdown^T, no biases.

    Reference: src/core/model/base/ModelCreatorBase.cpp:51-94 (up, gate, the
    unary op with x1 = gate, x2 = up, down), src/kernel/cuda/unary.cu:10-27.
    Gate and up are put into one matrix at load so that one product streams both.
    """

    graph_safe = True
    #: the input is used by ``ops.linear`` and by nothing else
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)       # how the files call gate, up and down
        if len(self.names) != 3:
            from ..config.base import ConfigError
            raise ConfigError("swiglu: 'names' are the names of gate, up and down")
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {
            self.names[0]: WeightSpec((I, H)),
            self.names[1]: WeightSpec((I, H)),
            self.names[2]: WeightSpec((H, I)),
        }

    def load_weights(self, weights, dtype, device):
        gate, up = weights[self.names[0]], weights[self.names[1]]
        if dtype == torch.bfloat16 and torch.device(device).type == "cuda":
            # bfloat16: gate and up rows interleaved in groups of 16 in one weight, so that one
            # product streams both and applies silu(gate) * up to its float32 accumulators
            from ..kernels import ops
            self.w_gate_up = ops.pack_gate_up(gate.to(dtype).contiguous().to(device),
                                              up.to(dtype).contiguous().to(device))
        else:
            # float32: gate and up stacked to [2I, H]; the activation is a kernel of its own
            self.w_gate_up = to_device(torch.cat([gate, up], 0), dtype, device)
        self.w_down = to_device(weights[self.names[2]], dtype, device)

    def forward(self, ctx, x):
        gu = ctx.ops.linear(x, self.w_gate_up)
        m = gu if getattr(self.w_gate_up, "glu_out", 0) else ctx.ops.swiglu(gu)
        return ctx.ops.linear(m, self.w_down, out_dtype=torch.float32, partials=True)


@register_feed_forward("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: the block leaves the sublayer out."""

    graph_safe = True
    is_none = True

    def __init__(self, hidden_size: int = 0):
        self.hidden_size = int(hidden_size)

    def forward(self, ctx, x):
        return None


@register_feed_forward("gelu_mlp")
class GeluMLP(FeedForward):
    """f = Wdown act(Wup z), no gate and no biases.  ``activation`` "gelu": the exact one,
    0.5 z (1 + erf(z / sqrt 2)), or with ``tanh_form`` its tanh approximation; "relu2": the
    square of relu, max(z, 0)^2."""

    graph_safe = True
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, intermediate_size: int, tanh_form: bool = False, activation: str = "gelu"):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.tanh_form = bool(tanh_form)
        self.activation = str(activation)
        if self.activation not in ("gelu", "relu2"):
            from ..config.base import ConfigError
            raise ConfigError(f"feed-forward: unknown activation '{activation}' (gelu, relu2)")
        self.w_up = self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"up": WeightSpec((I, H)), "down": WeightSpec((H, I))}

    def load_weights(self, weights, dtype, device):
        self.w_up = to_device(weights["up"], dtype, device)
        self.w_down = to_device(weights["down"], dtype, device)

    def forward(self, ctx, x):
        u = ctx.ops.linear(x, self.w_up)
        a = ctx.ops.relu_squared(u) if self.activation == "relu2" else ctx.ops.gelu(u, self.tanh_form)
        return ctx.ops.linear(a, self.w_down, out_dtype=torch.float32, partials=True)


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    """``num_experts`` small gated feed-forwards of which every token uses ``top``.

        s = sigmoid(Wr z)                      (float32)
        chosen: the ``top`` largest s + b      (b: a correction that moves the choice only)
        w_e = s_e / (sum of the chosen s + 1e-20)
        expert e: g = min(Wg z, limit), u = clamp(Wu z, -limit, limit),
                  y = g * sigmoid(act_alpha * g) * (u + 1),  f_e = Wd y
        f = sum over the chosen e of w_e f_e

    ``router_softmax``: s = softmax(Wr z) over all experts instead, and w_e = s_e as it is.
    ``normalize`` False: w_e = s_e as it is (the sigmoid's scores, not made to add up to one).
    ``limit`` None: no clamp; ``up_offset`` 0 and ``act_alpha`` 1: y = silu(g) * u.
    ``weight_input``: the weight multiplies what goes into the expert, f = sum of expert_e(w_e z),
    instead of what comes out.

    The experts' matrices lie stacked, [experts, out, in], so that a kernel finds an expert's
    rows by its number."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 limit: float | None, act_alpha: float = 1.702, correction: bool = True,
                 router_softmax: bool = False, up_offset: float = 1.0, normalize: bool = True,
                 weight_input: bool = False):
        self.router_softmax = bool(router_softmax)
        self.normalize = bool(normalize)
        self.weight_input = bool(weight_input)
        self.up_offset = float(up_offset)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.num_experts = int(num_experts)
        self.top = int(top)
        self.limit = float("inf") if limit is None else float(limit)
        self.act_alpha = float(act_alpha)
        self.has_correction = bool(correction)
        if not 0 < self.top <= self.num_experts:
            from ..config.base import ConfigError
            raise ConfigError(f"routed experts: top={self.top} of {self.num_experts} experts")
        self.w_gate = self.w_up = self.w_down = self.router = self.router_w = self.correction = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        specs = {"router": WeightSpec((self.num_experts, H))}
        if self.has_correction:
            specs["correction"] = WeightSpec((self.num_experts,), "vector")
        for e in range(self.num_experts):
            specs[f"e{e}.gate"] = WeightSpec((I, H))
            specs[f"e{e}.up"] = WeightSpec((I, H))
            specs[f"e{e}.down"] = WeightSpec((H, I))
        return specs

    def active_matrix_elements(self) -> int:
        """Matrix elements a token multiplies with: the router and its ``top`` experts."""
        H, I = self.hidden_size, self.intermediate_size
        return self.num_experts * H + self.top * 3 * H * I

    def streamed_matrix_elements(self, rows: int) -> int:
        """Matrix elements a step of ``rows`` tokens reads at least: the router and as many
        experts as the tokens can choose between them."""
        H, I = self.hidden_size, self.intermediate_size
        return self.num_experts * H + min(self.num_experts, rows * self.top) * 3 * H * I

    def load_weights(self, weights, dtype, device):
        E = self.num_experts

        def stack(which):
            from ..kernels.ops import pad_expert_rows
            return pad_expert_rows(torch.stack([weights[f"e{e}.{which}"].to(dtype) for e in range(E)], 0)).to(device)

        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        # The router's logits are float32 sums.  A router stored in bfloat16 multiplies exactly with
        # bfloat16 rows on the matrix cores (the products of two bfloat16 numbers are float32 numbers,
        # the sums are float32): the engine's own product serves.  One stored in more bits keeps them,
        # and the routing kernel forms the logits itself.
        self.router_w = None
        if dtype == torch.float32 or weights["router"].dtype == torch.bfloat16:
            self.router_w = to_device(weights["router"], dtype, device)
        self.router = weights["router"].to(torch.float32).contiguous().to(device) if self.router_w is None else None
        self.correction = (weights["correction"].to(torch.float32).contiguous().to(device)
                           if self.has_correction else None)

    def forward(self, ctx, x):
        ops = ctx.ops
        x = ops.as_tensor(x)
        if self.router_w is not None:
            idx, wts = ops.route_topk(None, None, self.correction, self.top,
                                      logits=ops.linear(x, self.router_w, out_dtype=torch.float32),
                                      softmax=self.router_softmax, normalize=self.normalize)
        else:
            idx, wts = ops.route_topk(x, self.router, self.correction, self.top, softmax=self.router_softmax,
                                      normalize=self.normalize)
        return ops.routed_experts(x, self.w_gate, self.w_up, self.w_down, idx, wts, self.limit, self.act_alpha,
                                  up_offset=self.up_offset, weight_input=self.weight_input)


@register_feed_forward("table_experts")
class TableExperts(FeedForward):
    """``num_experts`` small feed-forwards without a gate, f_e = Wd max(Wu z, 0)^2, of which every token
    uses ``top``: a table over the vocabulary (int32 [vocab, top], the entries of a row differ) names them
    by the token's id, and each counts 1 / top.  There is no router.  The experts' matrices lie stacked,
    [experts, out, in], as those of ``RoutedExperts``, and run on the same kernels."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, vocab_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.num_experts = int(num_experts)
        self.top = int(top)
        self.vocab_size = int(vocab_size)
        if not 0 < self.top <= self.num_experts:
            from ..config.base import ConfigError
            raise ConfigError(f"table experts: top={self.top} of {self.num_experts} experts")
        self.w_up = self.w_down = self.table = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        specs = {"table": WeightSpec((self.vocab_size, self.top), "index_table", bound=self.num_experts)}
        for e in range(self.num_experts):
            specs[f"e{e}.up"] = WeightSpec((I, H))
            specs[f"e{e}.down"] = WeightSpec((H, I))
        return specs

    def active_matrix_elements(self) -> int:
        return self.top * 2 * self.hidden_size * self.intermediate_size

    def streamed_matrix_elements(self, rows: int) -> int:
        return min(self.num_experts, rows * self.top) * 2 * self.hidden_size * self.intermediate_size

    def load_weights(self, weights, dtype, device):
        from ..kernels.ops import pad_expert_rows
        E = self.num_experts

        def stack(which):
            return pad_expert_rows(torch.stack([weights[f"e{e}.{which}"].to(dtype) for e in range(E)], 0)).to(device)

        self.w_up, self.w_down = stack("up"), stack("down")
        table = weights["table"].to(torch.int32)
        if int(table.min()) < 0 or int(table.max()) >= E:
            from ..config.base import ConfigError
            raise ConfigError(f"table experts: the table names experts outside 0 .. {E - 1}")
        self.table = table.contiguous().to(device)

    def forward(self, ctx, x):
        ops = ctx.ops
        x = ops.as_tensor(x)
        idx, wts = ops.route_by_table(self.table, ctx.batch.token_ids, self.num_experts)
        return ops.routed_experts(x, None, self.w_up, self.w_down, idx, wts, float("inf"), 1.0, up_offset=0.0)
