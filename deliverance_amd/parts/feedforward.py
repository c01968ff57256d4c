"""Dense feed-forward: fc (+ bias), activation, proj (+ bias), added into the residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/MLPBlock.java:250-321 (the
two-bias, no-gate form GPT-2 uses, :93-114); residual add TransformerBlock.java:188."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, StepContext, register_feed_forward, to_matrix, to_vector


class DenseFeedForward(FeedForward):
    graph_safe = True
    can_store = True          # with ``ctx.part_accumulate`` off the second product stores instead of adding

    def __init__(self, spec, params, dtype, device):
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}")
        self.fc_weight = to_matrix(params["fc_weight"], dtype, device)
        self.proj_weight = to_matrix(params["proj_weight"], dtype, device)
        self.fc_bias = to_vector(params.get("fc_bias"), dtype, device) if spec.bias else None
        self.proj_bias = to_vector(params.get("proj_bias"), dtype, device) if spec.bias else None
        if tuple(self.fc_weight.shape) != (self.inner, self.width):
            raise ValueError(f"fc weight is {list(self.fc_weight.shape)}, expected {[self.inner, self.width]}")
        if tuple(self.proj_weight.shape) != (self.width, self.inner):
            raise ValueError(f"proj weight is {list(self.proj_weight.shape)}, expected {[self.width, self.inner]}")

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor) -> bool:
        """Small steps: LayerNorm, fc, bias and activation in one kernel."""
        N = x.shape[0]
        ln = norm.fusable_params()
        if ln is None or not ops.can_fuse_ln(N, x, self.fc_weight):
            return False
        gain, bias, eps = ln
        mid = ctx.buf("ff_mid", N, self.inner, ctx.dtype)
        ops.linear_ln(x, None, N, gain, bias, eps, self.fc_weight, self.fc_bias, mid, act=self.activation)
        ops.linear(mid, self.proj_weight, self.proj_bias, x, accumulate=True)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        N = h.shape[0]
        mid = ctx.buf("ff_mid", N, self.inner, ctx.dtype)
        ops.linear(h, self.fc_weight, self.fc_bias, mid, act=self.activation)
        ops.linear(mid, self.proj_weight, self.proj_bias, x, accumulate=ctx.part_accumulate)


register_feed_forward("dense", DenseFeedForward)


class GatedFeedForward(FeedForward):
    """``down(act(gate h) * (up h))`` without biases; gate and up are one matrix [2 inner, width] (gate rows
    first), so one product reads h once."""
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        self.limit = float(getattr(spec, "limit", 0.0) or 0.0)
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}")
        if self.activation == "glu_capped" and not (self.limit > 0.0):
            raise ValueError(f"the capped gated form needs a positive limit, found {self.limit}")
        self.gate_up_weight = to_matrix(params["gate_up_weight"], dtype, device)
        self.down_weight = to_matrix(params["down_weight"], dtype, device)
        if tuple(self.gate_up_weight.shape) != (2 * self.inner, self.width):
            raise ValueError(f"gate|up weight is {list(self.gate_up_weight.shape)}, expected {[2 * self.inner, self.width]}")
        if tuple(self.down_weight.shape) != (self.width, self.inner):
            raise ValueError(f"down weight is {list(self.down_weight.shape)}, expected {[self.width, self.inner]}")

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        N = h.shape[0]
        mid = ctx.buf("ff_mid", N, self.inner, ctx.dtype)
        ops.gated_linear(ctx, h, self.gate_up_weight, mid, self.activation, self.limit)
        ops.linear(mid, self.down_weight, None, x, accumulate=ctx.part_accumulate)


class ExpertsFeedForward(FeedForward):
    """A mixture of experts (``ExpertsFeedForwardSpec``).  The router says which ``top`` experts a token uses and
    with what weights.  ``token_table``: row ``token id`` of an integer table names them, each with weight 1 / top.
    ``logistic_top``: 32-bit logits from a matrix; the ``top`` largest logistic scores, which are the weights.
    ``softmax_top``: 32-bit logits from a matrix and a bias; the ``top`` largest logits, weighted by the softmax over
    just those.
    The step's (token, choice) pairs are laid out expert by expert on the device (``ops.moe_route``), two grouped
    products run over that layout, and the pairs' results are added up per token; a weight on the input scales
    the pair's row in the first product.  A shared expert, if any, runs as a dense feed-forward for every token.
    Nothing is read back to the host, so a step can be recorded."""
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        self.n_experts, self.top, self.router = spec.n_experts, spec.top, spec.router
        self.gated = bool(getattr(spec, "gated", True))
        self.weight_on = getattr(spec, "weight_on", "output")
        self.renormalize = bool(getattr(spec, "renormalize", False))
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}")
        self.limit = float(getattr(spec, "limit", 0.0) or 0.0)
        if self.router not in ("token_table", "logistic_top", "softmax_top"):
            raise ValueError(f"unknown router {self.router!r}; known: 'token_table', 'logistic_top', 'softmax_top'")
        if self.activation == "glu_capped" and not (self.gated and self.limit > 0.0):
            raise ValueError(f"the capped gated form needs gated experts and a positive limit, found {self.limit}")
        if self.weight_on not in ("output", "input"):
            raise ValueError(f"a pair's weight goes on the 'output' or the 'input', not {self.weight_on!r}")
        if not (1 <= self.top <= self.n_experts):
            raise ValueError(f"top {self.top} of {self.n_experts} experts")
        first_rows = (2 if self.gated else 1) * self.inner
        # [experts, 2 inner | inner, width]: gate | up, or up alone
        self.gate_up_weight = to_matrix(params["gate_up_weight" if self.gated else "up_weight"], dtype, device)
        self.down_weight = to_matrix(params["down_weight"], dtype, device)             # [experts, width, inner]
        if tuple(self.gate_up_weight.shape) != (self.n_experts, first_rows, self.width):
            raise ValueError(f"experts' first weights are {list(self.gate_up_weight.shape)}, expected "
                             f"{[self.n_experts, first_rows, self.width]}")
        if tuple(self.down_weight.shape) != (self.n_experts, self.width, self.inner):
            raise ValueError(f"experts' down weights are {list(self.down_weight.shape)}, expected "
                             f"{[self.n_experts, self.width, self.inner]}")
        self.table = self.router_weight = None
        if self.router == "token_table":
            table = params["table"]
            if table.dim() != 2 or table.shape[1] != self.top or (spec.vocab_size and table.shape[0] != spec.vocab_size):
                raise ValueError(f"expert table is {list(table.shape)}, expected {[spec.vocab_size or 'vocab', self.top]}")
            if table.dtype not in (torch.int32, torch.int64) or int(table.min()) < 0 or int(table.max()) >= self.n_experts:
                raise ValueError(f"expert table must hold integers in 0..{self.n_experts - 1}")
            self.table = table.to(device=device, dtype=torch.int32).contiguous()
            if self.weight_on != "output":
                raise ValueError("a table router gives no weight to put on the input")
        else:
            self.router_weight = to_matrix(params["router_weight"], dtype, device)     # [experts, width]
            if tuple(self.router_weight.shape) != (self.n_experts, self.width):
                raise ValueError(f"router weight is {list(self.router_weight.shape)}, expected {[self.n_experts, self.width]}")
        self.router_bias = None
        if getattr(spec, "router_bias", False):
            self.router_bias = params["router_bias"].to(device=device, dtype=torch.float32).contiguous()
            if self.router_bias.numel() != self.n_experts:
                raise ValueError(f"the router's bias has {self.router_bias.numel()} entries for {self.n_experts} experts")
        self.weight = 1.0 / self.top
        self.last_choice = None
        self.shared = None
        if getattr(spec, "shared_inner", 0) and getattr(spec, "shared_gated", False):
            from ..config.specs import GatedFeedForwardSpec
            self.shared = GatedFeedForward(
                GatedFeedForwardSpec("gated", self.width, spec.shared_inner, spec.shared_activation or self.activation,
                                     limit=float(getattr(spec, "shared_limit", 0.0) or 0.0)),
                {"gate_up_weight": params["shared_gate_up_weight"], "down_weight": params["shared_down_weight"]}, dtype, device)
        elif getattr(spec, "shared_inner", 0):
            from ..config.specs import DenseFeedForwardSpec
            self.shared = DenseFeedForward(
                DenseFeedForwardSpec("dense", self.width, spec.shared_inner, spec.shared_activation or self.activation,
                                     bias=False),
                {"fc_weight": params["shared_up_weight"], "proj_weight": params["shared_down_weight"]}, dtype, device)

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        ids = weights = None
        if self.router_weight is not None:
            N = h.shape[0]
            z = ctx.buf("moe_logits", N, self.n_experts, torch.float32)      # 32-bit sums of the products
            ops.linear(h, self.router_weight, None, z)
            ids = ctx.buf("moe_ids", N, self.top, torch.int32)
            weights = ctx.buf("moe_weights", N, self.top, torch.float32)
            if self.router == "softmax_top":
                ops.moe_top(z, self.router_bias, self.top, "softmax", False, ids, weights)
            else:
                ops.moe_top(z, self.router_bias, self.top, "logistic", self.renormalize, ids, weights)
        self.last_choice = ids if ctx.debug_hook is not None else None      # handed to the layer debug hook
        ops.experts_forward(ctx, h, self.table, self.gate_up_weight, self.down_weight, self.n_experts, self.top,
                            self.weight, self.activation, x, accumulate=ctx.part_accumulate, ids=ids,
                            pair_weights=weights, gated=self.gated, weight_input=self.weight_on == "input",
                            limit=self.limit)
        if self.shared is not None:
            keep = ctx.part_accumulate
            ctx.part_accumulate = True          # the shared expert joins the experts' sum, stored or added above
            try:
                self.shared.forward(ctx, h, x)
            finally:
                ctx.part_accumulate = keep


register_feed_forward("gated", GatedFeedForward)
register_feed_forward("experts", ExpertsFeedForward)
