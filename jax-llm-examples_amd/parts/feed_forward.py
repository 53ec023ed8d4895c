"""Feed-forward parts.

``dense_swiglu``: ``(silu(x Wg) * (x Wu)) Wd`` (``llama4/llama4_jax/model.py:1142-1153``).
``moe_sigmoid_shared``: router logits in float32, the ``top_k`` largest per token,
gate = sigmoid of the chosen logit, the gate multiplies the expert's *input*
(``model.py:958-972, 1066-1071``), SwiGLU experts (``model.py:1076-1085``), sum
over the chosen experts (``model.py:1111``), plus one shared SwiGLU expert on the
unscaled input (``model.py:1137-1139``).  With the option ``shared_gate`` (off for Llama 4) the shared expert's output
is multiplied by ``sigmoid(w_sg . h)``, one number a token, formed in float32.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("dense_swiglu")
class DenseSwiGLU(FeedForward):
    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.inter = int(spec.intermediate_size)
        self.activation = str(spec.get("activation") or "silu")
        if self.activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"unknown activation {self.activation!r} (silu, gelu_tanh)")

    def param_specs(self):
        return {
            "w_gate_up": ParamSpec((2 * self.inter, self.hidden)),  # gate rows, then up rows
            "w_down": ParamSpec((self.hidden, self.inter)),
        }

    graph_safe = True

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        ops = ctx.ops
        if self.activation == "silu":
            return ops.linear(ops.swiglu_linear(h, self.params["w_gate_up"]), self.params["w_down"])
        return ops.linear(ops.swiglu_linear(h, self.params["w_gate_up"], activation=self.activation),
                          self.params["w_down"])


@register_feed_forward("moe_sigmoid_shared")
class MoESigmoidShared(FeedForward):
    wants_float32_input = True
    # h and h32 go to the kernel set's router and expert products only, which take rows that are not computed yet
    # (the router of a step of few tokens does addition, norm, logits, choice and grouping in one launch)
    accepts_deferred_norm = True

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_experts = int(spec.num_experts)
        self.top_k = int(spec.top_k)
        self.inter = int(spec.intermediate_size)
        self.shared_inter = int(spec.get("shared_intermediate_size") or 0)
        self.shared_gate = bool(spec.get("shared_gate", False))
        if self.shared_gate and not self.shared_inter:
            raise ValueError("a shared expert's gate needs a shared expert")
        self.tiled = False  # expert matrices are in the kernels' streaming layout (ops/layout.py)

    def param_specs(self):
        e, f, d = self.num_experts, self.inter, self.hidden
        specs = {
            "router": ParamSpec((e, d), policy="float32"),
            "w_gate_up": ParamSpec((e, 2 * f, d)),  # per expert [out, in]: gate rows, then up rows
            "w_down": ParamSpec((e, d, f)),
        }
        if self.shared_inter:
            specs["shared_gate_up"] = ParamSpec((2 * self.shared_inter, d))
            specs["shared_down"] = ParamSpec((d, self.shared_inter))
        if self.shared_gate:
            specs["shared_gate"] = ParamSpec((1, d), policy="float32")
        return specs

    graph_safe = True

    def step_weight_bytes(self, observed=None) -> int:
        """Of the routed experts only those that some token of the step chose (``observed``: the
        ``(expert ids, gates)`` this part handed to the step's tap; without it, all)."""
        n = self.num_experts if observed is None else int(torch.unique(observed[0]).numel())
        total = 0
        for name, t in self.params.items():
            b = t.numel() * t.element_size()
            total += b // self.num_experts * n if name in ("w_gate_up", "w_down") else b
        return total

    def flops_per_token(self) -> float:
        per = 0
        for name, t in self.params.items():
            per += t.numel() // self.num_experts * self.top_k if name in ("w_gate_up", "w_down") else t.numel()
        return 2.0 * per

    def finalize(self) -> None:
        from ..ops.layout import can_tile, tile_

        gu, dn = self.params["w_gate_up"], self.params["w_down"]
        if not self.tiled and can_tile(gu) and can_tile(dn) and self.inter % 16 == 0:
            tile_(gu)
            tile_(dn)
            self.tiled = True

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        ops = ctx.ops
        expert_ids, gates, grouping = ops.moe_route(h32, self.params["router"], self.top_k, group=True)
        tap = getattr(ctx, "tap", None)
        if tap is not None:  # whoever watches the step sees the choice and may replace it
            replaced = tap(self, "routing", (expert_ids, gates))
            if replaced is not None:
                expert_ids, gates = replaced
                grouping = None
        shared = (self.params["shared_gate_up"], self.params["shared_down"]) if self.shared_inter else None
        if self.shared_gate:
            return ops.moe_experts(h, expert_ids, gates, self.params["w_gate_up"], self.params["w_down"],
                                   shared_weights=shared, tiled=self.tiled, grouping=grouping,
                                   shared_gate=(h32, self.params["shared_gate"]))
        return ops.moe_experts(h, expert_ids, gates, self.params["w_gate_up"], self.params["w_down"],
                               shared_weights=shared, tiled=self.tiled, grouping=grouping)


@register_feed_forward("moe_scored")
class MoEScored(FeedForward):
    """Routed experts whose weights are scores, not gates on the input: router logits ``z = W_r h`` in float32,
    scores ``s = sigmoid(z)``; the ``top_k`` experts with the largest *choice scores* ``s + correction`` (a learned
    number per expert; option ``correction``) are chosen, lowest index first among equals, and the output is ``sum_e
    s_e expert_e(h)`` with the scores as they are (no renormalisation).  With ``groups``: the experts form that many
    equal groups of neighbours, a group's score is the sum of its ``group_score_terms`` largest choice scores, and
    only experts of the ``keep_groups`` best groups can be chosen.  An expert is ``W_down act(W_up h)`` without
    biases; ``activation``: ``relu2`` (the square of relu)."""

    wants_float32_input = True
    graph_safe = True

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_experts = int(spec.num_experts)
        self.top_k = int(spec.top_k)
        self.inter = int(spec.intermediate_size)
        self.activation = str(spec.get("activation") or "relu2")
        if self.activation != "relu2":
            raise ValueError(f"unknown activation {self.activation!r} (relu2)")
        self.has_correction = bool(spec.get("correction", False))
        g = spec.get("groups")
        self.groups = None if g is None else int(g)
        self.keep_groups = None if g is None else int(spec.keep_groups)
        self.group_terms = int(spec.get("group_score_terms") or 2)
        if self.groups is not None and (self.num_experts % self.groups or not 1 <= self.keep_groups <= self.groups
                                        or self.keep_groups * (self.num_experts // self.groups) < self.top_k):
            raise ValueError("groups of equal size, 1 <= keep_groups <= groups, and top_k experts within the kept groups")
        self.tiled = False

    def param_specs(self):
        e, f, d = self.num_experts, self.inter, self.hidden
        specs = {
            "router": ParamSpec((e, d), policy="float32", init=("normal", d ** -0.5)),
            "w_up": ParamSpec((e, f, d), init=("normal", d ** -0.5)),  # per expert [out, in]
            "w_down": ParamSpec((e, d, f), init=("normal", f ** -0.5)),
        }
        if self.has_correction:
            specs["correction"] = ParamSpec((e,), policy="float32", init=("normal", 0.3))
        return specs

    def step_weight_bytes(self, observed=None) -> int:
        n = self.num_experts if observed is None else int(torch.unique(observed[0]).numel())
        total = 0
        for name, t in self.params.items():
            b = t.numel() * t.element_size()
            total += b // self.num_experts * n if name in ("w_up", "w_down") else b
        return total

    def flops_per_token(self) -> float:
        per = 0
        for name, t in self.params.items():
            per += t.numel() // self.num_experts * self.top_k if name in ("w_up", "w_down") else t.numel()
        return 2.0 * per

    def finalize(self) -> None:
        from ..ops.layout import can_tile, tile_

        up, dn = self.params["w_up"], self.params["w_down"]
        if not self.tiled and can_tile(up) and can_tile(dn) and self.inter % 16 == 0:
            tile_(up)
            tile_(dn)
            self.tiled = True

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        ops = ctx.ops
        expert_ids, weights, grouping = ops.moe_choose(h32, self.params["router"], self.params.get("correction"),
                                                       self.top_k, self.groups, self.keep_groups, self.group_terms)
        tap = getattr(ctx, "tap", None)
        if tap is not None:  # whoever watches the step sees the choice and may replace it
            replaced = tap(self, "routing", (expert_ids, weights))
            if replaced is not None:
                expert_ids, weights = replaced
                grouping = None
        return ops.moe_experts_scored(h, expert_ids, weights, self.params["w_up"], self.params["w_down"],
                                      activation=self.activation, tiled=self.tiled, grouping=grouping)


@register_feed_forward("dense_polynorm")
class DensePolyNorm(FeedForward):
    """``W_down act(W_up h + b_up) + b_down`` with the polynomial activation
    ``act(z) = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3``: powers element by element, ``N`` divides a token's row
    by its root mean square (``eps`` inside the root; float32)."""

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.inter = int(spec.intermediate_size)
        self.eps = float(spec.eps)

    def param_specs(self):
        d, f = self.hidden, self.inter
        return {
            "w_up": ParamSpec((f, d), init=("normal", d ** -0.5)),
            "b_up": ParamSpec((f,), policy="float32", init=("normal", 0.1)),
            "w_down": ParamSpec((d, f), init=("normal", f ** -0.5)),
            "b_down": ParamSpec((d,), policy="float32", init=("normal", 0.1)),
            "coef": ParamSpec((4,), policy="float32", init=("uniform", -1.0, 1.0)),
        }

    graph_safe = True

    def forward_unbiased(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx):
        """``(W_down act(...), b_down)``: for a caller whose next kernel adds the bias itself."""
        ops = ctx.ops
        z = ops.linear(h, self.params["w_up"])
        a = ops.polynorm(z, self.params["b_up"], self.params["coef"], self.eps)
        return ops.linear(a, self.params["w_down"]), self.params["b_down"]

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        y, b = self.forward_unbiased(h, h32, ctx)
        return (y.float() + b).to(y.dtype)
