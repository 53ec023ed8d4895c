"""A recurrent mixer with a matrix memory per head that is written by the gated delta rule.

With ``q = silu(conv(W_q h))``, ``k = silu(conv(W_k h))`` (``kv_heads`` heads of ``dk`` elements; head ``h`` of the
memory uses q/k head ``h // (heads / kv_heads)``) and ``v = silu(conv(W_v h))`` (``heads`` heads of ``dv`` elements),
where ``conv`` is a short causal convolution over time on every channel (zeros before the sequence's start; without
taps: none), q and k made unit vectors per head (``x / sqrt(sum(x^2) + floor)``) and q then times ``dk^(-1/2)``, a
write strength ``beta = sigmoid(W_b h)`` and a decay ``g = exp(-exp(A) * softplus(W_a h + dt))`` per head::

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q             (S: dk x dv, zero at the start)

so the read-out sees the token's own write.  Every head's ``o`` is divided by its root mean square, multiplied by a
weight over ``dv`` (shared by the heads) and by ``silu(W_g h)``; ``W_o`` follows.  The memory is the request's state,
float32, in two halves (a step reads the half that the request's last committed step wrote and writes the other); the
convolution's last ``taps - 1`` projected rows are state too, in the run dtype.  ``beta`` and the decay are formed
in float32 from float32 rows with a float32 matrix; the unit vectors, the memory and its products are float32
whatever the run dtype; the projections, the convolution and its activation are in the run dtype.
"""
from __future__ import annotations

import torch

from .base import CacheNeed, Mixer, ParamSpec, register_mixer


@register_mixer("gated_delta")
class GatedDelta(Mixer):
    wants_float32_input = True  # (for the write strength and the decay)
    graph_safe = True

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_heads = int(spec.num_heads)
        self.num_kv_heads = int(spec.get("num_kv_heads") or self.num_heads)
        self.head_dim = int(spec.head_dim)
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.conv_taps = int(spec.get("conv_taps") or 0)
        self.norm_eps = float(spec.norm_eps)
        self.unit_floor = float(spec.get("unit_floor", 1e-6))
        if min(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim) < 1 or self.num_heads % self.num_kv_heads:
            raise ValueError("the gated delta rule needs positive sizes and heads a multiple of kv_heads")
        self.state_dtype = None
        self.conv_by_tap = None

    @property
    def channels(self) -> int:
        """The rows that pass the convolution: q, k, v."""
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.value_dim

    def param_specs(self):
        h, g, dk, dv, d = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, self.hidden
        specs = {
            "w_in": ParamSpec((self.channels, d), init=("normal", d ** -0.5)),  # rows: q heads, k heads, v heads
            "wg": ParamSpec((h * dv, d), init=("normal", d ** -0.5)),
            "w_gates": ParamSpec((2 * h, d), policy="float32", init=("normal", d ** -0.5)),  # beta rows, then decay rows
            "dt_bias": ParamSpec((h,), policy="float32", init=("normal", 1.0)),
            "a_log": ParamSpec((h,), policy="float32", init=("uniform", -2.0, 1.0)),
            "norm": ParamSpec((dv,), policy="float32", init=("uniform", 0.5, 1.5)),
            "wo": ParamSpec((d, h * dv), init=("normal", (h * dv) ** -0.5)),
        }
        if self.conv_taps:
            specs["conv"] = ParamSpec((self.channels, self.conv_taps), policy="float32", init=("normal", 0.6))
        return specs

    def allocate(self, dtype, device) -> None:
        super().allocate(dtype, device)
        self.state_dtype = dtype

    def finalize(self) -> None:
        self.conv_by_tap = self.params["conv"].t().contiguous() if self.conv_taps else None

    def cache_need(self) -> CacheNeed:
        states = [("memory", (2, self.num_heads, self.value_dim, self.head_dim), torch.float32)]  # (S transposed)
        if self.conv_taps > 1:
            states.append(("conv", (2, self.conv_taps - 1, self.channels), self.state_dtype))
        return CacheNeed(states=tuple(states))

    def mixing_flops(self, start: int, count: int) -> float:
        """Per token and head: the memory's product with the key, its update and its product with the query."""
        return 6.0 * self.num_heads * self.head_dim * self.value_dim * count

    def forward(self, h: torch.Tensor, ctx, cache, h32=None) -> torch.Tensor:
        ops = ctx.ops
        P = self.params
        proj = ops.linear(h, P["w_in"])
        gate = ops.linear(h, P["wg"])
        gates = ops.linear(h if h32 is None else h32, P["w_gates"], out_dtype=torch.float32)
        rows = ops.conv_rows(proj, None, self.conv_by_tap, self.conv_taps,
                             cache.states.get("conv") if self.conv_taps > 1 else None, ctx, activation="silu")
        o = ops.gated_delta(rows, gates, P["a_log"], P["dt_bias"], P["norm"], gate, self.num_heads, self.num_kv_heads,
                            self.head_dim, self.value_dim, self.norm_eps, self.unit_floor, cache.states["memory"], ctx)
        return ops.linear(o, P["wo"])
