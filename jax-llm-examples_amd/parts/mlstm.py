"""A recurrent mixer with a matrix memory per head (the mLSTM cell of xLSTM).

Per head, with ``q = W_q h / sqrt(dk)``, ``k = W_k h`` (``dk`` elements), ``v = W_v h`` (``dv`` elements) and two
gates of one number a head, ``a = W_i h + b_i`` and ``b = W_f h + b_f``, each squashed to ``cap * tanh(. / cap)``::

    i = a (a logarithm);   f = logsigmoid(b)
    m_t = max(f + m_{t-1}, i)
    C_t = exp(f + m_{t-1} - m_t) C_{t-1} + exp(i - m_t) k v^T        (dk x dv)
    n_t = exp(f + m_{t-1} - m_t) n_{t-1} + exp(i - m_t) k
    o_t = C_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)

``C``, ``n`` and ``m`` start at zero and are the request's state, float32, carried from step to step in two halves (a
step reads the half that the request's last committed step wrote and writes the other, so a step that is run twice
reads what its first run read).  Every head's ``o`` is divided by its root mean square, the heads side by side are
multiplied by a weight and by ``sigmoid(W_g h)``, and ``W_o`` follows.  The gates' pre-activations are formed from the
float32 normed rows with a float32 matrix; squashing, logsigmoid, the exponentials, the state and the division are
float32 whatever the run dtype; q, k, v and the output gate are in the run dtype.
"""
from __future__ import annotations

import torch

from .base import CacheNeed, Mixer, ParamSpec, register_mixer

DENOMINATOR_FLOOR = 1e-6


@register_mixer("mlstm")
class MatrixMemory(Mixer):
    wants_float32_input = True  # (for the gates)
    graph_safe = True

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_heads = int(spec.num_heads)
        self.head_dim = int(spec.head_dim)
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.gate_cap = float(spec.gate_cap)
        self.norm_eps = float(spec.norm_eps)
        if min(self.num_heads, self.head_dim, self.value_dim) < 1 or self.gate_cap <= 0:
            raise ValueError("the matrix memory needs positive sizes and a positive gate cap")

    @property
    def state_floats(self) -> int:
        """One head's state: the matrix, the normaliser and the running maximum."""
        return self.head_dim * self.value_dim + self.head_dim + 1

    def param_specs(self):
        h, dk, dv, d = self.num_heads, self.head_dim, self.value_dim, self.hidden
        return {
            # rows: q heads, k heads, v heads, output gate; each [out, in]
            "w_in": ParamSpec((2 * h * dk + 2 * h * dv, d), init=("normal", d ** -0.5)),
            "w_gates": ParamSpec((2 * h, d), policy="float32", init=("normal", d ** -0.5)),  # input gate rows, then forget
            "b_gates": ParamSpec((2 * h,), policy="float32", init=("normal", 1.0)),
            "norm": ParamSpec((h * dv,), policy="float32", init=("uniform", 0.5, 1.5)),
            "wo": ParamSpec((d, h * dv), init=("normal", (h * dv) ** -0.5)),
        }

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state_shape=(2, self.num_heads, self.state_floats), state_dtype=torch.float32)

    def mixing_flops(self, start: int, count: int) -> float:
        """Per token and head: the state's update and its product with the query."""
        return 4.0 * self.num_heads * self.head_dim * self.value_dim * count

    def forward(self, h: torch.Tensor, ctx, cache, h32=None) -> torch.Tensor:
        ops = ctx.ops
        rows = ops.linear(h, self.params["w_in"])
        gates = ops.linear(h if h32 is None else h32, self.params["w_gates"], out_dtype=torch.float32)
        o = ops.mlstm(rows, gates, self.params["b_gates"], self.params["norm"], self.num_heads, self.head_dim,
                      self.value_dim, self.gate_cap, self.norm_eps, DENOMINATOR_FLOOR, cache.state, ctx)
        return ops.linear(o, self.params["wo"])
