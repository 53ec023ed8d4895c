"""The Mazotar decoder as an architecture: its configuration, its plan and the names of its checkpoint tensors.

The model's ends: ``embed``, ``final.norm``, ``head``.  A layer ``i`` stores, under ``l<i>.``: its two norms
(``norm1`` for the mixer, ``norm2`` for the feed-forward), with several residual streams the two branches' stream
weights (``hc1.*`` and ``hc2.*``: ``in`` and ``out``, one number a stream, and ``mix``, ``[from, to]``), the mixer's
tensors under ``mix.`` and the feed-forward's under ``mlp.``.  Mixer ``attention``: ``q``, ``k``, ``v``, ``o``, the
norms' weights over the whole projections ``q.norm`` and ``k.norm``, the distance table ``rel`` (``[rows, heads]``)
and ``sink`` (one number a head); a layer that reads another's keys and values has no ``k``, ``v`` and ``k.norm``.
Mixer ``mlstm``: ``q``, ``k``, ``v``, ``g`` (the output gate), ``o``, the two gates ``i`` and ``f`` with biases
(``.b``), ``norm`` (over all heads' outputs).  Feed-forward ``dense``: ``gate``, ``up``, ``down``; ``moe``: ``router``,
the experts ``e<j>.gate|up|down``, and ``shared.gate|up|down`` with the gate's row ``shared.sg``.  Linear weights are
``[out, in]``.
"""
from __future__ import annotations

import math
from typing import Any, Mapping

from ..config.mazotar import MazotarConfig
from ..config.registry import register_architecture
from ..config.rovidra import DenseFeedForwardConfig
from ..config.specs import ModelPlan
from ..weights.bindings import TensorBinding


class MazotarArchitecture:
    names = ("Mazotar", "mazotar")
    # what of csrc/ a model of this design calls (a first run on a machine without a built library compiles these)
    kernel_sources = ("elementwise.hip", "streams.hip", "mlstm.hip", "attention_span.hip", "attention_generic.hip",
                      "attention_mfma.hip", "attention_f32.hip", "attention_prep.hip", "moe_route.hip", "gemm_skinny.hip",
                      "gemm_stream.hip", "gemm_grouped.hip", "gemm_generic.hip", "gemm_f32.hip", "sampling.hip")

    def parse_config(self, top: Mapping[str, Any]) -> MazotarConfig:
        return MazotarConfig.from_dict(top)

    def complete_config(self, cfg: MazotarConfig, shapes: Mapping[str, tuple]) -> MazotarConfig:
        return cfg.complete(shapes)

    def plan(self, cfg: MazotarConfig) -> ModelPlan:
        return cfg.plan()

    def config_to_dict(self, cfg: MazotarConfig, architecture: str | None = None) -> dict:
        return cfg.to_dict(architecture or "Mazotar")

    def unused_prefixes(self, cfg: MazotarConfig) -> tuple:
        """Tensors that a checkpoint may hold and this model does not read: the feed-forward's norm and stream weights
        of a layer that has no feed-forward."""
        return tuple(f"l{i}.{name}" for i, lc in enumerate(cfg.layers) if lc.mlp is None for name in ("norm2", "hc2."))

    def bindings(self, cfg: MazotarConfig, plan: ModelPlan) -> list[TensorBinding]:
        D, V, S = cfg.width, cfg.vocab, cfg.streams
        mat = lambda fan_in: ("normal", 1.0 / math.sqrt(fan_in))
        norm = ("uniform", 0.5, 1.5)
        out = [TensorBinding("embed", (V, D), "embed.weight", init=("normal", 1.0))]
        for i, lc in enumerate(cfg.layers):
            p, t = f"l{i}.", f"layers.{i}."
            m = lc.mixer
            out.append(TensorBinding(p + "norm1", (D,), t + "mixer_norm.weight", init=norm))
            for q in (1, 2):
                if S is None or (q == 2 and lc.mlp is None):
                    continue
                out += [TensorBinding(p + f"hc{q}.in", (S,), t + f"hc{q}.inw", init=("uniform", 0.2, 0.8)),
                        TensorBinding(p + f"hc{q}.out", (S,), t + f"hc{q}.outw", init=("uniform", 0.3, 1.0)),
                        TensorBinding(p + f"hc{q}.mix", (S, S), t + f"hc{q}.mix", init=("uniform", 0.0, 2.0 / S))]
            if lc.type == "attention":
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                out += [TensorBinding(p + "mix.q", (nq, D), t + "mixer.wqkv", rows=(0, nq), init=mat(D)),
                        TensorBinding(p + "mix.q.norm", (nq,), t + "mixer.q_norm", init=norm)]
                if m.kv_from is None:
                    out += [TensorBinding(p + "mix.k", (nk, D), t + "mixer.wqkv", rows=(nq, nq + nk), init=mat(D)),
                            TensorBinding(p + "mix.v", (nv, D), t + "mixer.wqkv", rows=(nq + nk, nq + nk + nv),
                                          init=mat(D)),
                            TensorBinding(p + "mix.k.norm", (nk,), t + "mixer.k_norm", init=norm)]
                out += [TensorBinding(p + "mix.rel", (m.bias_rows, m.heads), t + "mixer.rel", init=("normal", 1.0)),
                        TensorBinding(p + "mix.sink", (m.heads,), t + "mixer.sink", init=("normal", 1.0)),
                        TensorBinding(p + "mix.o", (D, m.heads * m.vdim), t + "mixer.wo", init=mat(m.heads * m.vdim))]
            else:
                nk, nv, H = m.heads * m.dim, m.heads * m.vdim, m.heads
                o = 0
                for name, rows in (("q", nk), ("k", nk), ("v", nv), ("g", nv)):
                    out.append(TensorBinding(p + f"mix.{name}", (rows, D), t + "mixer.w_in", rows=(o, o + rows),
                                             init=mat(D)))
                    o += rows
                out += [TensorBinding(p + "mix.i", (H, D), t + "mixer.w_gates", rows=(0, H), init=mat(D)),
                        TensorBinding(p + "mix.f", (H, D), t + "mixer.w_gates", rows=(H, 2 * H), init=mat(D)),
                        TensorBinding(p + "mix.i.b", (H,), t + "mixer.b_gates", rows=(0, H), init=("normal", 1.0)),
                        TensorBinding(p + "mix.f.b", (H,), t + "mixer.b_gates", rows=(H, 2 * H),
                                      init=("uniform", 1.0, 4.0)),
                        TensorBinding(p + "mix.norm", (nv,), t + "mixer.norm", init=norm),
                        TensorBinding(p + "mix.o", (D, nv), t + "mixer.wo", init=mat(nv))]
            if lc.mlp is None:
                continue
            out.append(TensorBinding(p + "norm2", (D,), t + "feed_forward_norm.weight", init=norm))
            ff = t + "feed_forward."
            if isinstance(lc.mlp, DenseFeedForwardConfig):
                F = lc.mlp.ff
                out += [TensorBinding(p + "mlp.gate", (F, D), ff + "w_gate_up", rows=(0, F), init=mat(D)),
                        TensorBinding(p + "mlp.up", (F, D), ff + "w_gate_up", rows=(F, 2 * F), init=mat(D)),
                        TensorBinding(p + "mlp.down", (D, F), ff + "w_down", init=mat(F))]
                continue
            F = lc.mlp.ff
            out.append(TensorBinding(p + "mlp.router", (lc.mlp.experts, D), ff + "router", init=mat(D)))
            for e in range(lc.mlp.experts):
                out += [TensorBinding(p + f"mlp.e{e}.gate", (F, D), ff + "w_gate_up", index=e, rows=(0, F), init=mat(D)),
                        TensorBinding(p + f"mlp.e{e}.up", (F, D), ff + "w_gate_up", index=e, rows=(F, 2 * F), init=mat(D)),
                        TensorBinding(p + f"mlp.e{e}.down", (D, F), ff + "w_down", index=e, init=mat(F))]
            if lc.mlp.shared_ff is not None:
                Fs = lc.mlp.shared_ff
                out += [TensorBinding(p + "mlp.shared.gate", (Fs, D), ff + "shared_gate_up", rows=(0, Fs), init=mat(D)),
                        TensorBinding(p + "mlp.shared.up", (Fs, D), ff + "shared_gate_up", rows=(Fs, 2 * Fs), init=mat(D)),
                        TensorBinding(p + "mlp.shared.down", (D, Fs), ff + "shared_down", init=mat(Fs)),
                        TensorBinding(p + "mlp.shared.sg", (1, D), ff + "shared_gate", init=mat(D))]
        out += [
            TensorBinding("final.norm", (D,), "final_norm.weight", init=norm),
            TensorBinding("head", (V, D), "lm_head.weight", init=mat(D)),
        ]
        return out


MAZOTAR = register_architecture(MazotarArchitecture())
