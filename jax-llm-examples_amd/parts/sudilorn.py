"""The Sudilorn decoder as an architecture: its configuration, its plan and the names of its checkpoint tensors.

The model's ends: ``embed``, ``final.norm``, ``head``.  A layer ``i`` stores, under ``l<i>.``: its two norms (``norm1``
for the mixer, ``norm2`` for the feed-forward; weights kept as their distance from one), the per-channel scales of the
two branch outputs (``ls1``, ``ls2``), the mixer's tensors under ``mix.`` and the feed-forward's under ``mlp.``.
Mixer ``attention``: ``q``, ``k``, ``v`` (q and k rows head by head, a head's two score maps one after the other),
their convolutions' taps ``q.conv``, ``k.conv``, ``v.conv`` (``[channels, taps]``), the q/k norms' weights
``q.norm``, ``k.norm`` (over a head's elements, shared by heads and maps), the four vectors of the maps' mixing
weight ``lq1``, ``lk1``, ``lq2``, ``lk2``, the output gate ``g`` and ``o``.  Mixer ``parallel``: under ``left.`` the
attention's ``q``, ``k``, ``v`` with biases (``.b``) and ``o``; under ``right.`` the delta rule's ``q``, ``k``, ``v``
with taps (``.conv``), the write strength's matrix ``b``, the decay's ``a``, ``dt_bias`` and ``A_log``, the head
norm's weight ``norm``, the output gate ``g`` and ``o``.  Feed-forward: ``router``, ``correction``, the experts
``e<j>.up|down``.  Linear weights are ``[out, in]``.
"""
from __future__ import annotations

import math
from typing import Any, Mapping

from ..config.registry import register_architecture
from ..config.specs import ModelPlan
from ..config.sudilorn import SudilornConfig
from ..weights.bindings import TensorBinding


class SudilornArchitecture:
    names = ("Sudilorn", "sudilorn")
    # what of csrc/ a model of this design calls (a first run on a machine without a built library compiles these)
    kernel_sources = ("elementwise.hip", "scaled.hip", "gated_delta.hip", "attention_heads.hip", "attention_conv.hip",
                      "attention_generic.hip", "attention_mfma.hip", "attention_f32.hip", "attention_prep.hip",
                      "moe_route.hip", "moe_choose.hip", "gemm_skinny.hip", "gemm_stream.hip", "gemm_grouped.hip",
                      "gemm_generic.hip", "gemm_f32.hip", "parallel.hip", "sampling.hip")

    def parse_config(self, top: Mapping[str, Any]) -> SudilornConfig:
        return SudilornConfig.from_dict(top)

    def plan(self, cfg: SudilornConfig) -> ModelPlan:
        return cfg.plan()

    def config_to_dict(self, cfg: SudilornConfig, architecture: str | None = None) -> dict:
        return cfg.to_dict(architecture or "Sudilorn")

    def unused_prefixes(self, cfg: SudilornConfig) -> tuple:
        """Tensors that a checkpoint may hold and this model does not read: the feed-forward's norm and scale of a
        layer that has no feed-forward."""
        return tuple(f"l{i}.{name}" for i, lc in enumerate(cfg.layers) if lc.mlp is None for name in ("norm2", "ls2"))

    def bindings(self, cfg: SudilornConfig, plan: ModelPlan) -> list[TensorBinding]:
        D, V = cfg.width, cfg.vocab
        mat = lambda fan_in: ("normal", 1.0 / math.sqrt(fan_in))
        norm = ("normal", 0.1)
        out = [TensorBinding("embed", (V, D), "embed.weight", init=("normal", 1.0))]

        def fused(p, t, target, pieces, taps=0, biased=False):
            """q | k | v stored apart, landing one behind the other in ``target`` (and their taps and biases)."""
            o = 0
            for name, rows in pieces:
                out.append(TensorBinding(p + name, (rows, D), t + target, rows=(o, o + rows), init=mat(D)))
                if taps:
                    out.append(TensorBinding(p + name + ".conv", (rows, taps), t + "conv", rows=(o, o + rows),
                                             init=("normal", 0.6)))
                if biased:
                    out.append(TensorBinding(p + name + ".b", (rows,), t + "bqkv", rows=(o, o + rows),
                                             init=("normal", 0.3)))
                o += rows

        for i, lc in enumerate(cfg.layers):
            p, t = f"l{i}.", f"layers.{i}."
            m = lc.mixer
            out += [TensorBinding(p + "norm1", (D,), t + "mixer_norm.weight", init=norm),
                    TensorBinding(p + "ls1", (D,), t + "mixer_scale.weight", init=("uniform", 0.5, 1.5))]
            if lc.type == "attention":
                x, tm = p + "mix.", t + "mixer."
                fused(x, tm, "wqkv", (("q", m.heads * 2 * m.dim), ("k", m.kv_heads * 2 * m.dim),
                                      ("v", m.kv_heads * m.vdim)), taps=m.conv)
                out += [TensorBinding(x + "q.norm", (m.dim,), tm + "q_norm", init=("uniform", 0.5, 1.5)),
                        TensorBinding(x + "k.norm", (m.dim,), tm + "k_norm", init=("uniform", 0.5, 1.5))]
                for name in ("lq1", "lk1", "lq2", "lk2"):
                    out.append(TensorBinding(x + name, (m.dim,), tm + "lam_" + name[1:], init=("normal", 0.3)))
                out += [TensorBinding(x + "g", (m.heads * m.vdim, D), tm + "wg", init=mat(D)),
                        TensorBinding(x + "o", (D, m.heads * m.vdim), tm + "wo", init=mat(m.heads * m.vdim))]
            else:
                a, b = m.left, m.right
                x, tm = p + "mix.left.", t + "mixer.left."
                fused(x, tm, "wqkv", (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)),
                      biased=True)
                out.append(TensorBinding(x + "o", (D, a.heads * a.vdim), tm + "wo", init=mat(a.heads * a.vdim)))
                x, tm = p + "mix.right.", t + "mixer.right."
                fused(x, tm, "w_in", (("q", b.kv_heads * b.dim), ("k", b.kv_heads * b.dim), ("v", b.heads * b.vdim)),
                      taps=b.conv)
                H = b.heads
                out += [TensorBinding(x + "b", (H, D), tm + "w_gates", rows=(0, H), init=mat(D)),
                        TensorBinding(x + "a", (H, D), tm + "w_gates", rows=(H, 2 * H), init=mat(D)),
                        TensorBinding(x + "dt_bias", (H,), tm + "dt_bias", init=("normal", 1.0)),
                        TensorBinding(x + "A_log", (H,), tm + "a_log", init=("uniform", -2.0, 1.0)),
                        TensorBinding(x + "norm", (b.vdim,), tm + "norm", init=("uniform", 0.5, 1.5)),
                        TensorBinding(x + "g", (H * b.vdim, D), tm + "wg", init=mat(D)),
                        TensorBinding(x + "o", (D, H * b.vdim), tm + "wo", init=mat(H * b.vdim))]
            if lc.mlp is None:
                continue
            out += [TensorBinding(p + "norm2", (D,), t + "feed_forward_norm.weight", init=norm),
                    TensorBinding(p + "ls2", (D,), t + "feed_forward_scale.weight", init=("uniform", 0.5, 1.5))]
            ff, F = t + "feed_forward.", lc.mlp.ff
            out += [TensorBinding(p + "mlp.router", (lc.mlp.experts, D), ff + "router", init=mat(D)),
                    TensorBinding(p + "mlp.correction", (lc.mlp.experts,), ff + "correction", init=("normal", 0.3))]
            for e in range(lc.mlp.experts):
                out += [TensorBinding(p + f"mlp.e{e}.up", (F, D), ff + "w_up", index=e, init=mat(D)),
                        TensorBinding(p + f"mlp.e{e}.down", (D, F), ff + "w_down", index=e, init=mat(F))]
        out += [TensorBinding("final.norm", (D,), "final_norm.weight", init=norm),
                TensorBinding("head", (V, D), "lm_head.weight", init=mat(D))]
        return out


SUDILORN = register_architecture(SudilornArchitecture())
