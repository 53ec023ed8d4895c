"""How a layer's parts are arranged.

``pre_norm`` (``llama4/llama4_jax/model.py:1166-1183``):
``h = x + mixer(norm(x))`` then ``x' = h + feed_forward(norm(h))``.  The residual
sum is kept in float32; adding a branch's output and the following norm are
one kernel, so a branch's output is *pending* on the residual until the next
norm (or the end of the model) applies it.
"""
from __future__ import annotations

import torch

from ..config.specs import LayerSpec
from .base import ParamSpec, Part, build_feed_forward, build_mixer, build_norm
from .residual import BranchSum, GatedBranch, ScaledSum

_ARRANGEMENTS = {}


def register_arrangement(name: str):
    def deco(cls):
        _ARRANGEMENTS[name] = cls
        return cls

    return deco


def build_block(spec: LayerSpec):
    try:
        cls = _ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {sorted(_ARRANGEMENTS)}") from None
    return cls(spec)


class ChannelScale(Part):
    """A learned factor per channel on a branch's output (float32); the kernel that adds the branch to the residual
    multiplies."""

    graph_safe = True

    def __init__(self, hidden: int) -> None:
        super().__init__()
        self.hidden = int(hidden)

    def param_specs(self):
        return {"weight": ParamSpec((self.hidden,), policy="float32", init=("uniform", 0.5, 1.5))}

    def flops_per_token(self) -> float:
        return 0.0


@register_arrangement("pre_norm")
class PreNormBlock:
    """``x += mixer(norm(x))``, then ``x += feed_forward(norm(x))``.  Options (``LayerSpec.options``), both off for
    Llama 4: ``branch_mult`` (a number every branch output is multiplied by before the sum) and ``layer_scale`` (with
    ``hidden_size``: a learned factor per channel on every branch output, :class:`ChannelScale`); with either, what
    stays pending on the residual is a :class:`~.residual.ScaledSum`.  A mixer may itself return such a sum (two
    mixers side by side with a weight each)."""

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.feed_forward = self.feed_forward_norm = None  # (a layer may have no feed-forward)
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)
        opt = spec.options or {}
        self.branch_mult = float(opt.get("branch_mult", 1.0))
        self.mixer_scale = self.feed_forward_scale = None
        if opt.get("layer_scale"):
            self.mixer_scale = ChannelScale(int(opt["hidden_size"]))
            if self.feed_forward is not None:
                self.feed_forward_scale = ChannelScale(int(opt["hidden_size"]))
        self.scaled = self.branch_mult != 1.0 or self.mixer_scale is not None

    def parts(self):
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm}
        if self.mixer_scale is not None:
            out["mixer_scale"] = self.mixer_scale
        if self.feed_forward is not None:
            out.update(feed_forward=self.feed_forward, feed_forward_norm=self.feed_forward_norm)
            if self.feed_forward_scale is not None:
                out["feed_forward_scale"] = self.feed_forward_scale
        return out

    def _branch(self, y, scale):
        if not self.scaled:
            return y
        return ScaledSum.of(y, self.branch_mult, None if scale is None else scale.params["weight"])

    def forward(self, residual, ctx, cache) -> None:
        want32 = bool(getattr(self.mixer, "wants_float32_input", False))
        h, h32 = self.mixer_norm.forward(residual, ctx, want32=want32)
        y = self.mixer.forward(h, ctx, cache, h32) if want32 else self.mixer.forward(h, ctx, cache)
        residual.add(self._branch(y, self.mixer_scale))
        ff = self.feed_forward
        if ff is None:
            return
        if getattr(ff, "accepts_deferred_norm", False):  # (it hands the rows to the kernel set only: see there)
            h, h32 = self.feed_forward_norm.forward(residual, ctx, want32=ff.wants_float32_input, defer=True)
        else:
            h, h32 = self.feed_forward_norm.forward(residual, ctx, want32=ff.wants_float32_input)
        residual.add(self._branch(ff.forward(h, h32, ctx), self.feed_forward_scale))


@register_arrangement("parallel")
class ParallelBlock:
    """Both branches read the same stream, each through a norm of its own, and their outputs are added together::

        x = x + (mixer(norm_a(x)) + feed_forward(norm_b(x)))

    The two norms share their statistics (one kernel forms both rows); the sum of the two outputs stays pending on
    the residual (a :class:`~.residual.BranchSum`).  The layer may have no feed-forward."""

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.feed_forward = self.feed_forward_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)
            if self.feed_forward_norm.eps != self.mixer_norm.eps:
                raise ValueError("the two norms of a parallel layer share their statistics: one eps")

    def parts(self):
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm}
        if self.feed_forward is not None:
            out.update(feed_forward=self.feed_forward, feed_forward_norm=self.feed_forward_norm)
        return out

    def forward(self, residual, ctx, cache) -> None:
        ff = self.feed_forward
        h_a, h_b = residual.normed_pair(ctx, self.mixer_norm.params.get("weight"),
                                        None if ff is None else self.feed_forward_norm.params.get("weight"),
                                        self.mixer_norm.eps)
        y = self.mixer.forward(h_a, ctx, cache)
        residual.add(BranchSum(y, None if ff is None else ff.forward(h_b, None, ctx)))


class SigmoidGate(Part):
    """``sigmoid(W h + b)`` per element of a branch's output; this part holds ``W`` and ``b``, the kernel that
    adds the branch to the residual applies the sigmoid and the product."""

    graph_safe = True

    def __init__(self, hidden: int) -> None:
        super().__init__()
        self.hidden = int(hidden)

    def param_specs(self):
        d = self.hidden
        return {"weight": ParamSpec((d, d), init=("normal", d ** -0.5)),
                "bias": ParamSpec((d,), policy="float32", init=("normal", 1.0))}

    def forward(self, h, ctx):
        """The gate before its sigmoid and without its bias: ``[N, hidden]`` in the run dtype."""
        return ctx.ops.linear(h, self.params["weight"])


class TokenShift(Part):
    """``h + (h_prev - h) * weight`` per element, ``h_prev`` the row of the token before (zeros before a
    sequence's first token).  The part holds the weight; the kernel that norms the rows does the mixing,
    from a per-request state that carries the last row from step to step."""

    graph_safe = True

    def __init__(self, hidden: int) -> None:
        super().__init__()
        self.hidden = int(hidden)

    def param_specs(self):
        return {"weight": ParamSpec((self.hidden,), policy="float32", init=("uniform", 0.0, 1.0))}

    def flops_per_token(self) -> float:
        return 0.0


@register_arrangement("sandwich_gated")
class SandwichGatedBlock:
    """A norm before and behind every branch, and a gate on its output::

        h = norm(x);  x += post_norm(branch(h') * sigmoid(W_g h + b_g))

    ``h'`` is ``h`` for the feed-forward and, with the option ``token_shift``, ``h`` mixed with the row of the
    token before for the mixer (:class:`TokenShift`; the gate reads ``h`` itself).  The layer may have no
    feed-forward.  The gated, normed branch output stays pending on the residual (a
    :class:`~.residual.GatedBranch`); the kernel that forms the next norm's rows adds it first.
    Options (``LayerSpec.options``): ``hidden_size``, ``post_norm`` (the spec of the two norms behind the
    branches), ``token_shift``."""

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        opt = spec.options
        d = int(opt["hidden_size"])
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.mixer_post_norm = build_norm(opt["post_norm"])
        self.mixer_gate = SigmoidGate(d)
        self.token_shift = TokenShift(d) if opt.get("token_shift") else None
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)
            self.feed_forward_post_norm = build_norm(opt["post_norm"])
            self.feed_forward_gate = SigmoidGate(d)
        self.hidden = d

    def parts(self):
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm, "mixer_post_norm": self.mixer_post_norm,
               "mixer_gate": self.mixer_gate}
        if self.token_shift is not None:
            out["token_shift"] = self.token_shift
        if self.feed_forward is not None:
            out.update(feed_forward=self.feed_forward, feed_forward_norm=self.feed_forward_norm,
                       feed_forward_post_norm=self.feed_forward_post_norm, feed_forward_gate=self.feed_forward_gate)
        return out

    def run_state_need(self) -> dict:
        """Per-request state of one run of this layer: the last token's normed row, for the shift."""
        return {"shift": ((self.hidden,), torch.float32)} if self.token_shift is not None else {}

    def forward(self, residual, ctx, cache) -> None:
        shift = None
        if self.token_shift is not None:
            shift = (self.token_shift.params["weight"], cache.run_state["shift"])
        h, hs = residual.normed_shifted(ctx, self.mixer_norm.params.get("weight"), self.mixer_norm.eps, shift)
        gate = self.mixer_gate.forward(h, ctx)
        y = self.mixer.forward(hs, ctx, cache)
        post = self.mixer_post_norm
        residual.add(GatedBranch(y, None, gate, self.mixer_gate.params["bias"], post.params.get("weight"), post.eps))
        ff = self.feed_forward
        if ff is None:
            return
        h, _ = residual.normed_shifted(ctx, self.feed_forward_norm.params.get("weight"), self.feed_forward_norm.eps,
                                       None)
        gate = self.feed_forward_gate.forward(h, ctx)
        if hasattr(ff, "forward_unbiased"):  # (the bias of its last product is added by the kernel that gates it)
            y, bias = ff.forward_unbiased(h, None, ctx)
        else:
            y, bias = ff.forward(h, None, ctx), None
        post = self.feed_forward_post_norm
        residual.add(GatedBranch(y, bias, gate, self.feed_forward_gate.params["bias"], post.params.get("weight"),
                                 post.eps))


class StreamWeights(Part):
    """What one branch of a layer over several residual streams learns about them: ``inw`` (how the branch's input
    is put together from the streams), ``mix`` (``[from, to]``: how the streams are mixed among themselves when the
    branch's output arrives) and ``outw`` (how much of the output every stream takes).  All float32."""

    graph_safe = True

    def __init__(self, streams: int) -> None:
        super().__init__()
        self.streams = int(streams)

    def param_specs(self):
        s = self.streams
        return {"inw": ParamSpec((s,), policy="float32", init=("uniform", 0.2, 0.8)),
                "outw": ParamSpec((s,), policy="float32", init=("uniform", 0.3, 1.0)),
                "mix": ParamSpec((s, s), policy="float32", init=("uniform", 0.0, 2.0 / s))}

    def flops_per_token(self) -> float:
        return 0.0


@register_arrangement("hyper_streams")
class HyperStreamsBlock:
    """Pre-norm branches over ``S`` residual streams (the plan's residual kind ``streams``)::

        u = sum_s inw[s] X_s;   y = branch(norm(u));   X_t <- sum_s mix[s, t] X_s + outw[t] y

    for the mixer and then for the feed-forward, each with stream weights of its own (``hc1``, ``hc2``).  The update
    stays pending on the streams; the kernel that forms the next branch's input makes it first.  The layer may have
    no feed-forward.  Options (``LayerSpec.options``): ``streams``."""

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        s = int(spec.options["streams"])
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.hc1 = StreamWeights(s)
        self.feed_forward = self.feed_forward_norm = self.hc2 = None
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)
            self.hc2 = StreamWeights(s)

    def parts(self):
        out = {"mixer": self.mixer, "mixer_norm": self.mixer_norm, "hc1": self.hc1}
        if self.feed_forward is not None:
            out.update(feed_forward=self.feed_forward, feed_forward_norm=self.feed_forward_norm, hc2=self.hc2)
        return out

    def forward(self, residual, ctx, cache) -> None:
        if not hasattr(residual, "branch_input"):
            raise TypeError("the hyper_streams arrangement works on the residual kind 'streams'")
        hc, norm = self.hc1.params, self.mixer_norm
        want32 = bool(getattr(self.mixer, "wants_float32_input", False))
        h, h32 = residual.branch_input(ctx, hc["inw"], norm.params.get("weight"), norm.eps, want32)
        y = self.mixer.forward(h, ctx, cache, h32) if want32 else self.mixer.forward(h, ctx, cache)
        residual.add_update(y, hc["mix"], hc["outw"])
        ff = self.feed_forward
        if ff is None:
            return
        hc, norm = self.hc2.params, self.feed_forward_norm
        h, h32 = residual.branch_input(ctx, hc["inw"], norm.params.get("weight"), norm.eps, ff.wants_float32_input)
        residual.add_update(ff.forward(h, h32, ctx), hc["mix"], hc["outw"])
