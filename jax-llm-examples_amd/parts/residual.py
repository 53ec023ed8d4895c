"""The residual stream of a step: float32 rows plus at most one pending branch
output.  The sum is applied by the next norm (one kernel does add and norm) or
when the value is asked for.

A plan may name another kind of stream (``ModelPlan.residual``).  ``streams``: ``S`` copies ``X_1 .. X_S`` of the
stream, all equal to the embedding's output at the start; a branch reads ``u = sum_s a_s X_s`` through its norm, and
its output ``y`` changes all copies at once, ``X_t <- sum_s M[s, t] X_s + o_t y``; at the model's end the copies are
added up.  ``a``, ``M`` and ``o`` belong to the branch (:class:`~.block.StreamWeights`).  The update stays pending
until the kernel that forms the next branch's input makes it."""
from __future__ import annotations

import torch


class GatedBranch:
    """A branch output that is not formed yet: ``rmsnorm((y + y_bias) * sigmoid(gate + gate_bias)) * weight``
    per row (statistics over the row, ``eps`` inside the root, float32).  ``y`` and ``gate`` are ``[N, hidden]``
    in the run dtype, the biases and the weight float32 ``[hidden]`` or ``None``.  The kernel that adds it to
    the residual reads the pieces directly."""

    def __init__(self, y, y_bias, gate, gate_bias, weight, eps: float) -> None:
        self.y, self.y_bias, self.gate, self.gate_bias, self.weight, self.eps = y, y_bias, gate, gate_bias, weight, float(eps)
        self.shape, self.dtype = y.shape, y.dtype

    def rows(self, ops, idx) -> "GatedBranch":
        return GatedBranch(ops.gather_rows(self.y, idx), self.y_bias, ops.gather_rows(self.gate, idx),
                           self.gate_bias, self.weight, self.eps)


class BranchSum:
    """The outputs of two branches that read the same rows (a layer with parallel branches): their sum
    ``a + b``, formed in float32 by the kernel that adds it to the residual.  ``b`` may be ``None``."""

    def __init__(self, a, b) -> None:
        self.a, self.b = a, b
        self.shape, self.dtype = a.shape, a.dtype

    def rows(self, ops, idx) -> "BranchSum":
        return BranchSum(ops.gather_rows(self.a, idx), None if self.b is None else ops.gather_rows(self.b, idx))


class ScaledSum:
    """A branch output that is not formed yet: ``vector * sum_i factor_i * term_i`` per row, formed in float32 by the
    kernel that adds it to the residual.  ``terms``: up to two ``(rows, factor)`` pairs, rows ``[N, hidden]`` in the
    run dtype or float32 (or a sum of expert outputs still in pieces), factors plain numbers; ``vector``: float32
    ``[hidden]`` or ``None``.  It is what a layer with a multiplier on its branches, a learned scale per channel, or
    two mixers side by side with a weight each leaves pending."""

    def __init__(self, terms, vector=None) -> None:
        self.terms = [(t, float(f)) for t, f in terms]
        if not 1 <= len(self.terms) <= 2:
            raise ValueError("a scaled sum has one or two terms")
        self.vector = vector
        self.shape, self.dtype = self.terms[0][0].shape, self.terms[0][0].dtype

    @classmethod
    def of(cls, y, factor: float = 1.0, vector=None) -> "ScaledSum":
        """``vector * factor * y`` where ``y`` is rows or itself a scaled sum (whose own vector must be ``None``)."""
        if isinstance(y, ScaledSum):
            if y.vector is not None:
                raise ValueError("a scaled sum with a vector cannot be scaled by another")
            return cls([(t, f * factor) for t, f in y.terms], vector)
        return cls([(y, factor)], vector)

    def rows(self, ops, idx) -> "ScaledSum":
        return ScaledSum([(ops.gather_rows(t, idx), f) for t, f in self.terms], self.vector)


class Residual:
    def __init__(self, x: torch.Tensor) -> None:
        assert x.dtype == torch.float32
        self._x = x
        self._deferred = None  # a norm (with its addition) that its consumer has been left to compute
        self.pending = None
        self.injected = None  # (float32 rows or None, float32 vector): added after what is pending (see inject)

    @property
    def x(self) -> torch.Tensor:
        if self._deferred is not None:
            self._x, self._deferred = self._deferred.residual(), None
        return self._x

    def add(self, delta) -> None:
        if self.pending is not None:
            raise AssertionError("a branch output is already pending on the residual")
        if delta.shape != self.x.shape:
            raise ValueError(f"branch output {tuple(delta.shape)} does not match residual {tuple(self.x.shape)}")
        self.pending = delta

    def inject(self, rows, vector) -> None:
        """``x + rows + vector`` (float32 ``[N, hidden]`` or ``None``, float32 ``[hidden]``), to be formed - after the
        pending branch output is added - by the kernel that makes the next norm's rows."""
        if self.injected is not None:
            raise AssertionError("something is already to be injected into the residual")
        self.injected = (rows, vector)

    def _settle_injected(self, ctx) -> None:
        """For consumers that do not know of injections: the sums are made now."""
        if self.injected is not None:
            x = self.value(ctx)
            ctx.ops.add_norm_pair(x, None, self.injected, None, None, 0.0, ctx.dtype, norm=False)
            self.injected = None

    def normed_pair(self, ctx, weight_a, weight_b, eps: float):
        """Adds what is pending and what is injected, and norms the rows once for two consumers: the same
        statistics, each consumer's own weight (``weight_b`` ``None``: one consumer).  Returns ``(h_a, h_b or
        None)`` in the run dtype."""
        h_a, h_b = ctx.ops.add_norm_pair(self.x, self.pending, self.injected, weight_a, weight_b, eps, ctx.dtype,
                                         second=weight_b is not None)
        self.pending = self.injected = None
        return h_a, h_b

    def normed(self, ctx, weight, eps: float, want32: bool = False, defer: bool = False):
        """``defer``: the part that takes the rows has said it accepts rows that are not computed yet (the
        kernel set's ``defer_norm``): it may then do addition and norm inside a launch of its own."""
        self._settle_injected(ctx)
        if defer and hasattr(ctx.ops, "defer_norm"):
            p = ctx.ops.defer_norm(self.x, self.pending, weight, eps, ctx.dtype)
            self.pending, self._deferred = None, p
            return p, (p if want32 else None)
        h, h32 = ctx.ops.add_rmsnorm(self.x, self.pending, weight, eps, ctx.dtype, want32)
        self.pending = None
        return h, h32

    def normed_shifted(self, ctx, weight, eps: float, shift=None):
        """Adds what is pending, norms the rows and, with ``shift = (weight, state)``, also gives the rows mixed
        with the rows of the tokens before them (see :class:`~.block.TokenShift`; ``state``: float32
        ``[slots, 2, hidden]``, the last row of every request, one half read and the other written by a
        step).  The addition is not done in place: a row's kernel forms the row before it anew.  Returns
        ``(h, shifted h or None)`` in the run dtype."""
        self._settle_injected(ctx)
        self._x, h, hs = ctx.ops.add_norm_shift(self.x, self.pending, weight, eps, ctx.dtype, shift, ctx)
        self.pending = None
        return h, hs

    def value(self, ctx) -> torch.Tensor:
        """The stream with what is pending added (what is injected belongs to the next run and stays)."""
        if self.pending is not None:
            ctx.ops.add_residual(self.x, self.pending)
            self.pending = None
        return self.x

    def rows(self, ctx, idx: torch.Tensor) -> "Residual":
        """The residual of the chosen rows only (what is pending stays pending)."""
        self._settle_injected(ctx)
        r = Residual(ctx.ops.gather_rows(self.x, idx))
        if self.pending is not None:
            if hasattr(self.pending, "rows"):
                r.pending = self.pending.rows(ctx.ops, idx)
            else:
                r.pending = ctx.ops.gather_rows(self.pending, idx)
        return r


class StreamUpdate:
    """A branch output ``y`` that is still to be worked into the streams: ``X_t <- sum_s mix[s, t] X_s + outw[t] y``."""

    def __init__(self, y, mix, outw) -> None:
        self.y, self.mix, self.outw = y, mix, outw


class StreamsResidual:
    """``S`` residual streams, float32 ``[N, S, hidden]``.  What the other kind offers where the model and the norms
    use it (``value``, ``rows``, ``normed``: all about the sum of the streams), and for the arrangement that knows of
    streams ``branch_input`` / ``add_update``."""

    def __init__(self, xs: torch.Tensor) -> None:
        assert xs.dtype == torch.float32 and xs.dim() == 3
        self.xs = xs
        self.streams = xs.shape[1]
        self.pending = None

    @classmethod
    def start(cls, x: torch.Tensor, streams: int) -> "StreamsResidual":
        """Every stream a copy of the embedding's output."""
        return cls(x.unsqueeze(1).expand(-1, int(streams), -1).contiguous())

    def add_update(self, y, mix, outw) -> None:
        if self.pending is not None:
            raise AssertionError("a branch output is already pending on the streams")
        if tuple(y.shape) != (self.xs.shape[0], self.xs.shape[2]):
            raise ValueError(f"branch output {tuple(y.shape)} does not match streams {tuple(self.xs.shape)}")
        self.pending = StreamUpdate(y, mix, outw)

    def branch_input(self, ctx, inw, weight, eps: float, want32: bool = False):
        """Makes the pending update, then ``u = sum_s inw[s] X_s`` (``inw`` ``None``: the plain sum) and its RMS
        norm with ``weight``; one kernel.  Returns ``(h, h in float32 or None)``."""
        h, h32 = ctx.ops.streams_mix_norm(self.xs, self.pending, inw, weight, eps, ctx.dtype, want32)
        self.pending = None
        return h, h32

    def normed(self, ctx, weight, eps: float, want32: bool = False, defer: bool = False):
        """The norm of the streams' sum (what the model's final norm asks for)."""
        return self.branch_input(ctx, None, weight, eps, want32)

    def value(self, ctx) -> torch.Tensor:
        """The sum of the streams, with what is pending worked in."""
        if self.pending is not None:
            ctx.ops.streams_mix_norm(self.xs, self.pending, None, None, 0.0, ctx.dtype, False, norm=False)
            self.pending = None
        return self.xs.sum(dim=1)

    @property
    def x(self) -> torch.Tensor:
        return self.xs.sum(dim=1)

    def rows(self, ctx, idx: torch.Tensor) -> "StreamsResidual":
        """The streams of the chosen rows only (what is pending stays pending)."""
        n, s, d = self.xs.shape
        r = StreamsResidual(ctx.ops.gather_rows(self.xs.view(n, s * d), idx).view(-1, s, d))
        if self.pending is not None:
            p = self.pending
            r.pending = StreamUpdate(ctx.ops.gather_rows(p.y, idx), p.mix, p.outw)
        return r


_RESIDUALS = {"streams": lambda spec, x: StreamsResidual.start(x, spec.streams)}


def build_residual(spec, x: torch.Tensor):
    """The residual stream of a step from the embedding's output ``x`` (float32 ``[N, hidden]``), of the kind the plan
    names (``None``: the plain one)."""
    if spec is None:
        return Residual(x)
    try:
        return _RESIDUALS[spec.kind](spec, x)
    except KeyError:
        raise KeyError(f"unknown residual kind {spec.kind!r}; known: {sorted(_RESIDUALS)}") from None
