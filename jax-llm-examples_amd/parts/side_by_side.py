"""Two mixers side by side: both read the same rows, and the layer's mixer output is ``left_scale * left(h) +
right_scale * right(h)``.  The sum is not formed here: it stays a :class:`~.residual.ScaledSum` that the kernel
which adds it to the residual forms in float32.  What the two need from the cache manager is put together: at most
one of them keeps keys and values in pages (its retention rule is the pair's), and the fixed-size state of either
arrives under its name with ``left.`` or ``right.`` in front (a child's single state tensor as ``<side>.state``)."""
from __future__ import annotations

import dataclasses

from .base import CacheNeed, Mixer, build_mixer, register_mixer
from .residual import ScaledSum


@register_mixer("side_by_side")
class SideBySide(Mixer):
    def __init__(self, spec) -> None:
        super().__init__()
        self.left = build_mixer(spec.left)
        self.right = build_mixer(spec.right)
        self.left_scale = float(spec.get("left_scale", 1.0))
        self.right_scale = float(spec.get("right_scale", 1.0))
        self.wants_float32_input = any(getattr(m, "wants_float32_input", False) for m in (self.left, self.right))
        self.graph_safe = all(getattr(m, "graph_safe", False) for m in (self.left, self.right))

    # the two mixers' parameters under ``left.`` and ``right.``
    def param_specs(self):
        return {f"{side}.{n}": s for side, m in (("left", self.left), ("right", self.right))
                for n, s in m.param_specs().items()}

    def allocate(self, dtype, device) -> None:
        for side, m in (("left", self.left), ("right", self.right)):
            m.allocate(dtype, device)
            for n, t in m.params.items():
                self.params[f"{side}.{n}"] = t

    def finalize(self) -> None:
        for side, m in (("left", self.left), ("right", self.right)):
            m.finalize()
            for n, t in m.params.items():  # (a mixer may replace a parameter by a re-laid one)
                self.params[f"{side}.{n}"] = t

    def step_weight_bytes(self, observed=None) -> int:
        return self.left.step_weight_bytes() + self.right.step_weight_bytes()

    def flops_per_token(self) -> float:
        return self.left.flops_per_token() + self.right.flops_per_token()

    def mixing_flops(self, start: int, count: int) -> float:
        return self.left.mixing_flops(start, count) + self.right.mixing_flops(start, count)

    def cache_need(self) -> CacheNeed:
        needs = {"left": self.left.cache_need(), "right": self.right.cache_need()}
        paged = [side for side, n in needs.items() if n.kv is not None or n.paged]
        if len(paged) > 1:
            raise ValueError("of two mixers side by side at most one keeps something per token")
        states = []
        for side, n in needs.items():
            if n.state_shape is not None:
                states.append((f"{side}.state", tuple(n.state_shape), n.state_dtype))
            states += [(f"{side}.{name}", tuple(shape), dt) for name, shape, dt in n.states]
        owner = needs[paged[0]] if paged else CacheNeed()
        return CacheNeed(kv=owner.kv, retention=owner.retention, paged=owner.paged, states=tuple(states))

    def _view(self, cache, side: str, child: Mixer):
        named = cache.states or {}
        own = {n[len(side) + 1:]: t for n, t in named.items() if n.startswith(side + ".")}
        need = child.cache_need()
        has_pages = need.kv is not None or bool(need.paged)
        return dataclasses.replace(cache, state=own.pop("state", None), states=own,
                                   kv=cache.kv if has_pages else None, pages=cache.pages if has_pages else None)

    def forward(self, h, ctx, cache, h32=None):
        outs = []
        for side, m in (("left", self.left), ("right", self.right)):
            view = self._view(cache, side, m)
            if getattr(m, "wants_float32_input", False):
                outs.append(m.forward(h, ctx, view, h32))
            else:
                outs.append(m.forward(h, ctx, view))
        return ScaledSum([(outs[0], self.left_scale), (outs[1], self.right_scale)])
