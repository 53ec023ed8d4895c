"""The generic decoder: embedding, the layers of a plan run in the plan's order,
final norm and output head (``llama4/llama4_jax/model.py:1186-1210``), each a part built from
its :class:`~..config.specs.PartSpec`.  It is built from a :class:`~..config.specs.ModelPlan` alone."""
from __future__ import annotations

import torch

from ..cache.manager import CacheView
from ..config.specs import ModelPlan
from .residual import build_residual
from ..config.specs import part
from . import embedding as _ends  # noqa: F401  (registers the built-in embedding and head)
from .base import CacheNeed, ParamSpec, Part, build_embedding, build_head, build_norm
from .block import build_block
from .loop import build_loop


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device) -> None:
        self.plan = plan
        self.dtype = dtype
        self.device = torch.device(device)
        # (a plan that does not describe its two ends gets a plain table and a plain linear head)
        self.embed = build_embedding(plan.embedding or part("token_embedding", vocab_size=plan.vocab_size,
                                                            hidden_size=plan.hidden_size))
        self.blocks = [build_block(spec) for spec in plan.layers]
        self.loop = None if plan.loop is None else build_loop(plan.loop)
        self.final_norm = build_norm(plan.final_norm)
        self.lm_head = build_head(plan.head or part("linear_head", vocab_size=plan.vocab_size,
                                                    hidden_size=plan.hidden_size, tied=plan.tie_word_embeddings))
        self._allocated = False

    # ------------------------------------------------------------------ parameters
    def named_parts(self) -> dict[str, Part]:
        out: dict[str, Part] = {"embed": self.embed}
        for i, b in enumerate(self.blocks):
            for name, p in b.parts().items():
                out[f"layers.{i}.{name}"] = p
        if self.loop is not None:
            out["loop"] = self.loop
        out["final_norm"] = self.final_norm
        out["lm_head"] = self.lm_head
        return out

    def param_specs(self) -> dict[str, ParamSpec]:
        return {f"{pn}.{n}": s for pn, p in self.named_parts().items() for n, s in p.param_specs().items()}

    def allocate(self) -> None:
        if not self._allocated:
            for p in self.named_parts().values():
                p.allocate(self.dtype, self.device)
            self._allocated = True

    def named_parameters(self) -> dict[str, torch.Tensor]:
        self.allocate()
        return {f"{pn}.{n}": t for pn, p in self.named_parts().items() for n, t in p.params.items()}

    def finalize(self) -> None:
        for p in self.named_parts().values():
            p.finalize()

    def num_parameters(self) -> int:
        n = 0
        for s in self.param_specs().values():
            k = 1
            for d in s.shape:
                k *= d
            n += k
        return n

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> dict[int, CacheNeed]:
        needs: dict[int, CacheNeed] = {}
        for e in self.plan.order:
            need = self.blocks[e.layer].mixer.cache_need()
            if e.cache in needs and needs[e.cache] != need:
                raise ValueError(f"runs that share cache {e.cache} need different things: {needs[e.cache]} vs {need}")
            needs[e.cache] = need
        return needs

    def run_state_needs(self) -> dict[int, dict]:
        """Fixed-size per-request state that the arrangements keep, by place in the run order (every run has its
        own, also a run that reads another run's cache): ``{name: (shape, dtype)}``."""
        out: dict[int, dict] = {}
        for k, e in enumerate(self.plan.order):
            need = getattr(self.blocks[e.layer], "run_state_need", None)
            need = need() if need is not None else {}
            if need:
                out[k] = dict(need)
        return out

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache) -> torch.Tensor:
        """Runs the step's tokens through every run of the order; returns float32
        logits ``[len(ctx.logits_indices), vocab]``."""
        ops = ctx.ops
        residual = build_residual(self.plan.residual, self.embed.forward(ctx.token_ids, ctx))
        embedded = None
        if self.loop is not None and getattr(self.loop, "needs_embedding_output", False):
            embedded = residual.x.clone()  # (the stream itself is added to in place)
        for k, e in enumerate(self.plan.order):
            if e.enters_pass is not None:
                self.loop.enter(residual, embedded, e.enters_pass, ctx)
            gi = cache.group_of.get(e.cache)
            view = CacheView(cache_id=e.cache, writes=e.writes_cache, group=gi, state=cache.state.get(e.cache),
                             run_state=cache.run_state.get(k),
                             states=getattr(cache, "named_state", {}).get(e.cache))
            if gi is not None:
                g = ctx.groups[gi]
                view.kv = cache.groups[gi].tensors.get(e.cache)
                view.pages = cache.groups[gi].pages.get(e.cache)
                view.block_table = g.block_table
                view.slot_mapping = g.slot_mapping
                view.attn_meta = g
            self.blocks[e.layer].forward(residual, ctx, view)
            if ctx.tap is not None:  # (whoever watches the step sees the residual stream behind every run)
                ctx.tap(self.blocks[e.layer], "residual", lambda r=residual: r.value(ctx).clone())
        if ctx.logits_indices.numel() == 0:
            residual.value(ctx)
            return torch.empty(0, self.plan.vocab_size, dtype=torch.float32, device=ctx.device)
        picked = residual.rows(ctx, ctx.logits_indices)
        h, _ = self.final_norm.forward(picked, ctx)
        return self.lm_head.forward(h, ctx, self.embed)
