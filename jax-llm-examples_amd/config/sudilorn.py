"""Typed configuration of the Sudilorn decoder, read from ``config.json``.

The file lists the model's layers one by one: ``{"architecture": "Sudilorn", "vocab": V, "width": D, "norm":
{"eps": e}, "residual_mult": m, "layers": [{"type": ..., "mixer": {...}, "mlp": {...} | null}, ...]}``.  A layer's
``type`` names its mixer.  Every size and constant that can differ between two models of the design is a key of the
file; a key this reader does not know is an error.

Mixer ``attention`` (two score maps per head over the same values): ``heads``, ``kv_heads``, ``dim`` (query/key
elements per head and map), ``vdim``, ``scale``, ``diff`` (the constant of the maps' mixing weight), ``conv`` (taps
of the convolution over time behind the projections; absent: none), ``mask = {"size"}`` (the window), ``rot =
{"base", "dims", "scaling": {"factor", "original", "fast", "slow"}}`` (``scaling`` may be absent).
Mixer ``parallel``: ``left`` (an attention with projection biases: ``heads``, ``kv_heads``, ``dim``, ``vdim``,
``scale``, ``mask = {"size", "keep_first"}``, ``rot = {"base", "dims"}``), ``right`` (the gated delta rule:
``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``), ``left_scale``, ``right_scale``.
Feed-forward ``moe``: ``router = {"experts", "top", "groups": {"count", "keep"}}`` (``groups`` may be absent),
``expert = {"ff"}``.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional

from .llama4 import ConfigError
from .rovidra import _need, _only
from .specs import LayerSpec, ModelPlan, OrderEntry, part

# fixed by the design
GROUP_SCORE_TERMS = 2  # a group of experts is scored by the sum of so many of its largest choice scores
UNIT_FLOOR = 1e-6  # inside the root of the delta rule's unit vectors


@dataclasses.dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[tuple]  # (factor, original, fast, slow) or None

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "RotaryConfig":
        _only(m, ("base", "dims", "scaling"), where)
        sc = m.get("scaling")
        if sc is not None:
            _only(sc, ("factor", "original", "fast", "slow"), where + ".scaling")
            sc = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow"))
        c = cls(base=float(_need(m, "base", where)), dims=int(_need(m, "dims", where)), scaling=sc)
        if c.dims < 2 or c.dims % 2:
            raise ConfigError(f"config.json: {where}.dims must be even and positive")
        return c

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return d

    def spec(self, pairing: str):
        return part("rope_yarn", theta=self.base, rotary_dim=self.dims, scaling=self.scaling, pairing=pairing)


def _mask(m: Optional[Mapping[str, Any]], where: str, may_keep: bool):
    """``(size or None, keep_first)``."""
    if m is None:
        return None, 0
    _only(m, ("size", "keep_first") if may_keep else ("size",), where)
    size = int(_need(m, "size", where))
    keep = int(m.get("keep_first") or 0)
    if size < 1 or keep < 0:
        raise ConfigError(f"config.json: {where}: a window of at least one token and no negative keep_first")
    return size, keep


def _retention(size: Optional[int], keep: int) -> tuple:
    if size is None:
        return ("all",)
    return ("window_keep", size, keep) if keep else ("window", size)


def _heads(m, where):
    heads = int(_need(m, "heads", where))
    kv = int(m["kv_heads"]) if m.get("kv_heads") is not None else heads
    dim = int(_need(m, "dim", where))
    vdim = int(m["vdim"]) if m.get("vdim") is not None else dim
    if min(heads, kv, dim, vdim) < 1 or heads % kv:
        raise ConfigError(f"config.json: {where}: positive sizes and heads a multiple of kv_heads are needed")
    return heads, kv, dim, vdim


@dataclasses.dataclass(frozen=True)
class DifferentialAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: int  # 0: no convolution
    window: Optional[int]
    rot: RotaryConfig

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "DifferentialAttentionConfig":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "diff", "conv", "mask", "rot"), where)
        heads, kv, dim, vdim = _heads(m, where)
        window, _ = _mask(m.get("mask"), where + ".mask", may_keep=False)
        c = cls(heads, kv, dim, vdim, float(_need(m, "scale", where)), float(_need(m, "diff", where)),
                int(m.get("conv") or 0), window, RotaryConfig.from_dict(_need(m, "rot", where), where + ".rot"))
        if c.rot.dims > c.dim or c.conv < 0:
            raise ConfigError(f"config.json: {where}: rot.dims beyond dim, or a negative conv")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "diff": self.diff, "rot": self.rot.to_dict()}
        if self.conv:
            d["conv"] = self.conv
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d

    def spec(self, D: int, eps: float):
        return part("attention", hidden_size=D, num_heads=self.heads, num_kv_heads=self.kv_heads, head_dim=self.dim,
                    value_dim=self.vdim, softmax_scale=self.scale, retention=_retention(self.window, 0),
                    position=self.rot.spec("half"),
                    qk_norm=part("rmsnorm", eps=eps, weighted=True, before_rotation=True),
                    conv_taps=self.conv, score_maps=part("differential", diff=self.diff, eps=eps), output_gate=True)


@dataclasses.dataclass(frozen=True)
class KeptWindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    keep_first: int
    rot: RotaryConfig

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "KeptWindowAttentionConfig":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"), where)
        heads, kv, dim, vdim = _heads(m, where)
        window, keep = _mask(m.get("mask"), where + ".mask", may_keep=True)
        c = cls(heads, kv, dim, vdim, float(_need(m, "scale", where)), window, keep,
                RotaryConfig.from_dict(_need(m, "rot", where), where + ".rot"))
        if c.rot.dims > c.dim:
            raise ConfigError(f"config.json: {where}: rot.dims beyond dim")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict()}
        if self.window is not None:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first} if self.keep_first else {"size": self.window}
        return d

    def spec(self, D: int, eps: float):
        return part("attention", hidden_size=D, num_heads=self.heads, num_kv_heads=self.kv_heads, head_dim=self.dim,
                    value_dim=self.vdim, softmax_scale=self.scale, retention=_retention(self.window, self.keep_first),
                    position=self.rot.spec("adjacent"), bias=True)


@dataclasses.dataclass(frozen=True)
class GatedDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "GatedDeltaConfig":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        heads, kv, dim, vdim = _heads(m, where)
        c = cls(heads, kv, dim, vdim, int(m.get("conv") or 0))
        if c.conv < 0:
            raise ConfigError(f"config.json: {where}: a negative conv")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim}
        if self.conv:
            d["conv"] = self.conv
        return d

    def spec(self, D: int, eps: float):
        return part("gated_delta", hidden_size=D, num_heads=self.heads, num_kv_heads=self.kv_heads, head_dim=self.dim,
                    value_dim=self.vdim, conv_taps=self.conv, norm_eps=eps, unit_floor=UNIT_FLOOR)


@dataclasses.dataclass(frozen=True)
class ParallelMixerConfig:
    left: KeptWindowAttentionConfig
    right: GatedDeltaConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "ParallelMixerConfig":
        _only(m, ("left", "right", "left_scale", "right_scale"), where)
        return cls(KeptWindowAttentionConfig.from_dict(_need(m, "left", where), where + ".left"),
                   GatedDeltaConfig.from_dict(_need(m, "right", where), where + ".right"),
                   float(_need(m, "left_scale", where)), float(_need(m, "right_scale", where)))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}

    def spec(self, D: int, eps: float):
        return part("side_by_side", hidden_size=D, left=self.left.spec(D, eps), right=self.right.spec(D, eps),
                    left_scale=self.left_scale, right_scale=self.right_scale)


@dataclasses.dataclass(frozen=True)
class GroupedExpertsConfig:
    experts: int
    top: int
    ff: int
    groups: Optional[int]  # None: every expert can be chosen
    keep: Optional[int]

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "GroupedExpertsConfig":
        _only(m, ("kind", "router", "expert"), where)
        if _need(m, "kind", where) != "moe":
            raise ConfigError(f"config.json: {where}.kind {m['kind']!r} is not known (moe)")
        router, expert = _need(m, "router", where), _need(m, "expert", where)
        _only(router, ("experts", "top", "groups"), where + ".router")
        _only(expert, ("ff",), where + ".expert")
        groups = router.get("groups")
        if groups is not None:
            _only(groups, ("count", "keep"), where + ".router.groups")
        c = cls(experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
                ff=int(_need(expert, "ff", where + ".expert")),
                groups=None if groups is None else int(_need(groups, "count", where + ".router.groups")),
                keep=None if groups is None else int(_need(groups, "keep", where + ".router.groups")))
        if not 1 <= c.top <= c.experts or c.ff < 1:
            raise ConfigError(f"config.json: {where}: 1 <= top <= experts and a positive width are needed")
        if c.groups is not None:
            if c.groups < 1 or c.experts % c.groups or not 1 <= c.keep <= c.groups:
                raise ConfigError(f"config.json: {where}.router.groups: equal groups and 1 <= keep <= count are needed")
            if c.keep * (c.experts // c.groups) < c.top:
                raise ConfigError(f"config.json: {where}.router: the kept groups hold fewer than top experts")
        return c

    def to_dict(self) -> dict:
        router = {"experts": self.experts, "top": self.top}
        if self.groups is not None:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        return {"kind": "moe", "router": router, "expert": {"ff": self.ff}}

    def spec(self, D: int):
        return part("moe_scored", hidden_size=D, num_experts=self.experts, top_k=self.top, intermediate_size=self.ff,
                    activation="relu2", correction=True, groups=self.groups, keep_groups=self.keep,
                    group_score_terms=GROUP_SCORE_TERMS)


@dataclasses.dataclass(frozen=True)
class SudilornLayerConfig:
    type: str
    mixer: Any
    mlp: Optional[GroupedExpertsConfig]


_MIXERS = {"attention": DifferentialAttentionConfig, "parallel": ParallelMixerConfig}


@dataclasses.dataclass(frozen=True)
class SudilornConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: tuple

    @classmethod
    def from_dict(cls, top: Mapping[str, Any]) -> "SudilornConfig":
        _only(top, ("architecture", "architectures", "model_type", "vocab", "width", "norm", "residual_mult", "layers"),
              "the top level")
        layers = []
        for i, entry in enumerate(_need(top, "layers", "the top level")):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = _need(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not known ({', '.join(sorted(_MIXERS))})")
            mlp = entry.get("mlp")
            layers.append(SudilornLayerConfig(
                kind, _MIXERS[kind].from_dict(_need(entry, "mixer", where), where + ".mixer"),
                None if mlp is None else GroupedExpertsConfig.from_dict(mlp, where + ".mlp")))
        if not layers:
            raise ConfigError("config.json: no layers")
        norm = _need(top, "norm", "the top level")
        _only(norm, ("eps",), "norm")
        mult = top.get("residual_mult")
        return cls(vocab=int(_need(top, "vocab", "the top level")), width=int(_need(top, "width", "the top level")),
                   norm_eps=float(_need(norm, "eps", "norm")), residual_mult=1.0 if mult is None else float(mult),
                   layers=tuple(layers))

    def to_dict(self, architecture: str = "Sudilorn") -> dict:
        return {"architecture": architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult,
                "layers": [{"type": lc.type, "mixer": lc.mixer.to_dict(),
                            "mlp": None if lc.mlp is None else lc.mlp.to_dict()} for lc in self.layers]}

    def plan(self) -> ModelPlan:
        D, eps = self.width, self.norm_eps
        norm = part("rmsnorm", eps=eps, size=D, unit_offset=True)
        layers = tuple(
            LayerSpec(mixer=lc.mixer.spec(D, eps), feed_forward=None if lc.mlp is None else lc.mlp.spec(D),
                      mixer_norm=norm, feed_forward_norm=norm, arrangement="pre_norm",
                      options={"hidden_size": D, "layer_scale": True, "branch_mult": self.residual_mult})
            for lc in self.layers)
        return ModelPlan(vocab_size=self.vocab, hidden_size=D, layers=layers,
                         order=tuple(OrderEntry(layer=i, cache=i) for i in range(len(layers))), final_norm=norm,
                         tie_word_embeddings=False,
                         embedding=part("token_embedding", vocab_size=self.vocab, hidden_size=D),
                         head=part("linear_head", vocab_size=self.vocab, hidden_size=D))
