"""Typed configuration of the Mazotar decoder, read from ``config.json``.

The file lists the model's layers one by one: ``{"architecture": "Mazotar", "vocab": V, "width": D,
"embedding": {"scale": s}, "norm": {"eps": e}, "streams": S, "layers": [{"type": ..., "mixer": {...},
"mlp": {...} | null}, ...]}``.  A layer's ``type`` names its mixer.  Every size and constant that can differ between
two models of the design is a key of the file; ``streams`` and ``embedding`` may be absent (one residual stream with
a plain sum; a multiplier of one), and a key this reader does not know is an error.

Mixer ``attention``: ``heads``, ``kv_heads``, ``dim`` (query/key elements per head), ``vdim`` (value elements per
head), ``scale`` (of the scores), ``q_temp = {"coef", "every"}`` (the position-dependent multiplier of the queries),
``bias_max`` (the distance at which the learned distance table's last row begins), optionally ``bias_rows`` (the
rows of that table; where the file does not say, the stored table's shape does, see ``complete``) and optionally
``kv_from = j``: the layer projects no keys and values and reads what layer ``j`` cached.
Mixer ``mlstm``: ``heads``, ``dim`` (query/key elements per head), ``vdim``, ``gate_cap`` (the soft cap of the two
gates' pre-activations).
Feed-forward ``dense``: ``ff``.  Feed-forward ``moe``: ``router = {"experts", "top"}``, ``expert = {"ff"}`` and
optionally ``shared = {"ff"}`` (an expert that every token uses, behind a sigmoid gate of one number a token).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional

from .llama4 import ConfigError
from .rovidra import DenseFeedForwardConfig, _need, _only
from .specs import LayerSpec, ModelPlan, OrderEntry, part

# fixed by the design
SINUSOID_BASE = 10000.0


@dataclasses.dataclass(frozen=True)
class BiasedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: Optional[float]  # None: no query temperature
    temp_every: Optional[float]
    bias_max: int
    kv_from: Optional[int]
    bias_rows: Optional[int] = None  # None: not known yet (the checkpoint's table says)

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "BiasedAttentionConfig":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "q_temp", "bias_max", "bias_rows", "kv_from"), where)
        heads, dim = int(_need(m, "heads", where)), int(_need(m, "dim", where))
        qt = m.get("q_temp")
        if qt is not None:
            _only(qt, ("coef", "every"), where + ".q_temp")
        c = cls(heads=heads, kv_heads=int(m["kv_heads"]) if m.get("kv_heads") is not None else heads, dim=dim,
                vdim=int(m["vdim"]) if m.get("vdim") is not None else dim, scale=float(_need(m, "scale", where)),
                temp_coef=None if qt is None else float(_need(qt, "coef", where + ".q_temp")),
                temp_every=None if qt is None else float(_need(qt, "every", where + ".q_temp")),
                bias_max=int(_need(m, "bias_max", where)),
                kv_from=None if m.get("kv_from") is None else int(m["kv_from"]),
                bias_rows=None if m.get("bias_rows") is None else int(m["bias_rows"]))
        if c.bias_rows is not None and c.bias_rows < 2:
            raise ConfigError(f"config.json: {where}.bias_rows must be at least 2")
        if min(c.heads, c.kv_heads, c.dim, c.vdim) < 1:
            raise ConfigError(f"config.json: {where}: sizes must be positive")
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: {c.heads} heads are no multiple of {c.kv_heads} kv_heads")
        if c.temp_every is not None and c.temp_every <= 0:
            raise ConfigError(f"config.json: {where}.q_temp.every must be positive")
        if c.bias_max < 2:
            raise ConfigError(f"config.json: {where}.bias_max must be at least 2")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "bias_max": self.bias_max}
        if self.temp_coef is not None:
            d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        if self.bias_rows is not None:
            d["bias_rows"] = self.bias_rows
        return d


@dataclasses.dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "MatrixMemoryConfig":
        _only(m, ("heads", "dim", "vdim", "gate_cap"), where)
        dim = int(_need(m, "dim", where))
        c = cls(heads=int(_need(m, "heads", where)), dim=dim,
                vdim=int(m["vdim"]) if m.get("vdim") is not None else dim, gate_cap=float(_need(m, "gate_cap", where)))
        if min(c.heads, c.dim, c.vdim) < 1 or c.gate_cap <= 0:
            raise ConfigError(f"config.json: {where}: sizes and gate_cap must be positive")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclasses.dataclass(frozen=True)
class RoutedFeedForwardConfig:
    experts: int
    top: int
    ff: int
    shared_ff: Optional[int]  # None: no shared expert

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "RoutedFeedForwardConfig":
        _only(m, ("kind", "router", "expert", "shared"), where)
        router, expert, shared = _need(m, "router", where), _need(m, "expert", where), m.get("shared")
        _only(router, ("experts", "top"), where + ".router")
        _only(expert, ("ff",), where + ".expert")
        if shared is not None:
            _only(shared, ("ff",), where + ".shared")
        c = cls(experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
                ff=int(_need(expert, "ff", where + ".expert")),
                shared_ff=None if shared is None else int(_need(shared, "ff", where + ".shared")))
        if not 1 <= c.top <= c.experts or c.ff < 1 or (c.shared_ff is not None and c.shared_ff < 1):
            raise ConfigError(f"config.json: {where}: 1 <= top <= experts and positive widths are needed")
        return c

    def to_dict(self) -> dict:
        d = {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


def _feed_forward(m: Optional[Mapping[str, Any]], where: str):
    if m is None:
        return None
    kind = _need(m, "kind", where)
    if kind == "dense":
        return DenseFeedForwardConfig.from_dict(m, where)
    if kind == "moe":
        return RoutedFeedForwardConfig.from_dict(m, where)
    raise ConfigError(f"config.json: {where}.kind {kind!r} is not known (dense, moe)")


@dataclasses.dataclass(frozen=True)
class MazotarLayerConfig:
    type: str
    mixer: Any
    mlp: Any  # DenseFeedForwardConfig, RoutedFeedForwardConfig or None


_MIXERS = {"attention": BiasedAttentionConfig, "mlstm": MatrixMemoryConfig}


@dataclasses.dataclass(frozen=True)
class MazotarConfig:
    vocab: int
    width: int
    embedding_scale: Optional[float]
    norm_eps: float
    streams: Optional[int]  # None: one stream and the plain residual sum
    layers: tuple

    @classmethod
    def from_dict(cls, top: Mapping[str, Any]) -> "MazotarConfig":
        _only(top, ("architecture", "architectures", "model_type", "vocab", "width", "embedding", "norm", "streams",
                    "layers"), "the top level")
        layers = []
        for i, entry in enumerate(_need(top, "layers", "the top level")):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = _need(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not known ({', '.join(sorted(_MIXERS))})")
            layers.append(MazotarLayerConfig(kind, _MIXERS[kind].from_dict(_need(entry, "mixer", where), where + ".mixer"),
                                             _feed_forward(entry.get("mlp"), where + ".mlp")))
        if not layers:
            raise ConfigError("config.json: no layers")
        for i, lc in enumerate(layers):
            j = getattr(lc.mixer, "kv_from", None)
            if j is None:
                continue
            if not 0 <= j < i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                raise ConfigError(f"config.json: layers[{i}].mixer.kv_from = {j} must name an earlier attention layer "
                                  "that has keys and values of its own")
            a, b = lc.mixer, layers[j].mixer
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise ConfigError(f"config.json: layers[{i}] reads the keys and values of layers[{j}], whose kv_heads, "
                                  "dim or vdim differ from its own")
        emb = top.get("embedding")
        scale = None
        if emb is not None:
            _only(emb, ("scale",), "embedding")
            scale = None if emb.get("scale") is None else float(emb["scale"])
        streams = top.get("streams")
        if streams is not None and int(streams) < 1:
            raise ConfigError("config.json: streams must be positive")
        return cls(vocab=int(_need(top, "vocab", "the top level")), width=int(_need(top, "width", "the top level")),
                   embedding_scale=scale, norm_eps=float(_need(_need(top, "norm", "the top level"), "eps", "norm")),
                   streams=None if streams is None else int(streams), layers=tuple(layers))

    def to_dict(self, architecture: str = "Mazotar") -> dict:
        d = {"architecture": architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [{"type": lc.type, "mixer": lc.mixer.to_dict(),
                         "mlp": None if lc.mlp is None else lc.mlp.to_dict()} for lc in self.layers]}
        if self.embedding_scale is not None:
            d["embedding"] = {"scale": self.embedding_scale}
        if self.streams is not None:
            d["streams"] = self.streams
        return d

    def complete(self, shapes: Mapping[str, tuple]) -> "MazotarConfig":
        """The sizes that the file leaves to the checkpoint, from its tensors' shapes: the rows of every attention
        layer's distance table (``l<i>.mix.rel``: ``[rows, heads]``)."""
        layers = []
        for i, lc in enumerate(self.layers):
            if lc.type == "attention" and lc.mixer.bias_rows is None:
                shape = shapes.get(f"l{i}.mix.rel")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"config.json: layers[{i}].mixer gives no bias_rows and the checkpoint has no "
                                      f"table l{i}.mix.rel to take them from")
                lc = dataclasses.replace(lc, mixer=dataclasses.replace(lc.mixer, bias_rows=int(shape[0])))
            layers.append(lc)
        return dataclasses.replace(self, layers=tuple(layers))

    def cache_of(self, i: int) -> int:
        j = getattr(self.layers[i].mixer, "kv_from", None)
        return i if j is None else j

    def plan(self) -> ModelPlan:
        D, eps = self.width, self.norm_eps
        norm = part("rmsnorm", eps=eps, size=D)
        layers, order = [], []
        for i, lc in enumerate(self.layers):
            m = lc.mixer
            if lc.type == "attention":
                if m.bias_rows is None:
                    raise ConfigError(f"config.json: layers[{i}].mixer: the rows of the distance table are not known "
                                      "(bias_rows, or a checkpoint to take them from)")
                mixer = part(
                    "attention", hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                    value_dim=m.vdim, softmax_scale=m.scale, retention=("all",), position=part("none"),
                    qk_norm=part("rmsnorm", eps=eps, weighted=True, span="projection"),
                    query_scale=None if m.temp_coef is None else part("log_floor_temperature", floor_scale=m.temp_every,
                                                                      attn_scale=m.temp_coef),
                    distance_bias=part("log_buckets", rows=m.bias_rows, max_distance=m.bias_max), sink=True, own_kv=m.kv_from is None)
            else:
                mixer = part("mlstm", hidden_size=D, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                             gate_cap=m.gate_cap, norm_eps=eps)
            if lc.mlp is None:
                ff = None
            elif isinstance(lc.mlp, DenseFeedForwardConfig):
                ff = part("dense_swiglu", hidden_size=D, intermediate_size=lc.mlp.ff)
            else:
                ff = part("moe_sigmoid_shared", hidden_size=D, num_experts=lc.mlp.experts, top_k=lc.mlp.top,
                          intermediate_size=lc.mlp.ff, shared_intermediate_size=lc.mlp.shared_ff or 0,
                          shared_gate=lc.mlp.shared_ff is not None)
            if self.streams is None:
                layers.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm, feed_forward_norm=norm))
            else:
                layers.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm, feed_forward_norm=norm,
                                        arrangement="hyper_streams", options={"streams": self.streams}))
            order.append(OrderEntry(layer=i, cache=self.cache_of(i),
                                    writes_cache=getattr(m, "kv_from", None) is None))
        return ModelPlan(vocab_size=self.vocab, hidden_size=D, layers=tuple(layers), order=tuple(order),
                         final_norm=norm, tie_word_embeddings=False,
                         embedding=part("token_embedding", vocab_size=self.vocab, hidden_size=D,
                                        multiplier=self.embedding_scale, sinusoid=SINUSOID_BASE),
                         residual=None if self.streams is None else part("streams", streams=self.streams),
                         head=part("linear_head", vocab_size=self.vocab, hidden_size=D))
