"""Grouped-query attention over the paged cache.

One class covers both of Llama 4's attention layers, by parameters only:
a position encoding that says how q and k are rotated (or none), an RMS norm of q
and k or none (weightless after the rotation for Llama 4; weights and the place
before the rotation are options), a retention rule (every earlier key, or the keys of the query's own chunk), and an
optional position-dependent query scale.  Further options, off for Llama 4: ``bias`` (q, k and v have
biases, added in the projection), ``conv_taps`` (a short causal convolution over time on every channel of q, k and
v, directly behind the projection: ``y[t] = sum_j w[:, j] * u[t - taps + 1 + j]``, zeros before the sequence's
start; the last ``taps - 1`` projected rows of every request are its state, kept in two halves so that a step that
is run twice reads what the first run read) and ``value_dim`` (values of another size than queries and keys: the
pages then hold heads of the larger of the two sizes, rounded up to a multiple of 8, filled up with zeros, and
the output projection skips the zeros).  A second family of options, off for Llama 4 as well: a q/k norm whose
``span`` is ``"projection"`` (one RMS norm over all heads' queries at once, and one over all keys, weights of that
size), ``distance_bias`` (a learned number per head and distance added to the scaled score;
``log_buckets``: a table of ``rows`` rows, the first half one distance each, the other half spread evenly over the
logarithm of the distance up to ``max_distance``, where the last row begins), ``sink`` (a learned number per head
whose exponential is one more term of the softmax's denominator) and ``own_kv = False`` (the layer projects no keys
and values: its run reads the cache that another run writes).  With any of these the rows go through
``qkv_span_prepare`` (norms over the projections, query scale, pages with heads filled up with zeros) and the
attention kernels that take a bias table and sinks.  A third family, off for Llama 4 too: ``score_maps``
(``differential``: every head has two score maps, each a softmax of its own with queries and keys of its own over the
same values; with ``lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` from four learned vectors the head's output is
``a1 - lam a2``, divided by its root mean square and multiplied by ``1 - diff``; q and k rows lie head by head as
``[map 1, map 2]``), ``output_gate`` (the heads side by side times ``sigmoid(W_g h)`` before the output projection),
a weighted q/k norm before the rotation together with a convolution, half-split pairs with a stretch, and the
retention rule ``window_keep`` (a window plus the sequence's first tokens).  With any of these the projected rows go
through ``conv_rows`` (bias, convolution, state), ``heads_prepare`` (norm, rotation, pages with filled-up heads; a
value head written once per score map, so that the attention kernels see ``maps * kv_heads`` key/value heads, the
queries re-ordered at load so that those of a key head lie together) and, for two maps, ``diff_combine``.  Formulas:
``llama4/llama4_jax/model.py:891-955`` (projections, rotation, q/k norm, order of
the cache write) and ``model.py:745-794`` (scores times ``softmax_scale``, causal
mask, float32 softmax, values).
"""
from __future__ import annotations

import math

import torch

from .base import CacheNeed, Mixer, ParamSpec, QKPreparation, build_position, first_needed_position, register_mixer


def log_bucket(distance: int, rows: int, max_distance: int) -> int:
    """The row of a distance table of ``rows`` rows for a key ``distance`` places back: below ``rows // 2`` every
    distance has its row; from there the rows are spread evenly over ``ln(distance)`` so that the last one begins at
    ``max_distance`` (float64)."""
    half = rows // 2
    if distance < half:
        return distance
    return min(rows - 1, half + int(math.floor(math.log(distance / half) / math.log(max_distance / half)
                                               * (rows - half))))


@register_mixer("attention")
class Attention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_heads = int(spec.num_heads)
        self.num_kv_heads = int(spec.num_kv_heads)
        self.head_dim = int(spec.head_dim)
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.softmax_scale = float(spec.softmax_scale)
        self.retention = tuple(spec.retention)
        self.position = build_position(spec.position, self.head_dim)
        qk_norm = spec.get("qk_norm")
        if qk_norm is not None and qk_norm.kind != "rmsnorm":
            raise ValueError(f"the attention mixer norms q and k with an rmsnorm, not {qk_norm.kind!r}")
        self.qk_norm_eps = None if qk_norm is None else float(qk_norm.eps)
        self.qk_norm_weighted = bool(qk_norm is not None and qk_norm.get("weighted", False))
        self.qk_norm_first = bool(qk_norm is not None and qk_norm.get("before_rotation", False))
        self.qk_norm_span = "head" if qk_norm is None else str(qk_norm.get("span") or "head")
        if self.qk_norm_span not in ("head", "projection"):
            raise ValueError(f"a q/k norm spans a head or the projection, not {self.qk_norm_span!r}")
        db = spec.get("distance_bias")
        if db is not None and db.kind != "log_buckets":
            raise ValueError(f"unknown distance_bias kind {db.kind!r}")
        self.bias_rows = None if db is None else int(db.rows)
        self.bias_max = None if db is None else int(db.max_distance)
        if db is not None and not 2 <= self.bias_rows // 2 < self.bias_max:
            raise ValueError("a log_buckets distance table needs at least 4 rows and a max_distance beyond half of them")
        self.has_sink = bool(spec.get("sink", False))
        self.own_kv = bool(spec.get("own_kv", True))
        # the path through the kernel that norms over whole projections, and the attention kernels with bias and sink
        self.spanned = (self.qk_norm_span == "projection" or db is not None or self.has_sink or not self.own_kv)
        qs = spec.get("query_scale")
        if qs is not None and qs.kind != "log_floor_temperature":
            raise ValueError(f"unknown query_scale kind {qs.kind!r}")
        self.query_scale = None if qs is None else (float(qs.floor_scale), float(qs.attn_scale))
        self.prep = QKPreparation(norm_eps=self.qk_norm_eps, norm_first=self.qk_norm_first,
                                  query_scale=self.query_scale)
        self.value_dim = int(spec.get("value_dim") or self.head_dim)
        self.biased = bool(spec.get("bias", False))
        self.conv_taps = int(spec.get("conv_taps") or 0)
        rot = self.position.rotation()
        maps = spec.get("score_maps")
        if maps is not None and maps.kind != "differential":
            raise ValueError(f"unknown score_maps kind {maps.kind!r}")
        self.maps = 1 if maps is None else 2
        self.diff = None if maps is None else float(maps.diff)
        self.head_norm_eps = None if maps is None else float(maps.eps)
        self.output_gate = bool(spec.get("output_gate", False))
        # the path through conv_rows and heads_prepare (see the module's text)
        self.general = (self.maps > 1 or self.output_gate or self.retention[0] == "window_keep"
                        or (not self.spanned and (self.conv_taps > 0 or self.biased or self.value_dim != self.head_dim)
                            and (self.qk_norm_weighted or self.qk_norm_first
                                 or (rot is not None and rot.pairing != "adjacent"))))
        self.lam = None
        if self.spanned:
            if self.qk_norm_span != "projection" or not self.qk_norm_weighted or self.qk_norm_first:
                raise ValueError("distance_bias, sink and own_kv=False come with a weighted q/k norm over the projection")
            if rot is not None or self.biased or self.conv_taps:
                raise ValueError("the attention mixer's path with a q/k norm over the projection has no rotation, no "
                                 "projection bias and no convolution")
        if self.general and (self.spanned or self.query_scale is not None or self.qk_norm_span != "head"):
            raise ValueError("score maps, an output gate, the window_keep rule and a weighted norm with a convolution "
                             "come without a norm over the projection, a distance table, sinks and a query scale")
        # the path through the convolution kernel, which also rotates, norms, fills up and writes the pages
        self.convolved = not self.spanned and not self.general and (self.conv_taps > 0 or self.value_dim != self.head_dim or self.biased
                                               or (rot is not None and rot.magnitude != 1.0))
        if self.convolved and (self.qk_norm_weighted or self.qk_norm_first or self.query_scale is not None):
            raise ValueError("the attention mixer's convolution path norms q and k without weights after the rotation "
                             "and has no query scale")
        # the head size of the pages
        self.page_dim = self.head_dim if not self.convolved else -(-max(self.head_dim, self.value_dim) // 8) * 8
        if self.spanned or self.general:  # (from 32 on a multiple of 32: the sizes the matrix-core attention kernels take)
            widest = max(self.head_dim, self.value_dim)
            self.page_dim = -(-widest // 32) * 32 if widest >= 32 else -(-widest // 8) * 8
        self.state_dtype = None
        self.bias_table = None

    def param_specs(self):
        hq, hk, dh, d = self.num_heads, self.num_kv_heads, self.head_dim, self.hidden
        dv = self.value_dim
        channels = self.channels
        extra = {}
        if self.spanned:
            extra["q_norm"] = ParamSpec((hq * dh,), policy="float32", init=("uniform", 0.5, 1.5))
            if self.own_kv:
                extra["k_norm"] = ParamSpec((hk * dh,), policy="float32", init=("uniform", 0.5, 1.5))
            if self.bias_rows is not None:
                extra["rel"] = ParamSpec((self.bias_rows, hq), policy="float32", init=("normal", 1.0))
            if self.has_sink:
                extra["sink"] = ParamSpec((hq,), policy="float32", init=("normal", 1.0))
        if self.biased:
            extra["bqkv"] = ParamSpec((channels,), policy="float32", init=("normal", 0.3))
        if self.conv_taps:
            extra["conv"] = ParamSpec((channels, self.conv_taps), policy="float32", init=("normal", 0.6))
        if self.output_gate:
            extra["wg"] = ParamSpec((hq * dv, d), init=("normal", d ** -0.5))
        if self.maps > 1:
            for name in ("lam_q1", "lam_k1", "lam_q2", "lam_k2"):
                extra[name] = ParamSpec((dh,), policy="float32", init=("normal", 0.3))
        return {
            # rows: q heads (head by head, a head's score maps one after the other), then k heads, then v heads
            "wqkv": ParamSpec((channels, d)),
            "wo": ParamSpec((d, hq * dv)),
            **extra,
            **({"q_norm": ParamSpec((dh,), policy="float32", init=("ones",)),
                "k_norm": ParamSpec((dh,), policy="float32", init=("ones",))}
               if self.qk_norm_weighted and not self.spanned else {}),
        }

    @property
    def channels(self) -> int:
        if not self.own_kv:  # (queries only)
            return self.num_heads * self.head_dim
        return (self.num_heads + self.num_kv_heads) * self.maps * self.head_dim + self.num_kv_heads * self.value_dim

    def distance_table(self) -> torch.Tensor:
        """The learned table told per head and distance, float32 ``[heads, max_distance + 1]``: column ``n`` is what a
        key ``n`` places back adds to the score, the last column what every key further back adds."""
        rel = self.params["rel"]
        row_of = [log_bucket(n, self.bias_rows, self.bias_max) for n in range(self.bias_max + 1)]
        return rel[torch.tensor(row_of, device=rel.device)].t().contiguous()

    def allocate(self, dtype, device) -> None:
        super().allocate(dtype, device)
        self.state_dtype = dtype

    def cache_need(self) -> CacheNeed:
        if self.general:  # (the attention kernels see a key/value head per score map)
            kv = (self.num_kv_heads * self.maps, self.page_dim)
            if self.conv_taps > 1:
                return CacheNeed(kv=kv, retention=self.retention, state_shape=(2, self.conv_taps - 1, self.channels),
                                 state_dtype=self.state_dtype)
            return CacheNeed(kv=kv, retention=self.retention)
        if self.conv_taps > 1:  # [half, tap, channel]: the last taps - 1 projected rows, as the projection left them
            return CacheNeed(kv=(self.num_kv_heads, self.page_dim), retention=self.retention,
                             state_shape=(2, self.conv_taps - 1, self.channels), state_dtype=self.state_dtype)
        return CacheNeed(kv=(self.num_kv_heads, self.page_dim), retention=self.retention)

    graph_safe = True

    def finalize(self) -> None:
        if self.spanned:
            self.bias_table = self.distance_table() if self.bias_rows is not None else None
        rot = self.position.rotation()
        if rot is not None:
            rot.inv_freq = rot.inv_freq.to(self.params["wqkv"].device)
        self.prep.rotation = rot
        self.prep.norm_weight_q = self.params.get("q_norm")
        self.prep.norm_weight_k = self.params.get("k_norm")
        self.prep.norm_span = self.qk_norm_span
        self.bias_run = None
        if self.biased:  # (the library's product adds a bias of its operands' dtype)
            self.bias_run = self.params["bqkv"].to(self.params["wqkv"].dtype)
        # a tap's weights of all channels side by side, as the kernels read them
        self.conv_by_tap = self.params["conv"].t().contiguous() if self.conv_taps else None
        if self.maps > 1 and self.lam is None:
            # the queries of a key head (a kv head's map) next to each other: [kv head][map][query head of the group]
            P = self.params
            self.lam = float(torch.exp((P["lam_q1"].double() * P["lam_k1"].double()).sum())
                             - torch.exp((P["lam_q2"].double() * P["lam_k2"].double()).sum()) + self.diff)
            r, dh = self.num_heads // self.num_kv_heads, self.head_dim
            order = [((g * r + j) * self.maps + mp) * dh + e for g in range(self.num_kv_heads)
                     for mp in range(self.maps) for j in range(r) for e in range(dh)]
            nq = len(order)
            idx = torch.tensor(order, device=P["wqkv"].device)
            for name in ("wqkv", "bqkv", "conv"):
                if name in P:
                    P[name][:nq] = P[name][:nq][idx]
            self.bias_run = None if not self.biased else P["bqkv"].to(P["wqkv"].dtype)
            self.conv_by_tap = P["conv"].t().contiguous() if self.conv_taps else None
        self.wo_padded = None
        if self.page_dim != self.value_dim and self.maps == 1:  # the attention's output has page_dim elements a head: zeros' columns
            wo = self.params["wo"]
            padded = torch.zeros(wo.shape[0], self.num_heads, self.page_dim, dtype=wo.dtype, device=wo.device)
            padded[:, :, : self.value_dim] = wo.view(wo.shape[0], self.num_heads, self.value_dim)
            self.wo_padded = padded.view(wo.shape[0], self.num_heads * self.page_dim)

    def mixing_flops(self, start: int, count: int) -> float:
        """Two products (scores, values) over the keys each query can see."""
        keys = sum(p - first_needed_position(self.retention, p) + 1 for p in range(start, start + count))
        return 2.0 * self.num_heads * (self.head_dim + self.value_dim) * keys

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        ops = ctx.ops
        if self.general:
            mp = self.maps
            proj, bias = ops.linear_bias(h, self.params["wqkv"], self.params.get("bqkv"), self.bias_run)
            gate = ops.linear(h, self.params["wg"]) if self.output_gate else None
            rows = ops.conv_rows(proj, bias, self.conv_by_tap, self.conv_taps, cache.state, ctx)
            q = ops.heads_prepare(rows, self.num_heads * mp, self.num_kv_heads * mp, self.num_kv_heads, self.head_dim,
                                  self.value_dim, self.page_dim, self.prep, ctx.positions,
                                  cache.kv if cache.writes else None, cache.slot_mapping)
            o = ops.paged_attention(q, cache.kv, cache.block_table, ctx.positions, ctx.token_segment, self.retention,
                                    self.softmax_scale, cache.attn_meta)
            if mp > 1:
                o = ops.diff_combine(o, self.lam, 1.0 - self.diff, self.head_norm_eps, gate, self.num_heads,
                                     self.num_kv_heads, self.page_dim, self.value_dim)
                return ops.linear(o, self.params["wo"])
            if gate is not None:
                if self.page_dim != self.value_dim:
                    raise ValueError("an output gate on heads that are filled up with zeros is not provided for")
                o = ops.sigmoid_mul(o, gate)
            return ops.linear(o, self.params["wo"] if self.wo_padded is None else self.wo_padded)
        if self.spanned:
            if cache.writes != self.own_kv:
                raise ValueError("a run writes its cache if and only if its layer projects keys and values")
            rows = ops.linear(h, self.params["wqkv"])
            q = ops.qkv_span_prepare(rows, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                                     self.page_dim, self.own_kv, self.prep, ctx.positions,
                                     cache.kv if cache.writes else None, cache.slot_mapping)
            o = ops.paged_attention(q, cache.kv, cache.block_table, ctx.positions, ctx.token_segment, self.retention,
                                    self.softmax_scale, cache.attn_meta, bias=self.bias_table,
                                    sink=self.params.get("sink"))
            return ops.linear(o, self.params["wo"] if self.wo_padded is None else self.wo_padded)
        if self.convolved:
            # the projection (its bias added by the product where the library does it, else by the kernel that reads
            # the rows next); then convolution from the rows and the request's state, rotation, norm, pages, attention
            proj, bias = ops.linear_bias(h, self.params["wqkv"], self.params.get("bqkv"), self.bias_run)
            o = ops.conv_attention(proj, bias, self.conv_by_tap, self.conv_taps, cache.state, self.num_heads,
                                   self.num_kv_heads, self.head_dim, self.value_dim, self.page_dim, self.prep, ctx,
                                   cache.kv, cache.writes, cache.slot_mapping, cache.block_table, self.retention,
                                   self.softmax_scale, cache.attn_meta)
            return ops.linear(o, self.params["wo"] if self.wo_padded is None else self.wo_padded)
        qkv = ops.linear(h, self.params["wqkv"])
        o = ops.attention_from_qkv(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx.positions, ctx.token_segment, self.prep,
            cache.kv, cache.writes, cache.slot_mapping, cache.block_table, self.retention, self.softmax_scale,
            cache.attn_meta,
        )
        return ops.linear(o, self.params["wo"])
