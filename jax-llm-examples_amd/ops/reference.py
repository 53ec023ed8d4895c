"""Plain PyTorch statements of every op the engine's kernels implement.

These functions define what each hand-written kernel computes.  They are what
the kernel tests compare against, and they let the cache manager, the step
function and the scheduler be exercised on a machine without a GPU.  They are
*not* a serving path: the engine refuses to run on a GPU without the compiled
kernels, and its entry points refuse a CPU device unless a test asks for these
ops by name.  All arithmetic is float32 inside; results are cast to the dtype
the kernel would write.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def retention_start(retention: tuple, pos: torch.Tensor) -> torch.Tensor:
    """First key position a query at ``pos`` may read (vectorised)."""
    kind = retention[0]
    if kind == "all":
        return torch.zeros_like(pos)
    if kind == "chunk":
        c = int(retention[1])
        return (pos // c) * c
    if kind == "window":
        return (pos - int(retention[1]) + 1).clamp_min(0)
    raise ValueError(f"unknown retention rule {retention!r}")


def values_t(kv_cache: torch.Tensor) -> torch.Tensor:
    """The value planes of the pages as ``[pages, kv_heads, head_dim, page_size]`` (how they lie in memory)."""
    p, _, hk, ps, dh = kv_cache.shape
    return kv_cache[:, 1].view(p, hk, dh, ps)  # a view: writes through it land in the cache


class ReferenceOps:
    name = "reference"

    # ------------------------------------------------------------------ embedding
    def embed(self, token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        return table[token_ids.long()].float()

    def embed_pair(self, token_ids, prev_token_ids, table, pair_table, buckets: int, mul_prev: int, mul_cur: int):
        """``table[token] + pair_table[(prev * mul_prev + token * mul_cur) mod buckets]``, and row ``buckets`` of the
        pair table where there is no token before (``prev < 0``); float32."""
        tok, prev = token_ids.long(), prev_token_ids.long()
        row = torch.where(prev < 0, torch.full_like(tok, buckets), (prev * mul_prev + tok * mul_cur) % buckets)
        return table[tok].float() + pair_table[row].float()

    def embed_sinusoid(self, token_ids, positions, table, multiplier: float, rates):
        """``table[token] * multiplier`` plus the position's sinusoid: entry ``2i`` is ``sin(pos * rates[i])``, entry
        ``2i + 1`` the cosine (``rates``: float32 ``[ceil(hidden / 2)]``; the angle a float32 product); float32."""
        x = table[token_ids.long()].float() * float(multiplier)
        d = x.shape[1]
        ang = positions.float()[:, None] * rates.float()[None, :]
        wave = torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(x.shape[0], -1)
        return x + wave[:, :d]

    # ------------------------------------------------------------------ several residual streams
    def streams_mix_norm(self, xs, update, inw, weight, eps: float, out_dtype, want32: bool = False, norm: bool = True):
        """``xs``: float32 ``[N, S, D]``, changed in place.  With ``update`` (a branch output ``y`` ``[N, D]``, ``mix``
        ``[S, S]`` indexed ``[from, to]``, ``outw`` ``[S]``): ``X_t <- sum_s mix[s, t] X_s + outw[t] y`` for all ``t``
        at once.  Then (``norm``) ``u = sum_s inw[s] X_s`` (``inw`` ``None``: the plain sum) and ``h = u /
        sqrt(mean(u^2) + eps) * weight``.  Returns ``(h in out_dtype, h in float32 or None)``."""
        if update is not None:
            y = self.materialize(update.y).float()
            new = torch.einsum("st,nsd->ntd", update.mix.float(), xs) + update.outw.float()[None, :, None] * y[:, None, :]
            xs.copy_(new)
        if not norm:
            return None, None
        u = xs.sum(dim=1) if inw is None else torch.einsum("s,nsd->nd", inw.float(), xs)
        h = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            h = h * weight.float()
        return h.to(out_dtype), (h if want32 else None)

    # ------------------------------------------------------------------ a matrix memory per head
    def mlstm(self, rows, gates, b_gates, norm_weight, num_heads: int, head_dim: int, value_dim: int, cap: float,
              eps: float, floor: float, state, ctx):
        """``rows``: ``[N, 2 H dk + 2 H dv]`` = q | k | v | output gate in the run dtype; ``gates``: float32 ``[N, 2 H]``
        = the input gates' and the forget gates' pre-activations without their biases ``b_gates``.  Per head, token
        by token from the request's state (``state[slot, phase]``: ``[H, dk dv + dk + 1]`` = C, n, m; the new state
        goes to ``state[slot, 1 - phase]``)::

            i = cap tanh((a + b_i) / cap);  f = logsigmoid(cap tanh((b + b_f) / cap));  m' = max(f + m, i)
            C' = exp(f + m - m') C + exp(i - m') k v^T;  n' likewise with k;  o = C'^T q / (max(|n' . q|, exp(-m')) + floor)

        with ``q`` times ``dk^(-1/2)``; then every head's ``o`` divided by its root mean square (``eps``), times
        ``norm_weight``, times the sigmoid of the output gate.  ``[N, H dv]`` in the run dtype."""
        n = rows.shape[0]
        H, dk, dv = num_heads, head_dim, value_dim
        r = rows.float()
        q = r[:, : H * dk].reshape(n, H, dk) * (dk ** -0.5)
        k = r[:, H * dk: 2 * H * dk].reshape(n, H, dk)
        v = r[:, 2 * H * dk: 2 * H * dk + H * dv].reshape(n, H, dv)
        og = r[:, 2 * H * dk + H * dv:]
        pre = gates.float() + b_gates.float()
        squashed = cap * torch.tanh(pre / cap)
        log_in, log_keep = squashed[:, :H], torch.nn.functional.logsigmoid(squashed[:, H:])
        out = torch.empty(n, H, dv, dtype=torch.float32, device=rows.device)
        cu = ctx.cu_seqlens.tolist()
        slots, phase = ctx.state_slots.tolist(), ctx.state_phase.tolist()
        for s in range(len(cu) - 1):
            st = state[slots[s], phase[s]].float()
            C = st[:, : dk * dv].reshape(H, dk, dv).clone()
            nn_ = st[:, dk * dv: dk * dv + dk].clone()
            m = st[:, dk * dv + dk].clone()
            for t in range(cu[s], cu[s + 1]):
                m_new = torch.maximum(log_keep[t] + m, log_in[t])
                keep, take = torch.exp(log_keep[t] + m - m_new), torch.exp(log_in[t] - m_new)
                C = keep[:, None, None] * C + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
                nn_ = keep[:, None] * nn_ + take[:, None] * k[t]
                m = m_new
                den = torch.maximum((nn_ * q[t]).sum(-1).abs(), torch.exp(-m)) + floor
                out[t] = torch.einsum("hkv,hk->hv", C, q[t]) / den[:, None]
            state[slots[s], 1 - phase[s]] = torch.cat([C.reshape(H, dk * dv), nn_, m[:, None]], dim=1).to(state.dtype)
        o = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
        o = o.reshape(n, H * dv) * norm_weight.float() * torch.sigmoid(og)
        return o.to(rows.dtype)

    # ------------------------------------------------------------------ norms
    def materialize(self, delta):
        """The tensor a branch output that is not formed yet stands for (float32)."""
        if hasattr(delta, "gate"):  # a GatedBranch: rmsnorm((y + b) * sigmoid(g + c)) * weight
            t = delta.y.float() if delta.y_bias is None else delta.y.float() + delta.y_bias.float()
            g = delta.gate.float() if delta.gate_bias is None else delta.gate.float() + delta.gate_bias.float()
            t = t * torch.sigmoid(g)
            t = t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + delta.eps)
            return t if delta.weight is None else t * delta.weight.float()
        if hasattr(delta, "a"):  # a BranchSum
            return delta.a.float() if delta.b is None else delta.a.float() + delta.b.float()
        if hasattr(delta, "terms"):  # a ScaledSum: vector * sum_i factor_i * term_i
            total = None
            for t, f in delta.terms:
                piece = self.materialize(t).float() * f
                total = piece if total is None else total + piece
            return total if delta.vector is None else total * delta.vector.float()
        return delta

    def add_norm_pair(self, x, delta, injected, weight_a, weight_b, eps: float, out_dtype, second: bool = False,
                      norm: bool = True):
        """``x += delta`` (in place, float32; a tensor, a sum of two branches or ``None``), then with ``injected =
        (rows, vector)`` ``x += rows`` (if any) and ``x += vector``; then ``h = x / sqrt(mean(x^2) + eps)`` once and
        ``h * weight_a`` and (``second``) ``h * weight_b``, in the run dtype.  ``norm=False``: the sums only."""
        if delta is not None:
            x.add_(self.materialize(delta).float())
        if injected is not None:
            rows, vector = injected
            if rows is not None:
                x.add_(rows)
            x.add_(vector.float())
        if not norm:
            return None, None
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        h_a = (h if weight_a is None else h * weight_a.float()).to(out_dtype)
        h_b = None
        if second:
            h_b = (h if weight_b is None else h * weight_b.float()).to(out_dtype)
        return h_a, h_b

    def add_norm_shift(self, x, delta, weight, eps: float, out_dtype, shift, ctx):
        """``x' = x + delta`` (a new tensor, float32; ``delta`` a tensor, a gated branch or ``None``), ``h =
        rmsnorm(x') * weight`` and, with ``shift = (w, state)``, ``hs = h + (h_prev - h) * w`` where ``h_prev`` is
        the float32 ``h`` of the token before: the row before in the same segment, or for a segment's first row
        the request's state (``state[slot, phase]``; zeros at position 0).  The last row's ``h`` of every segment
        goes into ``state[slot, 1 - phase]``.  Returns ``(x', h, hs or None)``."""
        x = x if delta is None else x + self.materialize(delta).float()
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            h = h * weight.float()
        hs = None
        if shift is not None:
            w, state = shift
            prev = torch.empty_like(h)
            prev[1:] = h[:-1]
            cu = ctx.cu_seqlens.long()
            first, last = cu[:-1], cu[1:] - 1
            slots, phase = ctx.state_slots.long(), ctx.state_phase.long()
            carried = state[slots, phase].float()
            carried = torch.where((ctx.positions.long()[first] == 0)[:, None], torch.zeros_like(carried), carried)
            prev[first] = carried
            state[slots, 1 - phase] = h[last].to(state.dtype)
            hs = (h + (prev - h) * w.float()).to(out_dtype)
        return x, h.to(out_dtype), hs

    def add_rmsnorm(self, x, delta, weight, eps: float, out_dtype, want32: bool = False):
        """``x += delta`` (in place, float32), then ``h = x / sqrt(mean(x^2) + eps) * weight``."""
        delta = self.materialize(delta)
        if delta is not None:
            x.add_(delta.float())
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            h = h * weight.float()
        return h.to(out_dtype), (h if want32 else None)

    def add_residual(self, x, delta) -> None:
        x.add_(self.materialize(delta).float())

    def gather_rows(self, x, idx):
        return x[idx.long()]

    # ------------------------------------------------------------------ matrix products
    def linear(self, h, w, out_dtype=None):
        out = h.float() @ w.float().t()
        return out.to(out_dtype or h.dtype)

    def lm_head(self, h, w, tiled: bool = False):
        assert not tiled, "the plain ops read row-major weights"
        return h.float() @ w.float().t()

    def linear_bias(self, h, w, bias, bias_run=None):
        """``h @ w.T + bias`` rounded once to the run dtype.  Returns ``(rows, bias still to be added or None)``:
        a kernel set may leave the addition to the kernel that reads the rows next."""
        out = h.float() @ w.float().t()
        if bias is not None:
            out = out + bias.float()
        return out.to(h.dtype), None

    def swiglu_linear(self, h, w_gate_up, activation: str = "silu"):
        return self.silu_mul(self.linear(h, w_gate_up), activation)

    def silu_mul(self, gate_up, activation: str = "silu"):
        """``act(gate) * up`` of the two halves of the last axis; ``act``: ``silu`` or ``gelu_tanh``."""
        f = gate_up.shape[-1] // 2
        g, u = gate_up[..., :f].float(), gate_up[..., f:].float()
        if activation == "gelu_tanh":
            a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
        else:
            a = torch.nn.functional.silu(g)
        return (a * u).to(gate_up.dtype)

    def softcap_(self, logits, cap: float):
        """``cap * tanh(logits / cap)`` in place."""
        return logits.copy_(torch.tanh(logits / cap) * cap)

    def sigmoid_mul(self, o, gate):
        """``o * sigmoid(gate)`` element by element (``gate``: a view with the same shape), float32 inside."""
        return (o.float() * torch.sigmoid(gate.float())).to(o.dtype)

    def conv_attention(self, proj, bias, conv_w, taps: int, state, num_heads: int, num_kv_heads: int, head_dim: int,
                       value_dim: int, page_dim: int, prep, ctx, kv_cache, writes: bool, slot_mapping, block_table,
                       retention, scale: float, meta=None):
        """From the projected q|k|v rows to the attention output ``[N, num_heads * page_dim]``: bias, convolution
        over time (with the requests' state), rotation and norm of q and k, pages written (if this run writes its
        cache), attention over the pages; see :meth:`conv_qk_prepare`."""
        q = self.conv_qk_prepare(proj, bias, conv_w, taps, state, num_heads, num_kv_heads, head_dim, value_dim,
                                 page_dim, prep, ctx, kv_cache if writes else None, slot_mapping)
        return self.paged_attention(q, kv_cache, block_table, ctx.positions, ctx.token_segment, retention, scale, meta)

    def conv_qk_prepare(self, proj, bias, conv_w, taps: int, state, num_heads: int, num_kv_heads: int, head_dim: int,
                        value_dim: int, page_dim: int, prep, ctx, kv_cache, slot_mapping):
        """From the projected rows ``[N, Hq*dk + Hk*dk + Hk*dv]`` to prepared queries and written pages.
        ``u = proj + bias`` (rounded to the run dtype); every channel's causal convolution over time, ``y[t] =
        sum_j conv_w[j] * u[t - taps + 1 + j]`` (``conv_w``: float32 ``[taps, channels]``), the rows before a segment's start from the request's state
        (``state[slot, phase]``: ``[taps - 1, channels]``, the oldest first; zeros before the sequence's start) -
        the last ``taps - 1`` rows of ``u`` go into ``state[slot, 1 - phase]``; ``y`` rounded to the run dtype; then
        q and k turned by ``prep.rotation`` (sines and cosines times its magnitude) and divided by their root mean
        square over the head; k and v written into their pages with heads of ``page_dim`` elements (zeros behind
        the ``head_dim`` or ``value_dim`` real ones).  Returns q ``[N, Hq, page_dim]``."""
        n = proj.shape[0]
        dt = proj.dtype
        hq, hk, dk, dv, D = num_heads, num_kv_heads, head_dim, value_dim, page_dim
        u = proj.float() if bias is None else (proj.float() + bias.float())
        u = u.to(dt).float()
        y = u
        if taps:
            y = torch.zeros_like(u)
            cu = ctx.cu_seqlens.tolist()
            slots, phase = ctx.state_slots.tolist(), ctx.state_phase.tolist()
            w = conv_w.float()
            for s in range(len(cu) - 1):
                lo, hi = cu[s], cu[s + 1]
                rows = u[lo:hi]
                if taps > 1:
                    rows = torch.cat([state[slots[s], phase[s]].float(), rows], dim=0)  # [taps - 1 + len, C]
                for j in range(taps):
                    y[lo:hi] += w[j] * rows[j: j + hi - lo]
                if taps > 1:
                    state[slots[s], 1 - phase[s]] = rows[rows.shape[0] - (taps - 1):].to(state.dtype)
            y = y.to(dt).float()
        q = y[:, : hq * dk].reshape(n, hq, dk)
        k = y[:, hq * dk: (hq + hk) * dk].reshape(n, hk, dk)
        v = y[:, (hq + hk) * dk:].reshape(n, hk, dv)
        q, k = self._turn(q, ctx.positions, prep.rotation), self._turn(k, ctx.positions, prep.rotation)
        if prep.norm_eps is not None:
            q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + prep.norm_eps)
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + prep.norm_eps)
        pad = lambda t: torch.nn.functional.pad(t, (0, D - t.shape[-1]))
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            page, off = (slot_mapping // ps).long(), (slot_mapping % ps).long()
            kv_cache[page, 0, :, off] = pad(k).to(kv_cache.dtype)
            values_t(kv_cache)[page, :, :, off] = pad(v).to(kv_cache.dtype)
        return pad(q).to(dt).contiguous()

    def conv_rows(self, proj, bias, conv_w, taps: int, state, ctx, activation=None):
        """``u = proj + bias`` rounded to the run dtype; ``y[t] = sum_j conv_w[j] * u[t - taps + 1 + j]`` per channel
        (``conv_w``: float32 ``[taps, channels]``; without taps ``y = u``), the rows before a segment's start from
        the request's state (``state[slot, phase]``: ``[taps - 1, channels]``, oldest first; zeros before the
        sequence's start), whose other half gets the last ``taps - 1`` rows of ``u``; ``activation = "silu"``:
        ``y * sigmoid(y)``; ``[N, channels]`` rounded to the run dtype."""
        dt = ctx.dtype
        u = proj.float() if bias is None else (proj.float() + bias.float())
        u = u.to(dt).float()
        y = u
        if taps:
            y = torch.zeros_like(u)
            cu = ctx.cu_seqlens.tolist()
            slots, phase = ctx.state_slots.tolist(), ctx.state_phase.tolist()
            w = conv_w.float()
            for s in range(len(cu) - 1):
                lo, hi = cu[s], cu[s + 1]
                rows = u[lo:hi]
                if taps > 1:
                    rows = torch.cat([state[slots[s], phase[s]].float(), rows], dim=0)
                for j in range(taps):
                    y[lo:hi] += w[j] * rows[j: j + hi - lo]
                if taps > 1:
                    state[slots[s], 1 - phase[s]] = rows[rows.shape[0] - (taps - 1):].to(state.dtype)
        if activation == "silu":
            y = y * torch.sigmoid(y)
        elif activation is not None:
            raise ValueError(f"unknown activation {activation!r}")
        return y.to(dt)

    def heads_prepare(self, rows, q_heads: int, k_heads: int, v_heads: int, head_dim: int, value_dim: int,
                      page_dim: int, prep, positions, kv_cache, slot_mapping):
        """``rows``: ``[N, q_heads dk + k_heads dk + v_heads dv]`` = q | k | v.  q and k per head: ``prep``'s RMS
        norm (weights of ``dk`` elements or none, before or after the rotation) and rotation (adjacent or half-split
        pairs of the leading elements, sines and cosines times the magnitude); k and v written into their pages
        (if ``kv_cache`` is given: ``k_heads`` heads of ``page_dim`` elements, zeros behind the real ones; value head
        ``j`` goes to the ``k_heads / v_heads`` key heads ``j * share .. (j + 1) * share - 1``).  Returns q ``[N,
        q_heads, page_dim]`` in the run dtype."""
        n = rows.shape[0]
        dt = rows.dtype
        dk, dv, D = head_dim, value_dim, page_dim
        r = rows.float()
        q = r[:, : q_heads * dk].reshape(n, q_heads, dk)
        k = r[:, q_heads * dk: (q_heads + k_heads) * dk].reshape(n, k_heads, dk)
        v = r[:, (q_heads + k_heads) * dk:].reshape(n, v_heads, dv)

        def norm(x, w):
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + prep.norm_eps)
            return x if w is None else x * w.float()

        if prep.norm_eps is not None and prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        q, k = self._turn(q, positions, prep.rotation), self._turn(k, positions, prep.rotation)
        if prep.norm_eps is not None and not prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        pad = lambda t: torch.nn.functional.pad(t, (0, D - t.shape[-1]))
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            page, off = (slot_mapping // ps).long(), (slot_mapping % ps).long()
            kv_cache[page, 0, :, off] = pad(k).to(kv_cache.dtype)
            values_t(kv_cache)[page, :, :, off] = pad(v).repeat_interleave(k_heads // v_heads, dim=1).to(kv_cache.dtype)
        return pad(q).to(dt).contiguous()

    def diff_combine(self, o, lam: float, out_scale: float, eps: float, gate, num_heads: int, num_kv_heads: int,
                     page_dim: int, value_dim: int):
        """``o``: ``[N, 2 H page_dim]``, the outputs of the two score maps in the order ``[kv head][map][query head
        of the group]``.  Per head ``d = a1 - lam * a2`` over its ``value_dim`` real elements, divided by its root
        mean square (``eps``), times ``out_scale`` and, with ``gate`` (``[N, H value_dim]``), times its sigmoid;
        ``[N, H value_dim]`` in the heads' own order, run dtype."""
        n = o.shape[0]
        H, G = num_heads, num_kv_heads
        a = o.float().reshape(n, G, 2, H // G, page_dim)[..., :value_dim]
        d = (a[:, :, 0] - lam * a[:, :, 1]).reshape(n, H, value_dim)
        d = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * out_scale
        d = d.reshape(n, H * value_dim)
        if gate is not None:
            d = d * torch.sigmoid(gate.float())
        return d.to(o.dtype)

    def gated_delta(self, rows, gates, a_log, dt_bias, norm_weight, out_gate, num_heads: int, num_kv_heads: int,
                    head_dim: int, value_dim: int, eps: float, floor: float, state, ctx):
        """``rows``: ``[N, 2 G dk + H dv]`` = q | k | v behind convolution and activation, run dtype; ``gates``:
        float32 ``[N, 2 H]`` = the write strengths' and the decays' pre-activations.  Per kv head q and k become unit
        vectors (``x / sqrt(sum(x^2) + floor)``), q times ``dk^(-1/2)``; ``beta = sigmoid(.)``, ``g = exp(-exp(a_log)
        softplus(. + dt_bias))``; per head, token by token from the request's memory (``state[slot, phase]``: ``[H,
        dv, dk]``, the transposed ``S``; the new one goes to ``state[slot, 1 - phase]``): ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
        o = S^T q``.  Then ``o`` divided by its root mean square per head (``eps``), times ``norm_weight`` (``[dv]``),
        times ``silu(out_gate)``.  ``[N, H dv]`` in the run dtype."""
        n = rows.shape[0]
        H, G, dk, dv = num_heads, num_kv_heads, head_dim, value_dim
        r = rows.float()
        q = r[:, : G * dk].reshape(n, G, dk)
        k = r[:, G * dk: 2 * G * dk].reshape(n, G, dk)
        v = r[:, 2 * G * dk:].reshape(n, H, dv)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + floor) * (dk ** -0.5)
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + floor)
        q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
        beta = torch.sigmoid(gates[:, :H].float())
        decay = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(gates[:, H:].float() + dt_bias.float()))
        out = torch.empty(n, H, dv, dtype=torch.float32, device=rows.device)
        cu = ctx.cu_seqlens.tolist()
        slots, phase = ctx.state_slots.tolist(), ctx.state_phase.tolist()
        for s in range(len(cu) - 1):
            S = state[slots[s], phase[s]].float().transpose(-1, -2).clone()
            for t in range(cu[s], cu[s + 1]):
                S = decay[t][:, None, None] * S
                u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
                S = S + k[t][:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S, q[t])
            state[slots[s], 1 - phase[s]] = S.transpose(-1, -2).to(state.dtype)
        o = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        g = out_gate.float()
        return (o.reshape(n, H * dv) * (g * torch.sigmoid(g))).to(rows.dtype)

    def batched_linear(self, a, w, tokens_first: bool = False):
        """``out[b] = a[b] @ w[b]`` for ``a [B, N, K]`` and ``w [B, K, M]`` (views with any strides);
        ``[B, N, M]``, or with ``tokens_first`` the same numbers laid out ``[N, B, M]``."""
        out = torch.bmm(a.float(), w.float()).to(a.dtype)
        return out.transpose(0, 1).contiguous() if tokens_first else out

    def polynorm(self, z, bias, coef, eps: float):
        """``c0 N(u) + c1 N(u^2) + c2 N(u^3) + c3`` with ``u = z + bias`` and ``N(v) = v / sqrt(mean(v^2) + eps)``
        over a row, float32 inside."""
        u = z.float() if bias is None else z.float() + bias.float()
        n = lambda v: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        c = coef.float()
        return (c[0] * n(u) + c[1] * n(u * u) + c[2] * n(u * u * u) + c[3]).to(z.dtype)

    # ------------------------------------------------------------------ attention over a cached latent
    @staticmethod
    def _turn(x, positions, rotation):
        """The leading ``rotary_dim`` elements of the last axis turned by ``pos * inv_freq`` (float32 angles)."""
        if rotation is None:
            return x
        rd = int(rotation.rotary_dim) or x.shape[-1]
        ang = positions.float()[:, None] * rotation.inv_freq.float()[None, :]
        grow = float(getattr(rotation, "magnitude", 1.0))
        sin, cos = torch.sin(ang) * grow, torch.cos(ang) * grow
        while sin.dim() < x.dim():
            sin, cos = sin.unsqueeze(1), cos.unsqueeze(1)
        head, rest = x[..., :rd], x[..., rd:]
        if rotation.pairing == "adjacent":
            pairs = head.reshape(*head.shape[:-1], rd // 2, 2)
            a, b = pairs[..., 0], pairs[..., 1]
            head = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).reshape(*head.shape[:-1], rd)
        else:
            a, b = head[..., : rd // 2], head[..., rd // 2:]
            head = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
        return torch.cat([head, rest], dim=-1)

    def latent_prepare(self, rows, num_heads: int, nope_dim: int, rope_dim: int, kv_rank: int, positions, rotation,
                       latent_norm, eps: float, latent_pages, rope_pages, slot_mapping, writes: bool,
                       latent_t_pages=None) -> None:
        """``rows``: ``[N, H * (nope + rope) (+ kv_rank + rope) (+ anything else)]``.  Turns the ``rope`` part of every head's
        query in place; if the run writes its cache: RMS-norms the latent (the ``kv_rank`` numbers behind the
        queries) with ``latent_norm``, turns the shared key part (the last ``rope`` numbers) and writes both
        into their pages at ``slot = page * page_size + offset``."""
        n = rows.shape[0]
        H, dn, dr = num_heads, nope_dim, rope_dim
        q = rows[:, : H * (dn + dr)].view(n, H, dn + dr)
        q[:, :, dn:] = self._turn(q[:, :, dn:].float(), positions, rotation).to(rows.dtype)
        if writes:
            c = rows[:, H * (dn + dr): H * (dn + dr) + kv_rank].float()
            c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps)
            if latent_norm is not None:
                c = c * latent_norm.float()
            kr = self._turn(rows[:, H * (dn + dr) + kv_rank: H * (dn + dr) + kv_rank + dr].float(), positions, rotation)
            ps = latent_pages.shape[1]
            page, off = (slot_mapping // ps).long(), (slot_mapping % ps).long()
            latent_pages[page, off] = c.to(latent_pages.dtype)
            rope_pages[page, off] = kr.to(rope_pages.dtype)
            if latent_t_pages is not None:  # a second copy, per page [kv_rank, page_size]
                latent_t_pages.view(latent_t_pages.shape[0], kv_rank, ps)[page, :, off] = c.to(latent_t_pages.dtype)

    def latent_attention(self, q_lat, q, nope_dim: int, latent_pages, rope_pages, block_table, positions,
                         token_segment, window, scale: float, meta=None, latent_t_pages=None, sink=None):
        """For every token and head: softmax over the visible cached tokens ``j`` (``0 <= pos - j < window``;
        all earlier ones without a window) of ``(q_lat . c_j + q_r . k_j) * scale``, and the sum of the ``c_j``
        with those weights.  ``q_lat``: ``[H, N, kv_rank]``; ``q``: ``[N, H, nope + rope]`` whose rotated part is
        ``q_r``.  ``sink``: float32 ``[H]``; ``exp(sink[h])`` is one more term of head ``h``'s denominator (no
        key, no value, not scaled).  Returns ``[N, H, kv_rank]``."""
        H, n, r = q_lat.shape
        ps = latent_pages.shape[1]
        out = torch.empty(n, H, r, dtype=q_lat.dtype, device=q_lat.device)
        for i in range(n):
            p = int(positions[i])
            s = 0 if window is None else max(0, p - int(window) + 1)
            kpos = torch.arange(s, p + 1, device=q_lat.device)
            pages = block_table[int(token_segment[i])][(kpos // ps).long()].long()
            if bool((pages < 0).any()):
                raise RuntimeError(f"token {i} at position {p} reads a page that was given back")
            off = (kpos % ps).long()
            c = latent_pages[pages, off].float()  # [T, r]
            kr = rope_pages[pages, off].float()  # [T, rope]
            sc = (q_lat[:, i].float() @ c.t() + q[i, :, nope_dim:].float() @ kr.t()) * scale
            if sink is None:
                pr = torch.softmax(sc, dim=-1)
            else:
                top = torch.maximum(sc.max(dim=-1, keepdim=True).values, sink.float()[:, None])
                e = torch.exp(sc - top)
                pr = e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink.float()[:, None] - top))
            out[i] = (pr @ c).to(out.dtype)
        return out

    # ------------------------------------------------------------------ attention
    def qk_prepare_kv_write(self, qkv, num_heads: int, num_kv_heads: int, head_dim: int, positions, prep,
                            kv_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor]):
        """Splits fused q|k|v rows and prepares q and k as ``prep`` (a
        :class:`~..parts.base.QKPreparation`) says: the rotation turns element pairs by the angle
        ``pos * inv_freq[j]`` (float32) - adjacent pairs ``(x[2j], x[2j+1])`` or half-split pairs
        ``(x[j], x[j + rotary_dim/2])`` of the leading ``rotary_dim`` elements; the RMS norm over the
        head (``x / sqrt(mean(x^2) + eps)``, times a weight if there is one) comes after the rotation,
        or before it with ``norm_first``; ``query_scale = (floor_scale, attn_scale)`` multiplies q by
        ``1 + attn_scale * ln(1 + floor((pos + 1) / floor_scale))``.  Then k and v are written into
        their page at ``slot = page * page_size + offset``.  ``kv_cache`` is ``[pages, 2, kv_heads,
        page_size * head_dim]`` in memory: plane 0 holds keys as ``[page_size, head_dim]``, plane 1
        holds values transposed, ``[head_dim, page_size]``.  Returns q ``[N, num_heads, head_dim]``."""
        n = qkv.shape[0]
        dt = qkv.dtype
        hq, hk, dh = num_heads, num_kv_heads, head_dim
        q = qkv[:, : hq * dh].float().reshape(n, hq, dh)
        k = qkv[:, hq * dh : (hq + hk) * dh].float().reshape(n, hk, dh)
        v = qkv[:, (hq + hk) * dh :].float().reshape(n, hk, dh)

        def norm(x, w):
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + prep.norm_eps)
            return x if w is None else x * w.float()

        if prep.norm_eps is not None and prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        rot = prep.rotation
        if rot is not None:
            rd = int(rot.rotary_dim) or dh
            ang = positions.float()[:, None] * rot.inv_freq.float()[None, :]
            grow = float(getattr(rot, "magnitude", 1.0))
            sin, cos = torch.sin(ang)[:, None, :] * grow, torch.cos(ang)[:, None, :] * grow

            def turn(x):
                head, rest = x[..., :rd], x[..., rd:]
                if rot.pairing == "adjacent":
                    pairs = head.reshape(n, -1, rd // 2, 2)
                    a, b = pairs[..., 0], pairs[..., 1]
                    head = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).reshape(n, -1, rd)
                else:
                    a, b = head[..., : rd // 2], head[..., rd // 2:]
                    head = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
                return torch.cat([head, rest], dim=-1)

            q, k = turn(q), turn(k)
        if prep.norm_eps is not None and not prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        if prep.query_scale is not None:
            floor_scale, attn_scale = prep.query_scale
            s = 1.0 + attn_scale * torch.log1p(torch.floor((positions.float() + 1.0) / floor_scale))
            q = q * s[:, None, None]
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            page = (slot_mapping // ps).long()
            off = (slot_mapping % ps).long()
            kv_cache[page, 0, :, off] = k.to(kv_cache.dtype)
            values_t(kv_cache)[page, :, :, off] = v.to(kv_cache.dtype)
        return q.to(dt)

    def qkv_span_prepare(self, rows, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, page_dim: int,
                         own_kv: bool, prep, positions, kv_cache, slot_mapping):
        """``rows``: ``[N, Hq dk]`` (queries only) or, with ``own_kv``, ``[N, Hq dk + Hk dk + Hk dv]``.  One RMS norm
        over all of a token's queries and one over all its keys (``prep.norm_weight_q`` / ``_k`` of those sizes,
        ``prep.norm_eps``), the queries times ``prep.query_scale``'s position-dependent factor; keys and values
        written into their pages (if ``kv_cache`` is given) with heads of ``page_dim`` elements, zeros behind the real
        ones.  Returns q ``[N, Hq, page_dim]`` in the run dtype."""
        n = rows.shape[0]
        dt = rows.dtype
        hq, hk, dk, dv, D = num_heads, num_kv_heads, head_dim, value_dim, page_dim
        r = rows.float()
        rms = lambda x, w: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + prep.norm_eps) * w.float()
        q = rms(r[:, : hq * dk], prep.norm_weight_q)
        if prep.query_scale is not None:
            floor_scale, attn_scale = prep.query_scale
            q = q * (1.0 + attn_scale * torch.log1p(torch.floor((positions.float() + 1.0) / floor_scale)))[:, None]
        pad = lambda t: torch.nn.functional.pad(t, (0, D - t.shape[-1]))
        if kv_cache is not None:
            if not own_kv:
                raise ValueError("rows without keys and values cannot fill pages")
            k = rms(r[:, hq * dk: (hq + hk) * dk], prep.norm_weight_k).reshape(n, hk, dk)
            v = r[:, (hq + hk) * dk:].reshape(n, hk, dv)
            ps = kv_cache.shape[3]
            page, off = (slot_mapping // ps).long(), (slot_mapping % ps).long()
            kv_cache[page, 0, :, off] = pad(k).to(kv_cache.dtype)
            values_t(kv_cache)[page, :, :, off] = pad(v).to(kv_cache.dtype)
        return pad(q.reshape(n, hq, dk)).to(dt).contiguous()

    def attention_from_qkv(self, qkv, num_heads, num_kv_heads, head_dim, positions, token_segment, prep, kv_cache,
                           writes: bool, slot_mapping, block_table, retention, scale: float, meta=None):
        """q and k prepared, k and v written (if this run writes its cache), attention over the pages."""
        q = self.qk_prepare_kv_write(qkv, num_heads, num_kv_heads, head_dim, positions, prep,
                                     kv_cache if writes else None, slot_mapping)
        return self.paged_attention(q, kv_cache, block_table, positions, token_segment, retention, scale, meta)

    def paged_attention(self, q, kv_cache, block_table, positions, token_segment, retention, scale: float, meta=None,
                        bias=None, sink=None):
        """For each token: softmax over the keys of its own request at positions
        ``[start(pos), pos]``, read from the pages its block table names.  ``bias``: float32 ``[Hq, L]``; a key ``n``
        places back adds ``bias[h, min(n, L - 1)]`` to head ``h``'s scaled score.  ``sink``: float32 ``[Hq]``;
        ``exp(sink[h])`` is one more term of head ``h``'s denominator (no key, no value, not scaled, no bias)."""
        n, hq, dh = q.shape
        hk, ps = kv_cache.shape[2], kv_cache.shape[3]
        g = hq // hk
        out = torch.empty(n, hq * dh, dtype=q.dtype, device=q.device)
        keep = 0
        if retention[0] == "window_keep":  # the window's keys and the sequence's first `keep` tokens
            keep, retention = int(retention[2]), ("window", retention[1])
        starts = retention_start(retention, positions)
        for i in range(n):
            p = int(positions[i])
            s = int(starts[i])
            kpos = torch.arange(s, p + 1, device=q.device)
            if keep and s > 0:
                kpos = torch.cat([torch.arange(0, min(keep, s), device=q.device), kpos])
            pages = block_table[int(token_segment[i])][(kpos // ps).long()].long()
            if bool((pages < 0).any()):
                raise RuntimeError(f"token {i} at position {p} reads a page that was given back")
            off = (kpos % ps).long()
            k = kv_cache[pages, 0, :, off].float()  # [T, hk, dh]
            v = values_t(kv_cache)[pages, :, :, off].float()
            qi = q[i].float().reshape(hk, g, dh)
            sc = torch.einsum("hgd,thd->hgt", qi, k) * scale
            if bias is not None:
                back = (p - kpos).clamp_max(bias.shape[1] - 1)
                sc = sc + bias.float()[:, back].reshape(hk, g, -1)
            if sink is None:
                pr = torch.softmax(sc, dim=-1)
            else:
                sk = sink.float().reshape(hk, g, 1)
                top = torch.maximum(sc.max(dim=-1, keepdim=True).values, sk)
                e = torch.exp(sc - top)
                pr = e / (e.sum(dim=-1, keepdim=True) + torch.exp(sk - top))
            out[i] = torch.einsum("hgt,thd->hgd", pr, v).reshape(-1).to(q.dtype)
        return out

    # ------------------------------------------------------------------ routed experts
    def moe_route(self, h32, router, top_k: int, group: bool = False):
        """Router logits in float32, the ``top_k`` largest per token (lowest index
        first among equals), gate = sigmoid of the chosen logit.  ``group``: a third result, the
        grouping of the choices by expert for ``moe_experts`` (none here: these ops do not group)."""
        logits = h32.float() @ router.float().t()
        # stable sort by (-logit, index): lowest index wins ties
        order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :top_k]
        vals = torch.gather(logits, 1, order)
        ids, gates = order.to(torch.int32), torch.sigmoid(vals)
        return (ids, gates, None) if group else (ids, gates)

    def moe_experts(self, h, expert_ids, gates, w_gate_up, w_down, shared=None, tiled: bool = False, grouping=None,
                    shared_weights=None, shared_gate=None):
        """``sum_j  W_down[e_j] (silu(g_j W_gate[e_j] h) * (g_j W_up[e_j] h))`` per token,
        plus ``shared`` if given (``shared_gate = (h32, w)``: times ``sigmoid(h32 . w)``, one float32 number a
        token); float32 result.  ``w_gate_up`` is ``[E, 2F, D]`` (gate rows then
        up rows), ``w_down`` ``[E, D, F]``.  Activations between the two products are
        rounded to the run dtype, as the kernels store them."""
        assert not tiled, "the plain ops read row-major weights"
        if shared is None and shared_weights is not None:
            shared = self.linear(self.swiglu_linear(h, shared_weights[0]), shared_weights[1])
        n, d = h.shape
        f = w_down.shape[2]
        out = torch.zeros(n, d, dtype=torch.float32, device=h.device)
        hf = h.float()
        for j in range(expert_ids.shape[1]):
            for e in torch.unique(expert_ids[:, j]).tolist():
                rows = (expert_ids[:, j] == e).nonzero().squeeze(-1)
                gu = (hf[rows] @ w_gate_up[e].float().t()) * gates[rows, j : j + 1]
                act = (torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]).to(h.dtype).float()
                out[rows] += (act @ w_down[e].float().t()).to(h.dtype).float()
        if shared is not None:
            if shared_gate is not None:
                h32, w = shared_gate
                shared = (shared.float() * torch.sigmoid(h32.float() @ w.float().reshape(-1, 1))).to(shared.dtype)
            out += shared.float()
        return out

    def moe_choose(self, h32, router, correction, top_k: int, groups=None, keep_groups=None, group_terms: int = 2):
        """Router logits ``z`` in float32, scores ``s = sigmoid(z)``, choice scores ``c = s + correction``
        (``correction``: float32 ``[E]`` or ``None``).  With ``groups``: the experts form that many equal groups of
        neighbours, a group's score is the sum of its ``group_terms`` largest ``c``, the ``keep_groups`` best groups
        (lowest index first among equals) stay and the others' experts cannot be chosen.  The ``top_k`` largest ``c``
        among those that can, lowest index first among equals.  Returns ``(ids int32 [N, top_k], their s float32,
        None)`` (the third: the grouping by expert that a kernel set may make in the same call)."""
        z = h32.float() @ router.float().t()
        s = torch.sigmoid(z)
        c = s if correction is None else s + correction.float()
        n, e = c.shape
        if groups is not None:
            per = e // groups
            gs = torch.sort(c.view(n, groups, per), dim=-1, descending=True).values[..., :group_terms].sum(-1)
            kept = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep_groups]
            allowed = torch.zeros(n, groups, dtype=torch.bool, device=c.device)
            allowed.scatter_(1, kept, True)
            c = c.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
        ids = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top_k]
        return ids.to(torch.int32), torch.gather(s, 1, ids), None

    def moe_experts_scored(self, h, expert_ids, weights, w_up, w_down, activation: str = "relu2", tiled: bool = False,
                           grouping=None):
        """``sum_j weights[j] * W_down[e_j] act(W_up[e_j] h)`` per token, float32 result; ``w_up`` ``[E, F, D]``,
        ``w_down`` ``[E, D, F]``; ``act = relu2``: the square of relu.  Activations between the two products and
        every expert's weighted output are rounded to the run dtype, as the kernels store them."""
        assert not tiled, "the plain ops read row-major weights"
        if activation != "relu2":
            raise ValueError(f"unknown activation {activation!r}")
        n, d = h.shape
        out = torch.zeros(n, d, dtype=torch.float32, device=h.device)
        hf = h.float()
        for j in range(expert_ids.shape[1]):
            for e in torch.unique(expert_ids[:, j]).tolist():
                rows = (expert_ids[:, j] == e).nonzero().squeeze(-1)
                act = (torch.relu(hf[rows] @ w_up[e].float().t()) ** 2).to(h.dtype).float()
                out[rows] += ((act @ w_down[e].float().t()) * weights[rows, j: j + 1].float()).to(h.dtype).float()
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, seeds, counters, any_top_k: bool = True):
        """Greedy where ``temperature == 0`` (lowest index among equals); otherwise
        Gumbel-max over ``logits / temperature`` restricted to the ``top_k`` largest
        (0 = all), with noise that depends only on (seed, counter, token id)."""
        m, v = logits.shape
        out = torch.empty(m, dtype=torch.int32, device=logits.device)
        ids = torch.arange(v, device=logits.device, dtype=torch.int64)
        for i in range(m):
            row = logits[i].float()
            t = float(temperature[i])
            if t <= 0.0:
                out[i] = int(torch.argmax(row))  # first maximal index
                continue
            z = row / t
            k = int(top_k[i])
            if 0 < k < v:
                kth = torch.topk(z, k).values[-1]
                z = torch.where(z >= kth, z, torch.full_like(z, -math.inf))
            u = uniform_from_hash(int(seeds[i]), int(counters[i]), ids)
            gumbel = -torch.log(-torch.log(u))
            out[i] = int(torch.argmax(z + gumbel))
        return out


def uniform_from_hash(seed: int, counter: int, ids: torch.Tensor) -> torch.Tensor:
    """A uniform in (0, 1) for every token id from a 32-bit mix of (seed, counter, id).
    The kernel computes the same integers; float32 result."""
    M = 0xFFFFFFFF

    def mix(x):
        x = x & M
        x = ((x ^ (x >> 16)) * 0x7FEB352D) & M
        x = ((x ^ (x >> 15)) * 0x846CA68B) & M
        return (x ^ (x >> 16)) & M

    s = mix(torch.tensor((seed * 0x9E3779B1 + 0x85EBCA6B) & M, dtype=torch.int64))
    c = mix(torch.tensor(((counter + 1) * 0xC2B2AE35) & M, dtype=torch.int64) ^ s)
    x = mix((ids.to(torch.int64) * 0x27D4EB2F + c) & M)
    x = mix(x ^ s)
    # 24 high bits -> (0, 1)
    return ((x >> 8).to(torch.float32) + 0.5) * (1.0 / 16777216.0)
