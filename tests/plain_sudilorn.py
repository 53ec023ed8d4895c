"""A plain, slow implementation of the Sudilorn decoder, written from its equations: one function per mechanism,
whole sequences at a time, float64 unless told otherwise.  It shares no code with the engine: it reads config.json
and model.safetensors itself (with the safetensors package), masks a full score matrix and walks the recurrent layer
token by token.

    x = E[tok];  per layer:  x += m * s1 * mixer(N(x; w1));  x += m * s2 * ff(N(x; w2))      N(v; w) = v / rms(v) * (1 + w)
    logits = head N(x; w_f)                                      rms(v) = sqrt(mean(v^2) + eps)

    mixer "attention" (two score maps per head over the same values):
        q, k, v = conv(W_q h), conv(W_k h), conv(W_v h)          conv: y[t] = sum_j c[:, j] u[t - K + 1 + j]
        q, k per head and map: v / rms(v) * w, then the leading `dims` elements turned (pairs i, i + dims/2)
        A_m = softmax(q_m . k_m * scale) over i - W < j <= i;   lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff
        o = (A_1 - lam A_2) v;  o / rms(o) * (1 - diff);  W_o (o * sigmoid(W_g h))
    mixer "parallel":  a * left(h) + b * right(h)
        left: q, k, v with biases, the leading `dims` elements turned (pairs 2i, 2i + 1), softmax over the keys j <= i
              with i - j < W or j < keep, W_o
        right: q, k, v = silu(conv(W . h));  q, k unit vectors per head (sum of squares + 1e-6), q / sqrt(dk)
              beta = sigmoid(W_b h);  g = exp(-exp(A) softplus(W_a h + dt))
              S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
              W_o (o / rms(o) * w * silu(W_g h))
    ff: z = W_r h;  s = sigmoid(z);  c = s + correction;  groups of neighbouring experts, a group's score the sum of its
        two largest c, the best `keep` groups stay;  the `top` largest c among them;  sum_e s_e W_down relu(W_up h)^2
"""
import json
import math
import os

import torch
from safetensors import safe_open

UNIT_FLOOR = 1e-6  # inside the root of the recurrent mixer's unit vectors


# --------------------------------------------------------------------------------------------------- small pieces
def rms_divide(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, weight, eps):
    return rms_divide(x, eps) * (1.0 + weight)


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(u, taps_weight, before=None):
    """u [T, C]; taps_weight [C, K], the last column is the current token's.  ``before``: the K - 1 rows in front of
    the sequence (zeros if None)."""
    if taps_weight is None:  # (a mixer without a convolution)
        return u
    T, C = u.shape
    K = taps_weight.shape[1]
    if before is None:
        before = torch.zeros(K - 1, C, dtype=u.dtype)
    rows = torch.cat([before, u], dim=0)
    y = torch.zeros_like(u)
    for j in range(K):
        y = y + taps_weight[:, j] * rows[j: j + T]
    return y


def rotary_rates(rot):
    """One rate per pair of the `dims` turned elements, and the factor on sines and cosines."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if sc is None:
        return f, 1.0
    where = lambda t: dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / sc["factor"] * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def turn(x, positions, rot, layout):
    """x [T, heads, d]; the leading rot['dims'] elements of every head are turned."""
    dims = rot["dims"]
    rates, grow = rotary_rates(rot)
    ang = torch.tensor([[p * r for r in rates] for p in positions], dtype=x.dtype)  # [T, dims/2]
    cos, sin = torch.cos(ang)[:, None, :] * grow, torch.sin(ang)[:, None, :] * grow
    out = x.clone()
    if layout == "half":
        a, b = x[..., : dims // 2], x[..., dims // 2: dims]
        out[..., : dims // 2] = a * cos - b * sin
        out[..., dims // 2: dims] = b * cos + a * sin
    else:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    return out


def visible(i, j, size, keep_first=0):
    """``size`` None: no window."""
    return j <= i and (size is None or i - j < size or j < keep_first)


def masked_softmax(scores, positions, size, keep_first=0):
    """scores [T, T] of one head; row i over the visible keys."""
    T = scores.shape[0]
    mask = torch.tensor([[visible(positions[i], positions[j], size, keep_first) for j in range(T)] for i in range(T)])
    return torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)


# --------------------------------------------------------------------------------------------------- mixers
def differential_attention(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ w[p + "q"].T, w.get(p + "q.conv")).reshape(T, H * 2, dk)
    k = causal_conv(h @ w[p + "k"].T, w.get(p + "k.conv")).reshape(T, G * 2, dk)
    v = causal_conv(h @ w[p + "v"].T, w.get(p + "v.conv")).reshape(T, G, dv)
    q = turn(rms_divide(q, eps) * w[p + "q.norm"], positions, m["rot"], "half")
    k = turn(rms_divide(k, eps) * w[p + "k.norm"], positions, m["rot"], "half")
    lam = (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum())
           + m["diff"])
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        a = []
        for mp in range(2):
            sc = (q[:, 2 * hd + mp] @ k[:, 2 * g + mp].T) * m["scale"]
            a.append(masked_softmax(sc, positions, m.get("mask", {}).get("size")) @ v[:, g])
        o = a[0] - lam * a[1]
        heads.append(rms_divide(o, eps) * (1.0 - m["diff"]))
    o = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def kept_window_attention(h, w, p, m, positions):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, dk)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, dk)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, dv)
    q, k = turn(q, positions, m["rot"], "pairs"), turn(k, positions, m["rot"], "pairs")
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        sc = (q[:, hd] @ k[:, g].T) * m["scale"]
        mask = m.get("mask", {})
        heads.append(masked_softmax(sc, positions, mask.get("size"), mask.get("keep_first", 0)) @ v[:, g])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def gated_delta(h, w, p, m, eps, state=None):
    """Token by token.  ``state``: None (a sequence's start) or (S [H, dk, dv], rows before for q, k, v)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    before = (None, None, None) if state is None else state[1]
    uq, uk, uv = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    q = silu(causal_conv(uq, w.get(p + "q.conv"), before[0])).reshape(T, G, dk)
    k = silu(causal_conv(uk, w.get(p + "k.conv"), before[1])).reshape(T, G, dk)
    v = silu(causal_conv(uv, w.get(p + "v.conv"), before[2])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + UNIT_FLOOR) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + UNIT_FLOOR)
    beta = torch.sigmoid(h @ w[p + "b"].T)  # [T, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    S = torch.zeros(H, dk, dv, dtype=h.dtype) if state is None else state[0].clone()
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = decay[t, hd] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, g])
            S[hd] = S[hd] + torch.outer(k[t, g], u)
            out[t, hd] = S[hd].T @ q[t, g]
    taps = w[p + "q.conv"].shape[1] if p + "q.conv" in w else 1
    tail = lambda u, b: torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype) if b is None else b, u])[-(taps - 1):] \
        if taps > 1 else u[:0]
    o = rms_divide(out, eps) * w[p + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, (S, (tail(uq, before[0]), tail(uk, before[1]), tail(uv, before[2])))


def parallel_mixer(h, w, p, m, eps, positions):
    left = kept_window_attention(h, w, p + "left.", m["left"], positions)
    right, _ = gated_delta(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# --------------------------------------------------------------------------------------------------- feed-forward
def choose_experts(z, correction, router):
    """z [E] logits of one token -> (chosen expert ids, their weights)."""
    E, top = router["experts"], router["top"]
    s = torch.sigmoid(z)
    c = s + correction
    groups = router.get("groups")
    allowed = [True] * E
    if groups is not None:
        n, per = groups["count"], E // groups["count"]
        score = []
        for gi in range(n):
            best = sorted((float(c[e]) for e in range(gi * per, (gi + 1) * per)), reverse=True)
            score.append(sum(best[:2]))
        kept = sorted(range(n), key=lambda gi: (-score[gi], gi))[: groups["keep"]]
        allowed = [(e // per) in kept for e in range(E)]
    order = sorted((e for e in range(E) if allowed[e]), key=lambda e: (-float(c[e]), e))[:top]
    return order, [s[e] for e in order]


def routed_experts(h, w, p, mlp, choices=None):
    T = h.shape[0]
    z = h @ w[p + "router"].T
    out = torch.zeros_like(h)
    picked = []
    for t in range(T):
        ids, weights = choose_experts(z[t], w[p + "correction"], mlp["router"])
        if choices is not None:  # (the caller's choice; the weights are still this token's own scores)
            ids = [int(e) for e in choices[t]]
            weights = [torch.sigmoid(z[t, e]) for e in ids]
        picked.append(ids)
        for e, g in zip(ids, weights):
            a = torch.relu(w[p + f"e{e}.up"] @ h[t]) ** 2
            out[t] = out[t] + g * (w[p + f"e{e}.down"] @ a)
    return out, picked


# --------------------------------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, dtype=torch.float64, taps=None, choices=None):
    """Logits [T, vocab] of one whole sequence.  ``taps``: a list that receives the stream behind every layer.
    ``choices``: per layer a [T, top] table of expert ids to use instead of the model's own choice."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    chosen = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = differential_attention(h, w, p + "mix.", layer["mixer"], eps, positions)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", layer["mixer"], eps, positions)
        else:
            raise ValueError(layer["type"])
        x = x + mult * w[p + "ls1"] * y
        if layer.get("mlp") is not None:
            h = offset_norm(x, w[p + "norm2"], eps)
            y, ids = routed_experts(h, w, p + "mlp.", layer["mlp"], None if choices is None else choices[i])
            chosen.append(ids)
            x = x + mult * w[p + "ls2"] * y
        else:
            chosen.append(None)
        if taps is not None:
            taps.append(x.clone())
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T, chosen


def load(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name)
    return cfg, w
