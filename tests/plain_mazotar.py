"""A plain, slow implementation of the Mazotar decoder, written from its equations: one function per mechanism,
whole sequences at a time, float64 unless told otherwise.  It shares no code with the engine: it reads
config.json and model.safetensors itself (with the safetensors package), masks a full score matrix and walks the
recurrent layer token by token.

    x_0 = E[tok] * c + P(pos)                       P(p)[2i] = sin(p b^(-2i/D)),  P(p)[2i+1] = cos(p b^(-2i/D)),  b = 10000
    S streams X_1..X_S = x_0.  For every branch (mixer, then feed-forward) of every layer:
        u = sum_s a_s X_s;   y = branch(N(u; w));   X_t <- sum_s M[s, t] X_s + o_t y        N(v; w) = v / sqrt(mean(v^2) + eps) * w
    (no ``streams`` in the configuration: one stream, x <- x + branch(N(x; w)))
    logits = head N(sum_s X_s; w_f)
"""
import json
import math
import os

import torch
from safetensors import safe_open

SINUSOID_BASE = 10000.0
DENOMINATOR_FLOOR = 1e-6


# --------------------------------------------------------------------------------------------------- small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def weighted_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def sinusoid_rows(positions, width, dtype):
    """[T, width]: entry 2i is sin(p * base^(-2i/width)), entry 2i+1 the cosine of the same angle."""
    out = torch.zeros(len(positions), width, dtype=dtype)
    for i in range((width + 1) // 2):
        rate = SINUSOID_BASE ** (-2.0 * i / width)
        ang = torch.tensor([p * rate for p in positions], dtype=dtype)
        out[:, 2 * i] = torch.sin(ang)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = torch.cos(ang)
    return out


def distance_bucket(n, rows, far):
    """Which row of a distance table a key ``n`` places back uses: the first half of the rows one place each, the
    other half spread evenly over ln(distance) up to ``far``, where the last row begins."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def query_temperature(p, coef, every):
    return 1.0 + coef * math.log(math.floor((p + 1) / every) + 1.0)


def capped(z, cap):
    return cap * torch.tanh(z / cap)


# --------------------------------------------------------------------------------------------------- mixers
def attention_keys_values(h, w, prefix, m, eps):
    """What a layer with projections of its own keeps: keys after their norm over the whole projection, values."""
    k = weighted_norm(h @ w[prefix + "k"].T, w[prefix + "k.norm"], eps)
    v = h @ w[prefix + "v"].T
    return k, v


def biased_sink_attention(h, w, prefix, m, eps, positions, keys, values):
    """h [T, D]; keys [T, G*dim] (normed), values [T, G*vdim] of the layer that owns them."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = weighted_norm(h @ w[prefix + "q"].T, w[prefix + "q.norm"], eps)
    qt = m.get("q_temp")  # (absent: no temperature)
    temp = torch.tensor([1.0 if qt is None else query_temperature(p, qt["coef"], qt["every"]) for p in positions],
                        dtype=h.dtype)
    q = (q * temp[:, None]).view(T, H, dk)
    k, v = keys.view(T, G, dk), values.view(T, G, dv)
    rel = w[prefix + "rel"]
    B = rel.shape[0]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    pos = torch.tensor(positions)
    back = (pos[:, None] - pos[None, :]).clamp_min(0)  # [query, key]: how many places back the key lies
    row_of = torch.tensor([distance_bucket(n, B, m["bias_max"]) for n in range(int(back.max()) + 1)])
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"] + rel[row_of[back], head]
        s = s.masked_fill(~mask, -math.inf)
        sink = w[prefix + "sink"][head]
        top = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
        e = torch.exp(s - top)
        p = e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - top))
        out[:, head] = p @ v[:, g]
    return out.reshape(T, H * dv) @ w[prefix + "o"].T


def matrix_memory(h, w, prefix, m, eps, state=None):
    """The recurrent layer, token by token.  ``state``: (S [H, dk, dv], n [H, dk], m [H]) or None for a sequence's
    start; returns (output [T, D], state after the last token)."""
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[prefix + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[prefix + "k"].T).view(T, H, dk)
    v = (h @ w[prefix + "v"].T).view(T, H, dv)
    log_in = capped(h @ w[prefix + "i"].T + w[prefix + "i.b"], cap)
    log_keep = torch.nn.functional.logsigmoid(capped(h @ w[prefix + "f"].T + w[prefix + "f.b"], cap))
    if state is None:
        S = torch.zeros(H, dk, dv, dtype=h.dtype)
        n = torch.zeros(H, dk, dtype=h.dtype)
        top = torch.zeros(H, dtype=h.dtype)
    else:
        S, n, top = (t.clone() for t in state)
    outs = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        new_top = torch.maximum(log_keep[t] + top, log_in[t])
        keep = torch.exp(log_keep[t] + top - new_top)
        take = torch.exp(log_in[t] - new_top)
        S = keep[:, None, None] * S + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = keep[:, None] * n + take[:, None] * k[t]
        top = new_top
        num = torch.einsum("hkv,hk->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-top)) + DENOMINATOR_FLOOR
        outs[t] = num / den[:, None]
    o = unit_rms(outs, eps).reshape(T, H * dv) * w[prefix + "norm"]
    o = o * torch.sigmoid(h @ w[prefix + "g"].T)
    return o @ w[prefix + "o"].T, (S, n, top)


# --------------------------------------------------------------------------------------------------- feed-forwards
def gated_ff(h, w, prefix):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def routed_ff(h, w, prefix, mlp, choices=None):
    """``choices``: [T, top] expert numbers to use instead of the router's own (its scores stay the router's)."""
    scores = torch.sigmoid(h @ w[prefix + "router"].T)
    top = mlp["router"]["top"]
    chosen = torch.sort(scores, dim=-1, descending=True, stable=True).indices[:, :top] if choices is None else choices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += gated_ff((scores[t, e] * h[t])[None], w, f"{prefix}e{e}.")[0]
    if mlp.get("shared") is not None:
        out = out + gated_ff(h, w, prefix + "shared.") * torch.sigmoid(h @ w[prefix + "shared.sg"].T)
    return out, chosen


# --------------------------------------------------------------------------------------------------- the model
class PlainMazotar:
    def __init__(self, config, tensors, dtype=torch.float64):
        self.cfg, self.dtype = config, dtype
        self.w = {k: (v.to(dtype) if v.dtype.is_floating_point else v) for k, v in tensors.items()}

    @classmethod
    def from_dir(cls, path, dtype=torch.float64):
        with open(os.path.join(path, "config.json")) as f:
            config = json.load(f)
        tensors = {}
        with safe_open(os.path.join(path, "model.safetensors"), "pt") as f:
            for k in f.keys():
                tensors[k] = f.get_tensor(k)
        return cls(config, tensors, dtype)

    def embed(self, tokens, positions):
        c, D = self.cfg, self.cfg["width"]
        x = self.w["embed"][torch.tensor(tokens)] * float(c.get("embedding", {}).get("scale", 1.0))
        return x + sinusoid_rows(positions, D, self.dtype)

    def forward(self, tokens, choices=None, watch=None):
        """Logits [T, vocab] of one whole sequence.  ``choices``: {layer: [T, top]} experts to use; ``watch``: a
        list that gets the stream (the sum of the streams) behind every layer."""
        c, w, eps = self.cfg, self.w, float(self.cfg["norm"]["eps"])
        T = len(tokens)
        positions = list(range(T))
        x0 = self.embed(tokens, positions)
        S = c.get("streams")
        X = [x0.clone() for _ in range(S)] if S is not None else [x0.clone()]
        kept = {}
        self.chosen = {}
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            for which in (1, 2):
                if which == 2 and layer.get("mlp") is None:
                    continue
                u = sum(w[f"{p}hc{which}.in"][s] * X[s] for s in range(S)) if S is not None else X[0]
                h = weighted_norm(u, w[f"{p}norm{which}"], eps)
                if which == 1:
                    m = layer["mixer"]
                    if layer["type"] == "attention":
                        src = m.get("kv_from")
                        if src is None:
                            kept[i] = attention_keys_values(h, w, p + "mix.", m, eps)
                            src = i
                        y = biased_sink_attention(h, w, p + "mix.", m, eps, positions, *kept[src])
                    elif layer["type"] == "mlstm":
                        y, _ = matrix_memory(h, w, p + "mix.", m, eps)
                    else:
                        raise ValueError(layer["type"])
                else:
                    mlp = layer["mlp"]
                    if mlp["kind"] == "dense":
                        y = gated_ff(h, w, p + "mlp.")
                    else:
                        y, self.chosen[i] = routed_ff(h, w, p + "mlp.", mlp, None if choices is None else choices.get(i))
                if S is None:
                    X = [X[0] + y]
                else:
                    mix, out = w[f"{p}hc{which}.mix"], w[f"{p}hc{which}.out"]
                    X = [sum(mix[s, t] * X[s] for s in range(S)) + out[t] * y for t in range(S)]
            if watch is not None:
                watch.append(sum(X))
        return weighted_norm(sum(X), w["final.norm"], eps) @ w["head"].T
