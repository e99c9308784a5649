"""Plain, slow float64 restatement of the Vokepel design, one function per mechanism, for the tests only.

Nothing here is shared with the product path: it reads the configuration dictionary itself, recomputes whole sequences from
their first token (no cache, no carried state: the recurrence simply runs over all tokens) and loops over heads and tokens.
Weights are dicts of float64 torch tensors under the checkpoint's names.

A layer is pre-norm and sequential:  x <- x + m * mixer(norm1(x));  x <- x + m * ff(norm2(x))  with one multiplier m for the
whole model.  A run of layers may repeat with the same weights; every repetition starts from  W_in [x; x0] + step[t]  with x0
the embedding output.  The logits come from the embedding table itself, scaled and soft-capped.
"""
import math

import torch

F = torch.float64


# ------------------------------------------------------------------------------------------------ small pieces
def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


def soft_cap(s, cap):
    return cap * torch.tanh(s / cap) if cap else s


def in_window(i, j, size):
    """May position i look at position j?  size 0 / None: every earlier position."""
    return 0 <= i - j and (not size or i - j < size)


def rotate_pairs(x, pos, dims, base):
    """x [heads, dim] of the token at position pos: coordinates (2i, 2i + 1), i < dims / 2, turn by pos * base^(-2i / dims)."""
    y = x.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, v = x[:, 2 * i], x[:, 2 * i + 1]
        y[:, 2 * i] = u * c - v * s
        y[:, 2 * i + 1] = v * c + u * s
    return y


def gru_candidate(u):
    """u + 1/2 on the non-negative side, sigmoid(u) on the negative one (continuous at 0)."""
    return torch.where(u >= 0, u + 0.5, torch.sigmoid(u))


# ------------------------------------------------------------------------------------------------ mixers
def windowed_attention(q, k, v, scale, size=None, cap=None, r1=None, r2=None, talk=None, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, V] of one sequence from its first token.  For every query position i, over the keys j
    it may see: score = q.k * scale; soft cap; minus r1[h] ln(1 + r2[h] (i - j)); the H scores of a key mixed by talk [H, H];
    softmax over the keys, the denominator also holding exp(sink[h]); weighted sum of the values.  Returns [T, H, V]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for i in range(T):
        js = [j for j in range(i + 1) if in_window(i, j, size)]
        dist = torch.tensor([float(i - j) for j in js], dtype=F)
        s = torch.zeros(H, len(js), dtype=F)
        for hh in range(H):
            g = hh // (H // G)
            s[hh] = soft_cap((k[js, g] @ q[i, hh]) * scale, cap)
            if r1 is not None:
                s[hh] = s[hh] - r1[hh] * torch.log1p(r2[hh] * dist)
        if talk is not None:
            s = talk @ s
        for hh in range(H):
            g = hh // (H // G)
            top = s[hh].max() if sink is None else torch.maximum(s[hh].max(), sink[hh])
            e = torch.exp(s[hh] - top)
            den = e.sum() + (0.0 if sink is None else torch.exp(sink[hh] - top))
            out[i, hh] = (e / den) @ v[js, g]
    return out


def biased_talking_attention(h, w, pre, m, eps):
    """Mixer `attention`: values are the un-normed keys, norms over the whole q / k rows, capped scores minus a logarithmic
    distance penalty per head, scores mixed across the heads before the softmax, element-wise output gate."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w[pre + "q"].T
    k = h @ w[pre + "k"].T
    v = k.reshape(T, G, D)
    q = rms_norm(q, w[pre + "q.norm"], eps).reshape(T, H, D)
    k = rms_norm(k, w[pre + "k.norm"], eps).reshape(T, G, D)
    out = windowed_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size"), m.get("softcap"), w[pre + "r1"], w[pre + "r2"],
                             w[pre + "talk"])
    return (out.reshape(T, H * D) * torch.sigmoid(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def rotary_sink_attention(h, w, pre, m):
    """Left half of mixer `parallel`: rotated q / k, sliding window, softmax whose denominator holds exp(sink) once per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D)
    k = (h @ w[pre + "k"].T).reshape(T, G, D)
    v = (h @ w[pre + "v"].T).reshape(T, G, V)
    rot = m.get("rot")
    if rot:
        q = torch.stack([rotate_pairs(q[t], t, rot["dims"], rot["base"]) for t in range(T)])
        k = torch.stack([rotate_pairs(k[t], t, rot["dims"], rot["base"]) for t in range(T)])
    out = windowed_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size"), sink=w[pre + "sink"])
    return out.reshape(T, H * V) @ w[pre + "o"].T


def min_gru_states(zl, u):
    """zl, u [T, R]: S_t = (1 - z_t) S_(t-1) + z_t c_t from S = 0, with z = sigmoid(zl) and c the candidate of u.  [T, R]."""
    z, c = torch.sigmoid(zl), gru_candidate(u)
    S = torch.zeros(zl.shape[1], dtype=F)
    rows = []
    for t in range(zl.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        rows.append(S)
    return torch.stack(rows)


def min_gru(h, w, pre):
    """Right half of mixer `parallel`: gates from the current token only, SiLU-gated read-out."""
    S = min_gru_states(h @ w[pre + "z"].T + w[pre + "z.b"], h @ w[pre + "x"].T + w[pre + "x.b"])
    return (S * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def mixer(kind, h, w, pre, m, eps):
    if kind == "attention":
        return biased_talking_attention(h, w, pre, m, eps)
    if kind == "parallel":
        return m["left_scale"] * rotary_sink_attention(h, w, pre + "left.", m["left"]) + m["right_scale"] * min_gru(h, w, pre + "right.")
    raise ValueError(kind)


def feed_forward(h, w, pre, ff):
    assert ff["kind"] == "dense"
    return relu_squared(h @ w[pre + "up"].T) @ w[pre + "down"].T


# ------------------------------------------------------------------------------------------------ the model
def layer_runs(cfg):
    """[(layer index, pass number or None)] in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens):
    """tokens: list of ids of ONE sequence.  Returns (logits [T, vocab], residual stream after every layer run [runs, T, width])."""
    w = {k: v.to(F) for k, v in w.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    loop = cfg.get("loop")
    trace = []
    for i, t in layer_runs(cfg):
        if t is not None and i == loop["start"]:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][t]
        e, pre = cfg["layers"][i], f"l{i}."
        x = x + mult * mixer(e["type"], rms_norm(x, w[pre + "norm1"], eps), w, pre + "mix.", e["mixer"], eps)
        if e.get("mlp"):
            x = x + mult * feed_forward(rms_norm(x, w[pre + "norm2"], eps), w, pre + "mlp.", e["mlp"])
        trace.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg["logit_scale"]
    return soft_cap(logits, cfg.get("logit_softcap")), torch.stack(trace)
