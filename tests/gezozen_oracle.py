"""Plain, slow float64 restatement of the Gezozen design, one function per mechanism, for the tests only.

Nothing here is shared with the product path: it reads the configuration dictionary itself, recomputes whole sequences from
their first token (no cache, no carried state: every recurrence simply runs over all tokens) and loops over heads and tokens.
Weights are dicts of float64 torch tensors under the checkpoint's names.

A layer normalises AFTER the sum, and its sublayers read the stream itself:
    x <- N1(a x + sigmoid(R1 x + r1) * mixer(x));   x <- N2(a x + sigmoid(R2 x + r2) * ff(x))
with one constant a for the model and N a root-mean-square norm taken separately over equal consecutive groups of the row.
Mixers: "parallel" (soft-capped causal attention beside gated linear attention), "parallel_2" (biased sliding-window attention
with stretched rotation frequencies beside retention), "delta" (short convolutions and the gated delta rule with one decay per
head).  Feed-forward: sigmoid-routed experts whose routing weight scales the expert's INPUT, plus a gated shared expert.
"""
import math

import torch

F = torch.float64


# ------------------------------------------------------------------------------------------------ small pieces
def silu(z):
    return z * torch.sigmoid(z)


def group_rms_norm(x, w, groups, eps):
    """x [..., n]: every one of `groups` equal consecutive parts divided by its own sqrt(mean(part^2) + eps); then times w."""
    shape = x.shape
    p = x.reshape(*shape[:-1], groups, shape[-1] // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(shape) * w


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def soft_cap(s, cap):
    return cap * torch.tanh(s / cap) if cap else s


def rotation_steps(rot):
    """(angle step per coordinate pair [dims / 2], multiplier of cos and sin) of a rotation entry {base, dims[, scaling]}.
    With `scaling` {factor, original, fast, slow} slow-turning pairs turn `factor` times slower, fast ones stay, and a linear
    ramp over the pair index joins them."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def turns_to_index(t):
        return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(turns_to_index(sc["fast"])), 0)
    hi = min(math.ceil(turns_to_index(sc["slow"])), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / sc["factor"] * ramp + f[i] * (1 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_halves(x, pos, rot):
    """x [heads, dim] of the token at position pos: coordinate i pairs with i + dims / 2 (i < dims / 2); the rest pass."""
    if not rot or not rot.get("dims"):
        return x
    steps, mul = rotation_steps(rot)
    half = rot["dims"] // 2
    y = x.clone()
    for i in range(half):
        a = pos * steps[i]
        c, s = math.cos(a) * mul, math.sin(a) * mul
        u, v = x[:, i], x[:, i + half]
        y[:, i] = u * c - v * s
        y[:, i + half] = v * c + u * s
    return y


def rotate_rows(x, rot):
    """x [T, heads, dim] of one sequence from position 0."""
    return torch.stack([rotate_halves(x[t], t, rot) for t in range(x.shape[0])])


# ------------------------------------------------------------------------------------------------ softmax attention
def softmax_attention(q, k, v, scale, cap=None, window=None):
    """q [T, H, D], k [T, G, D], v [T, G, V]: query head h reads key/value head h // (H / G); position i sees j <= i, and with a
    window only those with i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for i in range(T):
        j0 = 0 if not window else max(0, i - window + 1)
        for h in range(H):
            g = h // (H // G)
            s = soft_cap((k[j0:i + 1, g] @ q[i, h]) * scale, cap)
            out[i, h] = torch.softmax(s, 0) @ v[j0:i + 1, g]
    return out


def left_attention(h, w, pre, m, eps, biased):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def proj(name):
        y = h @ w[pre + name].T
        return y + w[pre + name + ".b"] if biased else y
    q, k, v = proj("q").reshape(T, H, D), proj("k").reshape(T, G, D), proj("v").reshape(T, G, V)
    q = rms_unit(q, eps) * w[pre + "q.norm"]
    k = rms_unit(k, eps) * w[pre + "k.norm"]
    q, k = rotate_rows(q, m.get("rot")), rotate_rows(k, m.get("rot"))
    o = softmax_attention(q, k, v, m["scale"], m.get("softcap"), (m.get("mask") or {}).get("size"))
    return o.reshape(T, H * V) @ w[pre + "o"].T


# ------------------------------------------------------------------------------------------------ linear recurrences
def decayed_outer_memory(q, k, v, decay):
    """Per head a matrix memory S [D, V] from zero:  S <- decay_t (rows) * S + k_t v_t^T;  o_t = S^T q_t.
    q, k [T, H, D], v [T, H, V], decay [T, H, D] (a number per key channel; broadcast one per head yourself)."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=F)
    out = []
    for t in range(T):
        S = decay[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def gated_linear_attention(h, w, pre, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, D)
    v = (h @ w[pre + "v"].T).reshape(T, H, V)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    decay = (torch.sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    o = decayed_outer_memory(q, k, v, decay)
    o = rms_unit(o, eps) * w[pre + "norm"]
    return (o.reshape(T, H * V) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def retention(h, w, pre, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = rotate_rows((h @ w[pre + "q"].T).reshape(T, H, D), m.get("rot"))
    k = rotate_rows((h @ w[pre + "k"].T).reshape(T, H, D), m.get("rot")) * D ** -0.5
    v = (h @ w[pre + "v"].T).reshape(T, H, V)
    decay = torch.tensor(m["decay"], dtype=F).reshape(1, H, 1).expand(T, H, D)
    o = rms_unit(decayed_outer_memory(q, k, v, decay), eps)
    return (o.reshape(T, H * V) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def short_conv(x, taps):
    """x [T, C], taps [C, n]: y[t, c] = sum_s taps[c, n - 1 - s] x[t - s, c] (the last column meets the current token)."""
    T, n = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for s in range(min(n, t + 1)):
            y[t] += taps[:, n - 1 - s] * x[t - s]
    return y


def delta_rule_memory(q, k, v, g, beta):
    """q, k [T, H, D], v [T, H, V], g, beta [T, H]:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=F)
    out = []
    for t in range(T):
        S = g[t].reshape(H, 1, 1) * S
        u = beta[t].reshape(H, 1) * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t].unsqueeze(-1) * u.unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def gated_delta(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def branch(name, heads, size):
        return silu(short_conv(h @ w[pre + name].T, w[pre + name + ".conv"])).reshape(T, heads, size)
    q, k, v = branch("q", G, D), branch("k", G, D), branch("v", H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    g = torch.exp(-torch.exp(w[pre + "A_log"]) * torch.nn.functional.softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    o = rms_unit(delta_rule_memory(q, k, v, g, beta), eps) * w[pre + "norm"]
    return (o.reshape(T, H * V) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def mixer(kind, h, w, pre, m, eps):
    if kind == "delta":
        return gated_delta(h, w, pre, m, eps)
    if kind == "parallel":
        return m["left_scale"] * left_attention(h, w, pre + "left.", m["left"], eps, False) + \
            m["right_scale"] * gated_linear_attention(h, w, pre + "right.", m["right"], eps)
    if kind == "parallel_2":
        return m["left_scale"] * left_attention(h, w, pre + "left.", m["left"], eps, True) + \
            m["right_scale"] * retention(h, w, pre + "right.", m["right"], eps)
    raise ValueError(kind)


# ------------------------------------------------------------------------------------------------ feed-forward
def glu_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(h, w, pre, top):
    """(expert ids [T, top], their sigmoid scores): the largest scores win, ties to the smaller index; no renormalisation."""
    s = torch.sigmoid(h @ w[pre + "router"].T)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(s, 1, order)


def router_margin(h, w, pre, top):
    """Smallest relative gap between the last chosen and the first rejected router logit over the rows of h (infinite when every
    expert is chosen): a gap near zero means that rounding may legitimately pick another expert."""
    z = torch.sort(h @ w[pre + "router"].T, -1, descending=True).values
    if top >= z.shape[1]:
        return math.inf
    return float(((z[:, top - 1] - z[:, top]) / z.abs().max(-1).values.clamp_min(1e-9)).min())


def feed_forward(h, w, pre, ff, margins=None):
    assert ff["kind"] == "moe"
    ids, score = route(h, w, pre, ff["router"]["top"])
    if margins is not None:
        margins.append(router_margin(h, w, pre, ff["router"]["top"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(ids[t].tolist(), score[t]):
            out[t] += glu_expert(s * h[t:t + 1], w, f"{pre}e{e}.")[0]      # the weight goes into the expert
    if ff.get("shared"):
        out = out + glu_expert(h, w, pre + "shared.") * torch.sigmoid(h @ w[pre + "shared.sg"].T)
    return out


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, w, tokens, margins=None):
    """tokens: list of ids of ONE sequence.  Returns (logits [T, vocab], residual stream after every layer [layers, T, width]).
    margins (a list): receives every routed layer's smallest router margin."""
    w = {k: v.to(F) for k, v in w.items()}
    eps, groups, a = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["postln_alpha"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    trace = []
    for i, e in enumerate(cfg["layers"]):
        pre = f"l{i}."
        y = mixer(e["type"], x, w, pre + "mix.", e["mixer"], eps) * torch.sigmoid(x @ w[pre + "rg1"].T + w[pre + "rg1.b"])
        x = group_rms_norm(a * x + y, w[pre + "norm1"], groups, eps)
        if e.get("mlp"):
            y = feed_forward(x, w, pre + "mlp.", e["mlp"], margins) * torch.sigmoid(x @ w[pre + "rg2"].T + w[pre + "rg2.b"])
            x = group_rms_norm(a * x + y, w[pre + "norm2"], groups, eps)
        trace.append(x)
    return group_rms_norm(x, w["final.norm"], groups, eps) @ w["head"].T, torch.stack(trace)
