"""The Kekelix decoder as a plain function of a whole sequence, in double precision: one function
per mechanism, no cache, no batching, no kernels.  What the engine computes is held against this.

Notation: h [T, D] rows of one sequence in order; W a dict of arrays by tensor name; weights are
stored [out, in] and applied as W x; positions count from 0.

    x0      = embed[token]
    pass t  : x = x + x0 (t > 0);  x = x + step[t]            before the first layer of a looped stretch's pass
    layer   : x = x + mixer(n1(x)) + ff(n2(x))               both branches read the same x; ff may be absent
    n(x)    = x / sqrt(mean(x^2) + eps) * (1 + w)
    logits  = embed n_final(x)
"""
from __future__ import annotations

import math

import numpy as np


def unit_rms(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotary_frequencies(rot):
    """Per pair i of `dims`/2 the angle a position advances by, and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = sc["factor"], sc["original"]

    def pair_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(pair_of(sc["fast"])), 0)
    hi = min(math.ceil(pair_of(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, rot, positions=None):
    """x [T, heads, n]: the first rot.dims entries of every head turn with the position, entry i
    paired with entry i + dims/2; the rest pass."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = rotary_frequencies(rot)
    out = np.array(x, np.float64)
    positions = range(x.shape[0]) if positions is None else positions
    for t, p in enumerate(positions):
        a = p * f
        c, s = np.cos(a) * mag, np.sin(a) * mag
        u, v = x[t, :, :half], x[t, :, half:dims]
        out[t, :, :half] = u * c - v * s
        out[t, :, half:dims] = v * c + u * s
    return out


def softmax_attention(q, k, v, scale, first_key=None, sink=False):
    """q [T, H, d], k [T, G, d], v [T, G, dv]: query i of head a over the keys first_key(i) .. i of
    KV head a // (H / G); `sink`: the denominator holds one more term, exp(0), that has no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        lo = 0 if first_key is None else first_key(i)
        for a in range(H):
            g = a // (H // G)
            s = k[lo:i + 1, g] @ q[i, a] * scale
            top = max(s.max(), 0.0) if sink else s.max()
            e = np.exp(s - top)
            out[i, a] = e @ v[lo:i + 1, g] / (e.sum() + (math.exp(-top) if sink else 0.0))
    return out


def difference_attention(h, W, p, m, eps):
    """Two softmax maps a head, over the same values, no positions:
    o = (a1 - lam a2), RMS-normed over the head's values without a weight, times (1 - diff)."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).reshape(T, H, 2, d)
    k = (h @ W[p + "k"].T).reshape(T, G, 2, d)
    v = (h @ W[p + "v"].T).reshape(T, G, dv)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, m["scale"])
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, m["scale"])
    lam = math.exp(float(W[p + "lq1"] @ W[p + "lk1"])) - math.exp(float(W[p + "lq2"] @ W[p + "lk2"])) + m["diff"]
    o = unit_rms(a1 - lam * a2, eps) * (1.0 - m["diff"])
    return o.reshape(T, H * dv) @ W[p + "o"].T


def sink_attention(h, W, p, m, eps):
    """Projections with biases, a rotation of part of every head, a softmax whose denominator has one more."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, dv)
    q, k = rotate(q, m["rot"]), rotate(k, m["rot"])
    return softmax_attention(q, k, v, m["scale"], sink=True).reshape(T, H * dv) @ W[p + "o"].T


def chunk_attention(h, W, p, m, eps):
    """The values are the keys as projected; queries and keys are turned, then made of unit RMS per
    head; a query sees the keys of its own chunk of mask.size positions up to itself."""
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    size = m["mask"]["size"]
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    k = (h @ W[p + "k"].T).reshape(T, G, d)
    v = k
    q, k = unit_rms(rotate(q, m["rot"]), eps), unit_rms(rotate(k, m["rot"]), eps)
    return softmax_attention(q, k, v, m["scale"], first_key=lambda i: i // size * size).reshape(T, H * d) @ W[p + "o"].T


MIXERS = {"attention": difference_attention, "attention_2": sink_attention, "attention_3": chunk_attention}


def clamped_expert(h, W, p, limit):
    g = np.minimum(h @ W[p + "gate"].T, limit)
    u = np.clip(h @ W[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def router_scores(h, W, p):
    return sigmoid(h @ W[p + "router"].T)


def routed_experts(h, W, p, mlp):
    """The `top` largest scores pick the experts; a pick's score multiplies what the expert reads."""
    top, limit = mlp["router"]["top"], mlp["expert"]["limit"]
    s = router_scores(h, W, p)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e in np.argsort(-s[t], kind="stable")[:top]:
            out[t] += clamped_expert(s[t, e] * h[t:t + 1], W, f"{p}e{e}.", limit)[0]
    return out


def router_margins(h, W, p, mlp):
    """Per row, how far the last pick's score lies above the first one not picked."""
    top = mlp["router"]["top"]
    s = router_scores(h, W, p)
    if top >= s.shape[1]:
        return np.full(h.shape[0], np.inf)
    z = -np.sort(-s, axis=1)
    return z[:, top - 1] - z[:, top]


def layer_runs(config):
    """(layer, pass number or None, first of its pass) in the order the layers run."""
    n = len(config["layers"])
    lp = config.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None, False) for i in range(lp["stop"], n)]


def forward(config: dict, W: dict, tokens, return_layers: bool = False, margins: list | None = None):
    """logits [T, vocab] of one sequence from its first token; with return_layers also the rows
    after every layer run; `margins` collects every routed layer run's margins per row."""
    W = {k: np.asarray(v, np.float64) for k, v in W.items()}
    eps = config["norm"]["eps"]
    x0 = W["embed"][np.asarray(tokens)]
    x = x0.copy()
    after = []
    for i, t, first in layer_runs(config):
        if first:
            if t > 0:
                x = x + x0
            x = x + W["loop.step"][t]
        entry = config["layers"][i]
        p = f"l{i}."
        branch = MIXERS[entry["type"]](offset_norm(x, W[p + "norm1"], eps), W, p + "mix.", entry["mixer"], eps)
        if entry.get("mlp"):
            h = offset_norm(x, W[p + "norm2"], eps)
            if margins is not None:
                margins.append(router_margins(h, W, p + "mlp.", entry["mlp"]))
            branch = branch + routed_experts(h, W, p + "mlp.", entry["mlp"])
        x = x + branch
        after.append(x)
    logits = offset_norm(x, W["final.norm"], eps) @ W["embed"].T
    return (logits, np.stack(after)) if return_layers else logits
