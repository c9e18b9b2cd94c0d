"""The Satedra decoder as a plain function of a whole sequence, in double precision: one function
per mechanism, no cache, no batching, no kernels.  What the engine computes is held against this.

Notation: h [T, D] rows of one sequence in order; W a dict of arrays by tensor name; weights are
stored [out, in] and applied as W x.

    x0     = embed[token]
    layer  : x = x + mixer(ln1(x));  x = x + ff(ln2(x))   (the second half only with a feed-forward)
    ln(x)  = (x - mean) / sqrt(var + eps) * w + b
    logits = head ln_final(x) * logit_scale
"""
from __future__ import annotations

import math

import numpy as np


def layer_norm(x, w, b, eps):
    x = np.asarray(x, np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotary_frequencies(rot):
    """Per pair i of `dims`/2 the angle a position advances by, and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = sc["factor"], sc["original"]

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot):
    """x [T, ..., n]: the first rot.dims entries of the last axis turn with the position, entry i
    paired with entry i + dims/2; the rest pass."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = rotary_frequencies(rot)
    out = np.array(x, np.float64)
    for t, p in enumerate(positions):
        a = p * f
        c, s = np.cos(a) * mag, np.sin(a) * mag
        u, v = x[t, ..., :half], x[t, ..., half:dims]
        out[t, ..., :half] = u * c - v * s
        out[t, ..., half:dims] = v * c + u * s
    return out


def latent_keys(h, W, p, m, eps, positions):
    """What a layer with a W_dkv of its own leaves for itself and for the layers that read it: the
    latent c [T, kv_rank] and the rotated key part [T, rot_dim]."""
    r = m["kv_rank"]
    low = h @ W[p + "dkv"].T
    c = rms_norm(low[:, :r], W[p + "dkv.norm"], eps)
    return c, rotate(low[:, r:], positions, m["rot"])


def latent_attention(h, W, p, m, eps, kv, positions=None):
    """m: {heads, dim, rot_dim, vdim, kv_rank, scale, mask: {size} (or none), rot}; kv = (c, k_rot) of this layer
    or of the one it reads."""
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    positions = range(T) if positions is None else positions
    c, k_rot = kv
    q = (h @ W[p + "q"].T).reshape(T, H, d + dr)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], positions, m["rot"])
    k = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, dv)
    window = (m.get("mask") or {}).get("size") or T           # no mask: every earlier key
    out = np.zeros((T, H, dv))
    for i in range(T):
        lo = max(0, i - window + 1)
        s = (np.einsum("hd,jhd->hj", q_plain[i], k[lo:i + 1]) + q_rot[i] @ k_rot[lo:i + 1].T) * m["scale"]
        s = np.exp(s - s.max(axis=1, keepdims=True))
        s /= s.sum(axis=1, keepdims=True)
        out[i] = np.einsum("hj,jhe->he", s, v[lo:i + 1])
    out = out * sigmoid(h @ W[p + "g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def gated_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def router_scores(h, W, p):
    z = h @ W[p + "router"].T
    s = np.exp(z - z.max(axis=1, keepdims=True))
    return s / s.sum(axis=1, keepdims=True)


def routed_experts(h, W, p, mlp):
    """Scores are a softmax over all router outputs; the picks are the largest of score +
    correction; the weights the picked scores over their sum, times a constant.  The last
    `identity` router outputs stand for experts that give their input back."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s = router_scores(h, W, p)
    choice = s + W[p + "correction"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = np.argsort(-choice[t], kind="stable")[:top]
        w = s[t, chosen] / (s[t, chosen].sum() + 1e-20) * r.get("scale", 1.0)
        for e, we in zip(chosen, w):
            out[t] += we * (gated_expert(h[t:t + 1], W, f"{p}e{e}.")[0] if e < E else h[t])
    if mlp.get("shared"):
        out += gated_expert(h, W, p + "shared.") * sigmoid(h @ W[p + "shared.sg"].T)
    return out


def router_margins(h, W, p, mlp):
    """Per row, how far the last pick's choice score lies above the first one not picked."""
    top = mlp["router"]["top"]
    choice = router_scores(h, W, p) + W[p + "correction"]
    if top >= choice.shape[1]:
        return np.full(h.shape[0], np.inf)
    z = -np.sort(-choice, axis=1)
    return z[:, top - 1] - z[:, top]


def feed_forward(h, W, p, mlp):
    return gated_expert(h, W, p) if mlp["kind"] == "dense" else routed_experts(h, W, p, mlp)


def forward(config: dict, W: dict, tokens, return_layers: bool = False, margins: list | None = None):
    """logits [T, vocab] of one sequence from its first token; with return_layers also the rows
    after every layer; `margins` collects every routed layer's margins per row."""
    W = {k: np.asarray(v, np.float64) for k, v in W.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    positions = range(len(tokens))
    after, kept = [], {}
    for i, entry in enumerate(config["layers"]):
        p = f"l{i}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        m = entry["mixer"]
        if m.get("kv_from") is None:
            kept[i] = latent_keys(h, W, p + "mix.", m, eps, positions)
        x = x + latent_attention(h, W, p + "mix.", m, eps, kept[i if m.get("kv_from") is None else m["kv_from"]], positions)
        if entry.get("mlp"):
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            if margins is not None and entry["mlp"]["kind"] == "moe":
                margins.append(router_margins(h, W, p + "mlp.", entry["mlp"]))
            x = x + feed_forward(h, W, p + "mlp.", entry["mlp"])
        after.append(x)
    logits = layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T * config.get("logit_scale", 1.0)
    return (logits, np.stack(after)) if return_layers else logits
