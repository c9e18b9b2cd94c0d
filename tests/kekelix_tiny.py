"""Small Kekelix configurations with weights made for the tests, and the plain model's logits for
them.

The weights are not the library's random ones: every kind of tensor gets a spread that makes its
mechanism count (norm weights away from zero, projection biases of the size of the projections,
vectors of the maps' difference that give a constant away from its additive part, routers whose
scores lie between nought and one, experts' products that reach past the limit so that the clamps
bind, vectors of the passes as large as the rows), and all are rounded to bfloat16 first, so that
both runtimes and the plain model read the same numbers.  The configurations differ from each other
in every size, and none has two sizes equal that the code could mix up (key and value sizes, heads
and KV heads, the rotated part and the head, stretches and pages)."""
from __future__ import annotations

import numpy as np
import torch

from begopel_tiny import distance, load, write_folder  # noqa: F401  (the same helpers serve every design)


def yarn(factor, original, fast, slow):
    return dict(factor=factor, original=original, fast=fast, slow=slow)


def difference(heads, kv_heads, dim, vdim, scale, diff):
    return "attention", dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, diff=diff)


def sinked(heads, kv_heads, dim, vdim, scale, rot_dims, base=10000.0, scaling=None):
    rot = dict(base=base, dims=rot_dims)
    if scaling is not None:
        rot["scaling"] = scaling
    return "attention_2", dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot)


def chunked(heads, kv_heads, dim, scale, rot_dims, size, base=10000.0):
    return "attention_3", dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale, rot=dict(base=base, dims=rot_dims),
                               mask=dict(size=size))


def moe(experts, top, ff, limit):
    return dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff, limit=limit))


def layer(mixer, mlp=None):
    kind, m = mixer
    return dict(type=kind, mixer=m, mlp=mlp)


def config(vocab, width, layers, eps=1e-6, loop=None):
    cfg = dict(architecture="Kekelix", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if loop is not None:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return cfg


# A: every mixer, a layer without feed-forward, a loop over the two middle layers; stretches of 37 and 70
# positions (neither a divisor nor a multiple of a page)
CONFIG_A = config(211, 72, [
    layer(sinked(6, 2, 20, 12, 0.25, 8, 5000.0, yarn(4.0, 64, 1.0, 0.25)), moe(5, 2, 24, 0.8)),
    layer(difference(4, 2, 12, 20, 0.3, 0.35), moe(6, 1, 16, 1.5)),
    layer(chunked(3, 1, 24, 0.4, 16, 37, 300.0), None),
    layer(chunked(2, 2, 28, 0.35, 28, 70, 5000.0), moe(4, 3, 32, 0.6)),
    layer(difference(3, 3, 10, 14, 0.35, 0.6), moe(3, 3, 20, 1.0)),
], eps=1e-5, loop=(1, 3, 3))

# B: sizes of real layers' kind, which the matrix-core attention takes in bfloat16 (cached keys of 64,
# 96 and 128, values of 64, 96 and 128); experts in multiples of 16 so that a prompt's picks go through
# the matrix cores; a loop that starts at the first layer and runs twice
CONFIG_B = config(515, 256, [
    layer(difference(8, 2, 32, 96, 0.18, 0.2), moe(8, 2, 64, 1.2)),
    layer(chunked(4, 2, 96, 0.3, 32, 100, 100000.0), moe(16, 1, 32, 0.9)),
    layer(sinked(8, 4, 64, 128, 0.125, 64, 20000.0, yarn(8.0, 128, 16.0, 1.0)), moe(4, 4, 48, 2.0)),
    layer(difference(4, 4, 64, 64, 0.12, 0.5), None),
    layer(chunked(8, 1, 128, 0.25, 64, 129, 20000.0), moe(8, 3, 64, 1.0)),
], loop=(0, 2, 2))

# C: no size is a multiple of 8; one head; stretches of one and of two positions; one expert; no loop;
# a rotation without scaling in the layer with biases
CONFIG_C = config(77, 50, [
    layer(chunked(1, 1, 6, 0.5, 2, 1, 50.0), moe(1, 1, 13, 0.7)),
    layer(sinked(3, 1, 7, 5, 0.4, 6, 10.0), moe(7, 3, 6, 1.1)),
    layer(difference(5, 1, 3, 9, 0.5, 0.1), moe(2, 2, 9, 0.5)),
    layer(chunked(2, 1, 10, 0.45, 10, 2, 4.0), None),
], eps=1e-4)

CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a configuration's tensors, written out from the design's naming (the
    library's own list is held against this one)."""
    D = cfg["width"]
    out = {"embed": (cfg["vocab"], D), "final.norm": (D,)}
    if cfg.get("loop"):
        out["loop.step"] = (cfg["loop"]["times"], D)
    for i, l in enumerate(cfg["layers"]):
        p, q, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out[p + "norm1"] = (D,)
        if l["type"] == "attention":
            out.update({q + "q": (2 * H * d, D), q + "k": (2 * G * d, D), q + "v": (G * dv, D), q + "o": (D, H * dv)})
            out.update({q + n: (d,) for n in ("lq1", "lk1", "lq2", "lk2")})
        elif l["type"] == "attention_2":
            out.update({q + "q": (H * d, D), q + "k": (G * d, D), q + "v": (G * dv, D), q + "o": (D, H * dv),
                        q + "q.b": (H * d,), q + "k.b": (G * d,), q + "v.b": (G * dv,)})
        else:
            out.update({q + "q": (H * d, D), q + "k": (G * d, D), q + "o": (D, H * d)})
        mlp = l["mlp"]
        if not mlp:
            continue
        f = p + "mlp."
        out[p + "norm2"] = (D,)
        out[f + "router"] = (mlp["router"]["experts"], D)
        ff = mlp["expert"]["ff"]
        for e in range(mlp["router"]["experts"]):
            out.update({f"{f}e{e}.gate": (ff, D), f"{f}e{e}.up": (ff, D), f"{f}e{e}.down": (D, ff)})
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """bfloat16 tensors by name."""
    gen = torch.Generator().manual_seed(seed)
    randn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(*shape)
        elif name == "loop.step":
            t = 0.7 * randn(*shape)
        elif last in ("norm1", "norm2", "norm"):
            t = 0.25 * randn(*shape)                                  # offsets from one
        elif last == "b":
            t = 0.6 * randn(*shape)                                   # as large as the projections themselves
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.9 * randn(*shape) / shape[0] ** 0.25                # dot products of the size of one: the two exponentials differ
        elif last == "router":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5
        elif last in ("gate", "up"):
            t = 1.6 * randn(*shape) / shape[1] ** 0.5                 # hidden products that reach past the limit on either side
        elif last == "down":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5                 # feed-forwards that weigh as much as the mixers
        elif last in ("q", "k"):
            t = 1.5 * randn(*shape) / shape[1] ** 0.5
        else:
            t = randn(*shape) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def as_arrays(weights: dict) -> dict:
    return {k: v.to(torch.float64).numpy() for k, v in weights.items()}


def plain_logits(cfg: dict, weights: dict, tokens) -> np.ndarray:
    from plain import kekelix_plain as P
    return P.forward(cfg, as_arrays(weights), list(tokens))


class Truth:
    """The plain model's logits of a sequence, and per token the smallest margin by which any of
    its routers picked."""

    def __init__(self, cfg: dict, weights: dict, tokens):
        from plain import kekelix_plain as P
        margins = []
        self.logits = P.forward(cfg, as_arrays(weights), list(tokens), margins=margins)
        self.margins = np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf)

    def __getitem__(self, rows):
        return self.logits[rows]


def near(got, truth: Truth, rows, dtype: str) -> bool:
    """Whether the engine's rows lie within the limit of the plain model's.  A token whose router
    picked by less than CLOSE_CALL is held to LOOSE instead: rounding may give it another expert,
    and then its row is another function's value; the AFTER tokens behind such a token, which read
    it through later layers' keys, are held to BEHIND."""
    rows = np.arange(len(truth.logits))[rows]
    got, want = np.atleast_2d(np.asarray(got, np.float64)), np.atleast_2d(truth.logits[rows])
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    spread = np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean())
    e = np.sqrt((d ** 2).mean(-1)) / spread
    close = truth.margins < CLOSE_CALL[dtype]
    behind = np.array([close[max(0, r - AFTER):r].any() for r in np.atleast_1d(rows)])
    limit = np.where(close[np.atleast_1d(rows)], LOOSE, np.where(behind, BEHIND, LIMIT[dtype]))
    # most of many rows lie far inside the limit whatever a few routers did
    ok = bool((e <= limit).all()) and (len(e) < 16 or float(np.median(e)) <= LIMIT[dtype] / 3)
    if not ok:
        for r, err, lim in zip(np.atleast_1d(rows), e, limit):
            if err > lim:
                print(f"row {r}: {err:.4f} over {lim}, its routers' smallest margin {truth.margins[r]:.5f}")
        print(f"median {np.median(e):.4f}")
    return ok


# in 32-bit the engine's sums differ from the plain model's double precision by rounding alone; in
# bfloat16 every product's input is rounded to eight bits, and a router's scores that lie close
# together may then pick another expert for a token
LIMIT = {"float32": 2e-4, "bfloat16": 0.08}
# scores lie between nought and one; the rows that a deep layer's router reads carry a percent of rounding
CLOSE_CALL = {"float32": 1e-5, "bfloat16": 2e-2}
LOOSE, BEHIND, AFTER = 1.5, 0.35, 8
