"""Small Satedra configurations with weights made for the tests, and the plain model's logits for
them.

The weights are not the library's random ones: every kind of tensor gets a spread that makes its
mechanism count (norm weights and biases away from their neutral values, corrections of the
router's scores that change which experts are picked, gates away from a half), and all are rounded
to bfloat16 first, so that both runtimes and the plain model read the same numbers.  The
configurations differ from each other in every size, and none has two sizes equal that the code
could mix up (unrotated, rotated and value sizes, latents, heads, the experts' and the shared
expert's widths); windows differ from layer to layer, also between a layer and the one whose
latents it reads."""
from __future__ import annotations

import numpy as np
import torch

from begopel_tiny import distance, load, write_folder  # noqa: F401  (the same helpers serve every design)


def yarn(factor, original, fast, slow):
    return dict(factor=factor, original=original, fast=fast, slow=slow)


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, window, base=10000.0, scaling=None, kv_from=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim, scaling=scaling))
    if window:
        m["mask"] = dict(size=window)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, identity=0, scale=1.0, shared=None):
    return dict(kind="moe", router=dict(experts=experts, top=top, identity=identity, scale=scale), expert=dict(ff=ff),
                shared=None if shared is None else dict(ff=shared))


def layer(m, mlp=None):
    return dict(type="latent_attention", mixer=m, mlp=mlp)


def config(vocab, width, layers, eps=1e-6, logit_scale=1.0):
    return dict(architecture="Satedra", vocab=vocab, width=width, norm=dict(eps=eps), logit_scale=logit_scale, layers=layers)


_YA = yarn(4.0, 64, 1.0, 0.25)          # the ramp runs from pair 1 to pair 3 of six
# A: a dense layer, routed layers with and without identity picks and shared expert, a layer without
# feed-forward, two layers that read the first one's latents (one with a narrower window, one with a
# wider one), a layer that sees every key
CONFIG_A = config(211, 72, [
    layer(mixer(3, 20, 12, 28, 40, 0.21, 37, 5000.0, _YA), dense(100)),
    layer(mixer(4, 12, 12, 20, 40, 0.3, 21, 5000.0, _YA, kv_from=0), moe(6, 2, 24, identity=2, scale=1.5, shared=36)),
    layer(mixer(2, 24, 8, 16, 24, 0.25, 0, 300.0, None), None),
    layer(mixer(3, 20, 12, 28, 40, 0.21, 70, 5000.0, _YA, kv_from=0), moe(5, 3, 32, identity=0, scale=1.0, shared=None)),
    layer(mixer(2, 24, 8, 16, 24, 0.25, 66, 300.0, None, kv_from=2), moe(4, 1, 16, identity=3, scale=0.7, shared=20)),
], eps=1e-5, logit_scale=1.7)

# B: sizes of real layers' kind; latents and rotated parts that the matrix-core attention takes in
# bfloat16 (keys of 96 and 128, values of 64); every router output picked in one layer
_YB = yarn(8.0, 128, 16.0, 1.0)
CONFIG_B = config(515, 256, [
    layer(mixer(8, 32, 32, 64, 64, 0.12, 100, 100000.0, _YB), moe(8, 3, 64, identity=2, scale=2.5, shared=128)),
    layer(mixer(4, 64, 32, 32, 64, 0.1, 64, 100000.0, _YB, kv_from=0), dense(512)),
    layer(mixer(8, 16, 64, 32, 64, 0.11, 130, 20000.0, None), moe(4, 6, 128, identity=2, scale=1.0, shared=64)),
    layer(mixer(2, 64, 64, 128, 64, 0.09, 129, 20000.0, None, kv_from=2), moe(8, 3, 64, identity=0, scale=0.5, shared=None)),
], logit_scale=0.5)

# C: no size is a multiple of 8; one head; a window of one and of two; one expert beside one identity pick
CONFIG_C = config(77, 50, [
    layer(mixer(1, 5, 6, 7, 9, 0.45, 2, 50.0, yarn(1.5, 20, 3.0, 0.5)), moe(1, 1, 13, identity=1, scale=3.0, shared=9)),
    layer(mixer(3, 7, 2, 5, 11, 0.4, 1, 10000.0, None), dense(21)),
    layer(mixer(5, 3, 6, 9, 9, 0.5, 33, 50.0, yarn(1.5, 20, 3.0, 0.5), kv_from=0), moe(7, 3, 6, identity=2, scale=1.0, shared=None)),
], eps=1e-4, logit_scale=3.0)

CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a configuration's tensors, written out from the design's naming (the
    library's own list is held against this one)."""
    D = cfg["width"]
    out = {"embed": (cfg["vocab"], D), "final.norm": (D,), "final.norm.b": (D,), "head": (cfg["vocab"], D)}
    for i, l in enumerate(cfg["layers"]):
        p, q, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        out.update({p + "norm1": (D,), p + "norm1.b": (D,), q + "q": (H * (d + dr), D), q + "uk": (H * d, r), q + "uv": (H * dv, r),
                    q + "g": (H, D), q + "o": (D, H * dv)})
        if m.get("kv_from") is None:
            out.update({q + "dkv": (r + dr, D), q + "dkv.norm": (r,)})
        mlp = l["mlp"]
        if not mlp:
            continue
        f = p + "mlp."
        out.update({p + "norm2": (D,), p + "norm2.b": (D,)})
        if mlp["kind"] == "dense":
            out.update({f + "gate": (mlp["ff"], D), f + "up": (mlp["ff"], D), f + "down": (D, mlp["ff"])})
            continue
        n_out = mlp["router"]["experts"] + mlp["router"]["identity"]
        out.update({f + "router": (n_out, D), f + "correction": (n_out,)})
        names = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
        if mlp.get("shared"):
            names.append(("shared.", mlp["shared"]["ff"]))
            out[f + "shared.sg"] = (1, D)
        for n, ff in names:
            out.update({f + n + "gate": (ff, D), f + n + "up": (ff, D), f + n + "down": (D, ff)})
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """bfloat16 tensors by name."""
    gen = torch.Generator().manual_seed(seed)
    randn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(*shape) + 0.3                                   # a mean that the layer norm has to take off
        elif last in ("norm1", "norm2", "norm"):
            t = 1.0 + 0.2 * randn(*shape)
        elif name.endswith(("norm1.b", "norm2.b", "final.norm.b")):
            t = 0.3 * randn(*shape)
        elif last == "correction":
            t = 0.15 * randn(*shape)                                  # of the size of the scores' differences: it changes the picks
        elif last == "router":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5
        elif last == "sg":
            t = 3.0 * randn(*shape) / shape[1] ** 0.5
        elif last == "g":
            t = 3.0 * randn(*shape) / shape[1] ** 0.5                 # gates from near zero to near one
        elif last == "down":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5                 # feed-forwards that weigh as much as the mixers
        elif last in ("q", "dkv"):
            t = 1.5 * randn(*shape) / shape[1] ** 0.5
        else:
            t = randn(*shape) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def as_arrays(weights: dict) -> dict:
    return {k: v.to(torch.float64).numpy() for k, v in weights.items()}


def plain_logits(cfg: dict, weights: dict, tokens) -> np.ndarray:
    from plain import satedra_plain as P
    return P.forward(cfg, as_arrays(weights), list(tokens))


class Truth:
    """The plain model's logits of a sequence, and per token the smallest margin by which any of
    its routers picked."""

    def __init__(self, cfg: dict, weights: dict, tokens):
        from plain import satedra_plain as P
        margins = []
        self.logits = P.forward(cfg, as_arrays(weights), list(tokens), margins=margins)
        self.margins = np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf)

    def __getitem__(self, rows):
        return self.logits[rows]


def near(got, truth: Truth, rows, dtype: str) -> bool:
    """Whether the engine's rows lie within the limit of the plain model's.  A token whose router
    picked by less than CLOSE_CALL is held to LOOSE instead: rounding may give it another expert,
    and then its row is another function's value.  (Later tokens read earlier ones through the
    cached latents, which are written before the feed-forward of their layer, but a later layer's
    latents do carry the change on, thinned by the other keys of a window: the AFTER tokens behind
    such a token are held to BEHIND.)"""
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
    ok = bool((e <= limit).all()) and (len(e) < 16 or float(np.median(e)) <= LIMIT[dtype] / 4)
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
# scores are shares of one among a handful of outputs; the rows that a deep layer's router reads carry a percent of rounding
CLOSE_CALL = {"float32": 1e-5, "bfloat16": 2e-2}
LOOSE, BEHIND, AFTER = 1.5, 0.35, 8
