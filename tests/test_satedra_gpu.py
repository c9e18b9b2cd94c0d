"""Satedra in the engine against the plain model of tests/plain/satedra_plain.py: every mechanism
alone, prompts against token-by-token decoding, prompts cut into portions, batches of unequal
requests, slots and pages that are used again, one key that the asking token's attention rests on
far back, at page borders, at the first places and just inside and just outside every window (of a
layer that keeps latents and of one that reads another's, narrower and wider than the keeper's), in
prompts and decoded, long decoding through recorded steps, and greedy generation through the entry
points.

The configurations are those of tests/satedra_tiny.py; the plain model computes a whole sequence
from scratch in double precision, so every schedule has one truth: the function of the sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import satedra_tiny as st

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def tokens_for(cfg, n, seed):
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


_MODELS, _TRUTH = {}, {}


def model_of(which, dtype, seed=0):
    key = (which, dtype, seed)
    if key not in _MODELS:
        cfg = st.CONFIGS[which]
        w = st.make_weights(cfg, seed)
        _MODELS[key] = (cfg, w, st.load(cfg, w, dtype))
    return _MODELS[key]


def truth_of(which, seed, tokens):
    key = (which, seed, tuple(tokens))
    if key not in _TRUTH:
        cfg = st.CONFIGS[which]
        _TRUTH[key] = st.Truth(cfg, st.make_weights(cfg, seed), tokens)
    return _TRUTH[key]


def new_session(model, max_tokens=4096, **kw):
    from picolm_amd.engine import Session
    return Session(model, max_tokens=max_tokens, **kw)


def run_whole(session, tokens):
    [slot] = session.begin(1)
    got = session.step([slot], [tokens], [list(range(len(tokens)))]).double().cpu().numpy()
    session.release([slot])
    return got


def test_the_models_tensors_are_the_designs():
    from picolm_amd.engine.builder import build_from_config_dict
    for cfg in st.CONFIGS.values():
        specs = {s.name: tuple(s.shape) for s in build_from_config_dict(cfg).tensor_specs() if not s.optional or s.name == "head"}
        assert specs == st.tensor_shapes(cfg)


# ------------------------------------------------------------------------------ each mechanism alone
def one_layer(mixer, mlp=None, **kw):
    return st.config(61, 48, [st.layer(mixer, mlp)], **kw)


_Y = st.yarn(4.0, 64, 8.0, 2.0)
_PLAIN_MIXER = st.mixer(2, 12, 8, 10, 14, 0.3, 50)
ALONE = {
    "latent attention": one_layer(st.mixer(3, 12, 8, 20, 28, 0.4, 200)),
    "a window of 5": one_layer(st.mixer(3, 12, 8, 20, 28, 0.4, 5)),
    "a window of one": one_layer(st.mixer(2, 12, 8, 20, 28, 0.4, 1)),
    "a window of a page": one_layer(st.mixer(2, 12, 8, 20, 28, 0.4, 64)),
    "no window": one_layer(st.mixer(2, 12, 8, 20, 28, 0.4, 0)),
    "scaled rotation": one_layer(st.mixer(3, 12, 16, 20, 28, 0.4, 40, 500.0, _Y)),                                  # a ramp from the first pair on
    "scaled rotation whose ramp starts later": one_layer(st.mixer(3, 12, 16, 20, 28, 0.4, 40, 500.0, st.yarn(4.0, 80, 1.0, 0.25))),
    "scaled rotation whose ramp is one pair wide": one_layer(st.mixer(2, 8, 12, 6, 10, 0.4, 40, 30.0, st.yarn(16.0, 40, 2.0, 1.9))),
    "a rotated part of two": one_layer(st.mixer(3, 14, 2, 6, 10, 0.4, 40, 2.0, st.yarn(2.0, 8, 4.0, 1.0))),
    # keys [latent | rotated part] and latents that the matrix-core attention takes in bfloat16
    "keys of 64 over latents of 32": one_layer(st.mixer(4, 24, 32, 16, 32, 0.3, 70)),
    "keys of 96, values of 64": one_layer(st.mixer(4, 24, 32, 40, 64, 0.3, 33, 1000.0, _Y)),
    "keys of 128, values of 96, forty heads": one_layer(st.mixer(40, 8, 32, 12, 96, 0.5, 65)),
    "keys of 128, values of 64": one_layer(st.mixer(2, 32, 64, 48, 64, 0.2, 100)),
    "keys of 320": one_layer(st.mixer(2, 16, 32, 24, 288, 0.25, 90)),          # beyond what a thread's registers hold of a key
    "one head, latents of 5": one_layer(st.mixer(1, 7, 4, 3, 5, 0.6, 9)),
    "a dense feed-forward": one_layer(_PLAIN_MIXER, st.dense(40)),
    "routed experts": one_layer(_PLAIN_MIXER, st.moe(6, 2, 24, identity=0, scale=1.0, shared=None)),
    "routed experts, identity picks": one_layer(_PLAIN_MIXER, st.moe(4, 2, 24, identity=3, scale=1.0, shared=None)),
    "routed experts, only identity picks beside one expert": one_layer(_PLAIN_MIXER, st.moe(1, 2, 24, identity=4, scale=2.0, shared=None)),
    "routed experts, a shared expert and a scale": one_layer(_PLAIN_MIXER, st.moe(5, 3, 16, identity=1, scale=2.5, shared=40)),
    "routed experts, one pick": one_layer(_PLAIN_MIXER, st.moe(5, 1, 36, identity=2, scale=0.5, shared=12)),
    "routed experts, every output picked": one_layer(_PLAIN_MIXER, st.moe(3, 5, 20, identity=2, scale=1.0, shared=12)),
    # in bfloat16 a prompt of 64 rows and more sorts its picks by expert for the matrix cores
    "routed experts, widths in multiples of 16": one_layer(_PLAIN_MIXER, st.moe(6, 2, 32, identity=2, scale=1.5, shared=48)),
    "routed experts, more experts than rows a tile": one_layer(_PLAIN_MIXER, st.moe(40, 3, 48, identity=5, scale=1.0, shared=None)),
    "routed experts, widths that are no multiples of 8": st.config(61, 45, [st.layer(st.mixer(1, 9, 6, 5, 7, 0.4, 30),
                                                                                     st.moe(4, 2, 13, identity=1, scale=1.0, shared=7))]),
    "eps and the logits' scale": one_layer(_PLAIN_MIXER, st.dense(24), eps=1e-2, logit_scale=7.0),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("what", list(ALONE))
def test_each_mechanism_alone(what, dtype):
    cfg = ALONE[what]
    w = st.make_weights(cfg, 11)
    tokens = tokens_for(cfg, 70, 3)            # past a page's end
    want = st.Truth(cfg, w, tokens)
    s = new_session(st.load(cfg, w, dtype), 256)
    assert st.near(run_whole(s, tokens), want, slice(None), dtype)
    # and the same decoded token by token
    [slot] = s.begin(1)
    for i, t in enumerate(tokens):
        got = s.step([slot], [[t]]).double().cpu().numpy()
        assert st.near(got, want, i, dtype), (what, "token", i)
    s.release([slot])


# ------------------------------------------------------------------------------ prompts, decoding, portions
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_prompt_decoding_and_portions(which, dtype):
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 150, 1)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 1024)
    assert st.near(run_whole(s, tokens), want, slice(None), dtype)
    # most of it at once, the rest one by one (past the page border at 128, and windows that pass over decoded tokens)
    [slot] = s.begin(1)
    got = s.step([slot], [tokens[:101]], [[0, 1, 2, 63, 64, 100]]).double().cpu().numpy()
    assert st.near(got, want, [0, 1, 2, 63, 64, 100], dtype)
    for i in range(101, 150):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert st.near(got, want, i, dtype), ("decoded", i)
    s.release([slot])
    # portions of several sizes, down to two tokens and one, every row wanted
    for sizes in ([2, 2, 3, 57, 1, 64, 21], [64, 64, 22], [1, 1, 2, 146], [149, 1], [36, 37, 38, 39]):
        assert sum(sizes) == 150
        [slot] = s.begin(1)
        at = 0
        for n in sizes:
            got = s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy()
            assert st.near(got, want, slice(at, at + n), dtype), (sizes, "portion at", at)
            at += n
        s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_equal_the_whole_prompt_beyond_rounding(dtype):
    """How a prompt is cut does not show in the logits: against each other, not only against the
    plain model, and much closer than the limit that bfloat16 needs there."""
    cfg, w, model = model_of("A", dtype)
    tokens = tokens_for(cfg, 131, 5)
    s = new_session(model, 1024)
    whole = run_whole(s, tokens)
    [slot] = s.begin(1)
    parts, at = [], 0
    for n in (2, 63, 2, 61, 3):
        parts.append(s.step([slot], [tokens[at:at + n]], [list(range(n))]).double().cpu().numpy())
        at += n
    s.release([slot])
    assert st.distance(np.concatenate(parts), whole) <= (1e-5 if dtype == "float32" else 0.03)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_a_long_prompt(which, dtype):
    """Several pages and several tiles of queries, windows that end inside earlier pages; whole, in
    two long portions, and beside short requests in a batch, then decoded on."""
    cfg, w, model = model_of(which, dtype)
    tokens = tokens_for(cfg, 405, 8)
    want = truth_of(which, 0, tokens)
    s = new_session(model, 2048)
    assert st.near(run_whole(s, tokens[:401]), want, slice(0, 401), dtype)
    [slot] = s.begin(1)
    rows = [0, 63, 64, 127, 128, 199]
    got = s.step([slot], [tokens[:200]], [rows]).double().cpu().numpy()
    assert st.near(got, want, rows, dtype)
    got = s.step([slot], [tokens[200:401]], [list(range(201))]).double().cpu().numpy()
    assert st.near(got, want, slice(200, 401), dtype)
    for i in range(401, 405):
        got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
        assert st.near(got, want, i, dtype), ("decoded", i)
    s.release([slot])
    others = [tokens_for(cfg, n, 30 + n) for n in (10, 257)]
    slots = s.begin(3)
    got = s.step(slots, [tokens[:400]] + others).double().cpu().numpy()
    assert st.near(got[0], want, 399, dtype)
    for i, q in enumerate(others):
        assert st.near(got[1 + i], truth_of(which, 0, q), len(q) - 1, dtype), ("beside the long one", i)
    got = s.step(slots[:1], [[tokens[400]]]).double().cpu().numpy()
    assert st.near(got, want, 400, dtype)
    s.release(slots)


# ------------------------------------------------------------------------------ batches
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "C"])
def test_a_batch_of_unequal_requests_equals_each_alone(which, dtype):
    cfg, w, model = model_of(which, dtype)
    lens, n_dec = [1, 2, 65, 37, 64, 130], 5
    seqs = [tokens_for(cfg, n + n_dec, 20 + i) for i, n in enumerate(lens)]
    truth = [truth_of(which, 0, q) for q in seqs]
    s = new_session(model, 2048)
    slots = s.begin(len(seqs))
    got = s.step(slots, [q[:n] for q, n in zip(seqs, lens)], [list(range(n)) for n in lens]).double().cpu().numpy()
    at = 0
    for i, n in enumerate(lens):
        assert st.near(got[at:at + n], truth[i], slice(0, n), dtype), ("prompt", i)
        at += n
    # and against each alone, much closer than the plain model is in bfloat16: what else is in the batch does not show
    alone = new_session(model, 512)
    at = 0
    for i, n in enumerate(lens):
        assert st.distance(got[at:at + n], run_whole(alone, seqs[i][:n])) <= (1e-5 if dtype == "float32" else 0.03), ("alone", i)
        at += n
    # the shorter ones end earlier: after two steps the first two leave the batch
    live = list(range(len(seqs)))
    for j in range(n_dec):
        if j == 2:
            s.release([slots[0], slots[1]])
            live = live[2:]
        got = s.step([slots[i] for i in live], [[seqs[i][lens[i] + j]] for i in live]).double().cpu().numpy()
        for row, i in enumerate(live):
            assert st.near(got[row], truth[i], lens[i] + j, dtype), ("step", j, "sequence", i)
    s.release([slots[i] for i in live])


@pytest.mark.parametrize("dtype", DTYPES)
def test_slots_and_pages_that_are_used_again(dtype):
    """A page's old latents are not seen: sequences run one after another through a session that
    has room for little more than one of them."""
    cfg, w, model = model_of("A", dtype)
    s = new_session(model, 256, n_slots=2)
    for k, n in enumerate([130, 5, 70, 130, 1, 64]):
        tokens = tokens_for(cfg, n, 40 + k)
        want = truth_of("A", 0, tokens)
        [slot] = s.begin(1)
        cut = max(1, n - 3)
        rows = [0, cut - 1]
        got = s.step([slot], [tokens[:cut]], [rows]).double().cpu().numpy()
        assert st.near(got, want, rows, dtype), ("prompt", k)
        for i in range(cut, n):
            got = s.step([slot], [[tokens[i]]]).double().cpu().numpy()
            assert st.near(got, want, i, dtype), ("sequence", k, "token", i)
        s.release([slot])
    # two sequences that swap slots between uses
    a, b = tokens_for(cfg, 40, 90), tokens_for(cfg, 66, 91)
    for order in ((a, b), (b, a)):
        slots = s.begin(2)
        got = s.step(slots, list(order)).double().cpu().numpy()
        for i, q in enumerate(order):
            assert st.near(got[i], truth_of("A", 0, q), len(q) - 1, dtype)
        s.release(slots)


# ------------------------------------------------------------------------------ far keys, page borders, windows' edges
def lookup_model(windows, asks=0, kv_rank=64, dim=64, vdim=16, heads=2, width=64):
    """Layers of latent attention of which layer `asks` looks a token's partner up, while the others
    add nothing (their output products are zero); layers after the first read the first one's
    latents, each through a window of its own (`windows`, 0: every key).

    All but the last eight entries of a latent read the first half of the width, the last eight
    (kept small, so that the others decide the latent's norm) the second half.  The unrotated
    queries of the asking layer are W_uk of a head times the same rows that make the latent, so the
    score of two tokens with the same first half is as high as a token's with itself; values read
    the last eight entries.  Token t + 700 has the first half of token t's embedding.  The rotated
    parts are small beside that.  So the asking token's output rests on its partner wherever the
    partner stands, if the window lets it be seen, and far above the chance products of hundreds of
    other keys, while the partner's value is its own."""
    keys, half = kv_rank - 8, width // 2
    rot_dim = 32 if kv_rank == 64 else 16      # keys of 96 over latents of 64 go through the matrix-core kernel in bfloat16
    layers = [st.layer(st.mixer(heads, dim, rot_dim, vdim, kv_rank, 30.0 / kv_rank, wd, 10000.0, st.yarn(4.0, 64, 8.0, 2.0),
                                kv_from=0 if i else None), None) for i, wd in enumerate(windows)]
    cfg = st.config(1400, width, layers)
    w = st.make_weights(cfg, 5)
    w["embed"] = (6.0 * w["embed"].double()).to(torch.bfloat16)
    w["embed"][700:, :half] = w["embed"][:700, :half]
    dkv = w["l0.mix.dkv"]
    dkv[:keys, half:] = 0
    dkv[keys:kv_rank, :half] = 0
    dkv[keys:kv_rank] = (0.25 * dkv[keys:kv_rank].double()).to(torch.bfloat16)
    dkv[kv_rank:] = (0.2 * dkv[kv_rank:].double()).to(torch.bfloat16)
    w["l0.mix.dkv.norm"] = torch.ones(kv_rank, dtype=torch.bfloat16)
    for i in range(len(windows)):
        p = f"l{i}.mix."
        w[f"l{i}.norm1"], w[f"l{i}.norm1.b"] = torch.ones(width, dtype=torch.bfloat16), torch.zeros(width, dtype=torch.bfloat16)
        if i != asks:
            w[p + "o"] = torch.zeros_like(w[p + "o"])
            continue
        uk = torch.randn(heads * dim, kv_rank, generator=torch.Generator().manual_seed(2), dtype=torch.float64) / dim ** 0.5
        uk[:, keys:] = 0
        w[p + "uk"] = uk.to(torch.bfloat16)
        q = w[p + "q"].double().view(heads, dim + rot_dim, width)
        q[:, :dim] = (w[p + "uk"].double() @ dkv[:kv_rank].double()).view(heads, dim, width)
        q[:, dim:] *= 0.2
        w[p + "q"] = q.reshape(heads * (dim + rot_dim), width).to(torch.bfloat16)
        w[p + "uv"][:, :keys] = 0
        w[p + "uv"] = (4.0 * w[p + "uv"].double()).to(torch.bfloat16)
        w[p + "g"] = torch.zeros_like(w[p + "g"])
        w[p + "o"] = (16.0 * w[p + "o"].double()).to(torch.bfloat16)          # the branch outweighs the rows it is added to
    return cfg, w


def distinct_tokens(n, needle_at, vocab, seed):
    """n unrelated tokens, except that the last one's partner stands at `needle_at`."""
    rng = np.random.default_rng(seed)
    tokens = [int(t) for t in rng.permutation(vocab // 2)[:n]]
    tokens[needle_at] = tokens[-1] + vocab // 2
    return tokens


def without_the_partner(tokens, needle_at, vocab):
    other = list(tokens)
    other[needle_at] = next(t for t in range(vocab // 2) if t not in tokens)
    return other


_FAR = {}


def asking_sequence(key, cfg, w, n, needle_at, seed, seen=True, asks=0):
    """n tokens whose last one's partner stands at `needle_at`, the plain model's logits of the last
    token, and a check that the test can tell: with the partner replaced by an unrelated token
    the logits differ by far more than rounding if the partner is seen (tokens are drawn again until
    they do), and not at all if a window hides it (while they would with a window one key wider)."""
    if key in _FAR:
        return _FAR[key]
    while True:
        tokens = distinct_tokens(n, needle_at, cfg["vocab"], seed)
        other = without_the_partner(tokens, needle_at, cfg["vocab"])
        want, missed = st.plain_logits(cfg, w, tokens)[-1], st.plain_logits(cfg, w, other)[-1]
        if not seen:
            assert st.distance(missed, want) < 1e-9, "the key must not count"
            wider = json.loads(json.dumps(cfg))
            wider["layers"][asks]["mixer"]["mask"]["size"] += 1
            counts = st.distance(st.plain_logits(wider, w, other)[-1], st.plain_logits(wider, w, tokens)[-1])
        else:
            counts = st.distance(missed, want) if needle_at != n - 1 else 1.0
        if counts > 0.2:
            _FAR[key] = (tokens, want)
            return _FAR[key]
        seed += 1000


def ask_in_a_prompt_and_decoded(s, tokens, want, dtype, what):
    [slot] = s.begin(1)
    got = s.step([slot], [tokens]).double().cpu().numpy()
    assert st.distance(got, want) <= st.LIMIT[dtype], ("prompt",) + what
    s.release([slot])
    [slot] = s.begin(1)
    s.step([slot], [tokens[:-1]], [[]])
    got = s.step([slot], [tokens[-1:]]).double().cpu().numpy()
    assert st.distance(got, want) <= st.LIMIT[dtype], ("decoded",) + what
    s.release([slot])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kv_rank", [40, 64])
def test_one_far_key_among_hundreds(kv_rank, dtype):
    """The asking token is the last; the key it asks for lies hundreds back, at the first places of
    the sequence, and just before and after page borders.  Both in a prompt and decoded.  (Latents
    of 64 with a rotated part of 32 go through the matrix-core kernel in bfloat16.)"""
    cfg, w = lookup_model([0], 0, kv_rank)
    s = new_session(st.load(cfg, w, dtype), 2048)
    n = 500
    for needle_at in (0, 1, 63, 64, 65, 128, 383, 498):
        tokens, want = asking_sequence((kv_rank, needle_at), cfg, w, n, needle_at, needle_at)
        ask_in_a_prompt_and_decoded(s, tokens, want, dtype, (needle_at,))


WINDOWS = [([70], 0, 64), ([64], 0, 64), ([129], 0, 64), ([2], 0, 64), ([1], 0, 64), ([33], 0, 64),
           ([100, 37], 1, 64), ([37, 100], 1, 64), ([37, 100], 0, 64), ([100, 37], 0, 64), ([90, 0, 65], 2, 64), ([0, 128], 1, 64),
           ([128, 0], 0, 64), ([70], 0, 40), ([100, 37], 1, 40), ([37, 100], 1, 40), ([37, 100], 0, 40)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("windows,asks,kv_rank", WINDOWS)
def test_a_key_just_inside_and_just_outside_a_window(windows, asks, kv_rank, dtype):
    """The partner of the last token stands at the last place its layer's window still shows and at
    the one before: seen, the logits rest on it; not seen, they are what they are without it.  The
    asking layer keeps latents of its own or reads the first layer's, through a window narrower or
    wider than the keeper's."""
    cfg, w = lookup_model(windows, asks, kv_rank)
    size = windows[asks]
    s = new_session(st.load(cfg, w, dtype), 1024)
    for n in (size + 3, 300):
        if n <= size:
            continue
        for back, seen in ((size - 1, True), (size, False)):
            tokens, want = asking_sequence((tuple(windows), asks, kv_rank, n, back), cfg, w, n, n - 1 - back, n + back, seen, asks)
            ask_in_a_prompt_and_decoded(s, tokens, want, dtype, (n, back))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("windows,asks,kv_rank", [([70], 0, 64), ([100, 37], 1, 64), ([37, 100], 1, 64), ([37, 100], 0, 40)])
def test_a_window_passes_over_decoded_tokens(windows, asks, kv_rank, dtype):
    """A short prompt that holds the partner, then single tokens until the asking one: the window's
    far edge lies among tokens of the prompt at first and has passed the partner in the end.  In a
    batch with a sequence that started elsewhere."""
    cfg, w = lookup_model(windows, asks, kv_rank)
    size = windows[asks]
    s = new_session(st.load(cfg, w, dtype), 1024)
    beside = distinct_tokens(400, 3, cfg["vocab"], 77)
    for back, seen in ((size - 1, True), (size, False)):
        n = 6 + back
        tokens, want = asking_sequence(("decoded", tuple(windows), asks, kv_rank, back), cfg, w, n, 5, back, seen, asks)
        slots = s.begin(2)
        s.step(slots, [tokens[:8], beside[:400 - (n - 8)]], [[], []])
        for i in range(8, n):
            got = s.step(slots, [[tokens[i]], [beside[400 - n + i]]]).double().cpu().numpy()
        assert st.distance(got[0], want) <= st.LIMIT[dtype], (back, seen)
        s.release(slots)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_sequence(dtype):
    """Sequences of one, two and three tokens, alone and in one batch; windows of one and two."""
    cfg, w, model = model_of("C", dtype)
    s = new_session(model, 512)
    seqs = [tokens_for(cfg, n, 60 + n) for n in (1, 2, 3, 1)]
    for q in seqs:
        assert st.near(run_whole(s, q), truth_of("C", 0, q), slice(None), dtype)
    slots = s.begin(len(seqs))
    got = s.step(slots, seqs).double().cpu().numpy()
    for i, q in enumerate(seqs):
        assert st.near(got[i], truth_of("C", 0, q), len(q) - 1, dtype)
    s.release(slots)


# ------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_long_decoding_through_recorded_steps(which, dtype):
    """Three sequences decoded 200 tokens, over page borders and past every window; from the second
    step of a shape on the engine replays its recording."""
    cfg, w, model = model_of(which, dtype)
    lens, n_dec = [3, 60, 120], 200
    seqs = [tokens_for(cfg, n + n_dec, 70 + i) for i, n in enumerate(lens)]
    truth = [truth_of(which, 0, q) for q in seqs]
    s = new_session(model, 2048)
    slots = s.begin(3)
    s.step(slots, [q[:n] for q, n in zip(seqs, lens)])
    for j in range(n_dec):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            assert st.near(got[i], truth[i], n + j, dtype), ("step", j, "sequence", i)
    assert s.recorded_steps() >= 1
    s.release(slots)


# ------------------------------------------------------------------------------ the entry points
@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    cfg = st.CONFIGS["A"]
    return st.write_folder(str(tmp_path_factory.mktemp("satedra") / "a"), cfg, st.make_weights(cfg, 0))


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(dtype, folder_a):
    import picolm_amd
    cfg = st.CONFIGS["A"]
    prompts = [tokens_for(cfg, n, 50 + n) for n in (4, 9, 66)]
    got = picolm_amd.generate(folder_a, prompts, max_new_tokens=10, stop_ids=(), dtype=dtype)
    for p, r in zip(prompts, got):
        assert len(r.tokens) == 10 and r.finish == "length"
        seq = list(p)
        for k in range(10):
            t = truth_of("A", 0, seq)
            lg = t.logits[-1]
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 4 * st.LIMIT[dtype] * lg.std() or t.margins[-st.AFTER - 1:].min() < st.CLOSE_CALL[dtype]:
                break                              # a near tie, or a router's close call: either choice is right
            assert r.tokens[k] == int(np.argmax(lg)), (k, r.tokens)
            seq.append(r.tokens[k])


def test_trace_replay_and_command_line(folder_a, tmp_path):
    """bin/trace_run on a folder: a prompt, single tokens and a second request that joins later in a
    slot that was given back; bin/picolm generates from the same folder."""
    cfg = st.CONFIGS["A"]
    a, b = tokens_for(cfg, 20, 1), tokens_for(cfg, 9, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:19], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[19:20], "want": [0]}], "end": ["a"]},
             {"step": 4, "entries": [{"id": "b", "tokens": b, "want": [8]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder_a, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ta, tb = truth_of("A", 0, a), truth_of("A", 0, b)
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])
    assert st.near(read(0), ta, [0, 16], "float32")
    assert st.near(read(1), ta, 17, "float32")
    assert not os.path.exists(os.path.join(out, "2.f32"))
    assert st.near(read(3), ta, 19, "float32")
    assert st.near(read(4), tb, 8, "float32")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "picolm"), folder_a, "-p", " ".join(map(str, b)), "-n", "4", "-t", "0",
                        "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert len(r.stdout.split()) == 4
    assert int(r.stdout.split()[0]) == int(np.argmax(tb.logits[-1]))


def test_trace_replay_counts_tokens_where_the_cache_counts_pages(folder_a, tmp_path):
    """--max-tokens is the sum of the live requests' tokens; each of them fills its last page only partly."""
    cfg = st.CONFIGS["A"]
    seqs = {f"r{i}": tokens_for(cfg, 3 + i, 80 + i) for i in range(6)}
    steps = [{"step": 0, "entries": [{"id": k, "tokens": q[:-1], "want": [len(q) - 2]} for k, q in seqs.items()], "end": []},
             {"step": 1, "entries": [{"id": k, "tokens": q[-1:], "want": [0]} for k, q in seqs.items()], "end": list(seqs)}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder_a, "--dtype", "float32", "--out", out,
                        "--max-tokens", str(sum(len(q) for q in seqs.values()))], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    got = [np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]) for i in (0, 1)]
    for row, q in enumerate(seqs.values()):
        t = truth_of("A", 0, q)
        assert st.near(got[0][row], t, len(q) - 2, "float32") and st.near(got[1][row], t, len(q) - 1, "float32")
