"""Kekelix without a GPU: the configuration's faults by key, the layer calls of a looped stretch and
their cache entries, and closed forms that pin the plain model of tests/plain/kekelix_plain.py
itself."""
import copy
import json
import math

import numpy as np
import pytest
import torch

import kekelix_tiny as kt
from picolm_amd.config import ConfigError, resolve
from picolm_amd.config.kekelix import KekelixConfig
from picolm_amd.engine.builder import build_from_config_dict
from plain import kekelix_plain as P


def test_the_registry_knows_the_name_and_the_configuration_round_trips():
    for cfg in kt.CONFIGS.values():
        assert resolve(cfg).name == "Kekelix"
        typed = KekelixConfig.from_dict(cfg)
        assert KekelixConfig.from_dict(typed.to_dict()) == typed
        assert KekelixConfig.from_dict(json.loads(json.dumps(typed.to_dict()))) == typed
        assert typed.vocab_size == cfg["vocab"] and typed.hidden_size == cfg["width"]


@pytest.mark.parametrize("path,value,names", [
    (("vocab",), None, "vocab"), (("width",), 0, "width"), (("norm", "eps"), 0.0, "norm.eps"),
    (("layers", 0, "type"), "attention_4", "layers[0].type"), (("layers", 0, "mixer", "heads"), None, "layers[0].mixer.heads"),
    (("layers", 0, "mixer", "kv_heads"), 4, "layers[0].mixer.kv_heads"), (("layers", 0, "mixer", "rot"), None, "layers[0].mixer.rot"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "layers[0].mixer.rot.dims"), (("layers", 0, "mixer", "rot", "dims"), 22, "layers[0].mixer.rot.dims"),
    (("layers", 0, "mixer", "rot", "base"), 0.0, "layers[0].mixer.rot.base"),
    (("layers", 0, "mixer", "rot", "scaling", "factor"), None, "layers[0].mixer.rot.scaling.factor"),
    (("layers", 0, "mixer", "rot", "scaling", "slow"), 0.0, "layers[0].mixer.rot.scaling.slow"),
    (("layers", 1, "mixer", "diff"), None, "layers[1].mixer.diff"), (("layers", 1, "mixer", "dim"), 600, "layers[1].mixer.dim"),
    (("layers", 1, "mixer", "scale"), 0.0, "layers[1].mixer.scale"), (("layers", 2, "mixer", "mask"), None, "layers[2].mixer.mask"),
    (("layers", 2, "mixer", "mask", "size"), 0, "layers[2].mixer.mask.size"),
    (("layers", 0, "mlp", "kind"), "dense", "layers[0].mlp.kind"), (("layers", 0, "mlp", "router", "top"), 9, "layers[0].mlp.router.top"),
    (("layers", 0, "mlp", "expert", "limit"), 0.0, "layers[0].mlp.expert.limit"), (("layers", 0, "mlp", "expert"), None, "layers[0].mlp.expert"),
    (("loop", "stop"), 9, "loop"), (("loop", "times"), 0, "loop.times"),
])
def test_a_fault_names_its_key(path, value, names):
    cfg = copy.deepcopy(kt.CONFIG_A)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        KekelixConfig.from_dict(cfg)
    assert names in str(e.value)


def test_every_pass_over_the_loop_has_cache_entries_of_its_own():
    model = build_from_config_dict(kt.CONFIG_A)
    # five layers, then one entry block per pass; layers 1 and 2 run three times in a row
    assert len(model.blocks) == 5 + 3
    assert [c.block for c in model.order] == [0, 5, 1, 2, 6, 1, 2, 7, 1, 2, 3, 4]
    kv = [b.kv for b in model.bindings]
    held = [x for x in kv if x is not None]
    assert len(held) == len(set(held)) == 9 and all(b.state is None for b in model.bindings)
    assert [x is None for x in kv] == [False, True, False, False, True, False, False, True, False, False, False, False]
    # the two maps' keys of a token lie side by side in one cached key; the values of a stretch layer are of the keys' size
    groups = {(g.n_kv_heads, g.head_dim, g.value_dim): g.n_entries for g in model.cache_spec.kv_groups}
    assert groups == {(2, 20, 12): 1, (2, 24, 20): 3, (1, 24, 24): 3, (2, 28, 28): 1, (3, 20, 14): 1}
    assert all(g.window == 0 for g in model.cache_spec.kv_groups)
    names = {s.name for s in model.tensor_specs() if not s.optional}
    assert names == set(kt.tensor_shapes(kt.CONFIG_A)) and "l2.norm2" not in names
    for cfg in kt.CONFIGS.values():
        specs = {s.name: tuple(s.shape) for s in build_from_config_dict(cfg).tensor_specs() if not s.optional}
        assert specs == kt.tensor_shapes(cfg)
    # without a loop, and with a loop of one pass, the embedding's rows are not kept
    assert not build_from_config_dict(kt.CONFIG_C).embedding.keeps_output and build_from_config_dict(kt.CONFIG_A).embedding.keeps_output
    once = copy.deepcopy(kt.CONFIG_A)
    once["loop"]["times"] = 1
    assert not build_from_config_dict(once).embedding.keeps_output


def test_the_plain_order_of_layer_runs():
    assert P.layer_runs(kt.CONFIG_A) == [(0, None, False), (1, 0, True), (2, 0, False), (1, 1, True), (2, 1, False), (1, 2, True),
                                         (2, 2, False), (3, None, False), (4, None, False)]
    assert P.layer_runs(kt.CONFIG_C) == [(i, None, False) for i in range(4)]
    assert KekelixConfig.from_dict(kt.CONFIG_A).layer_runs() == P.layer_runs(kt.CONFIG_A)
    assert KekelixConfig.from_dict(kt.CONFIG_B).layer_runs() == P.layer_runs(kt.CONFIG_B)


# ------------------------------------------------------------------------------ closed forms of the plain model
def test_the_plain_norm_has_eps_inside_the_root_and_a_weight_around_zero():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    w = np.array([0.0, 1.0, -0.5, 0.25])
    assert np.allclose(P.offset_norm(x, w, 0.5), x / math.sqrt(12.5 + 0.5) * np.array([1.0, 2.0, 0.5, 1.25]))
    assert np.allclose(P.unit_rms(x, 3.5), x / 4.0)


def test_the_plain_rotation_turns_the_first_entries_of_a_head_in_halves():
    rot = dict(base=100.0, dims=4)
    x = np.array([[[1.0, 2.0, 3.0, 4.0, 9.0]]])                       # one token, one head; the fifth entry is not turned
    out = P.rotate(x, rot, [3])[0, 0]
    a0, a1 = 3.0, 0.3
    assert np.allclose(out, [math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                             3 * math.cos(a0) + math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 9.0])
    assert np.allclose(P.rotate(x, rot, [0]), x)
    # scaled: base e, eight entries, original = 2 pi e: a pair that turns t times within `original` positions is pair
    # 4 (1 - ln t); fast = e^0.7 gives 1.2, slow = e^0.1 gives 3.6: ramps 0, 0, 1/3, 2/3
    rot = dict(base=math.e, dims=8, scaling=kt.yarn(5.0, 2 * math.pi * math.e, math.exp(0.7), math.exp(0.1)))
    got, mag = P.rotary_frequencies(rot)
    assert np.allclose(got, np.exp(-np.arange(4) / 4.0) * np.array([1.0, 1.0, 1 - 1 / 3 + 1 / 15, 1 - 2 / 3 + 2 / 15]), rtol=1e-12)
    assert math.isclose(mag, 1 + 0.1 * math.log(5.0))


def test_the_plain_softmax_with_and_without_one_more_in_its_denominator():
    q = np.array([[[1.0, 0.0]], [[1.0, 0.0]]])                        # two tokens, one head
    k = np.array([[[math.log(2.0), 0.0]], [[math.log(3.0), 0.0]]])
    v = np.array([[[1.0, 0.0]], [[0.0, 1.0]]])
    assert np.allclose(P.softmax_attention(q, k, v, 1.0)[1, 0], [2 / 5, 3 / 5])
    assert np.allclose(P.softmax_attention(q, k, v, 1.0, sink=True)[1, 0], [2 / 6, 3 / 6])
    assert np.allclose(P.softmax_attention(q, k, v, 1.0, sink=True)[0, 0], [2 / 3, 0.0])
    assert np.allclose(P.softmax_attention(q, k, v, 2.0)[1, 0], [4 / 13, 9 / 13])
    # very negative scores: the extra term takes almost everything, and nothing overflows
    assert np.allclose(P.softmax_attention(q, -1000 * k, v, 1.0, sink=True)[1, 0], [0.0, 0.0])
    # the first key a query sees
    assert np.allclose(P.softmax_attention(q, k, v, 1.0, first_key=lambda i: i)[1, 0], [0.0, 1.0])
    # grouped heads: query heads 0, 1 read KV head 0, heads 2, 3 read KV head 1
    q4 = np.ones((1, 4, 2))
    v2 = np.array([[[1.0, 2.0], [3.0, 4.0]]])
    assert np.allclose(P.softmax_attention(q4, np.ones((1, 2, 2)), v2, 1.0)[0], [[1, 2], [1, 2], [3, 4], [3, 4]])


def one_layer(mixer, mlp=None, width=16, **kw):
    return kt.config(50, width, [kt.layer(mixer, mlp)], **kw)


def test_the_plain_difference_of_two_maps():
    """One token: both maps give the value itself, so o = (1 - lam) v, normed to unit RMS and times
    (1 - diff)."""
    cfg = one_layer(kt.difference(2, 1, 4, 6, 0.5, 0.3))
    W = kt.as_arrays(kt.make_weights(cfg, 3))
    h = np.random.default_rng(0).normal(size=(1, 16))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    v = h @ W[p + "v"].T
    lam = math.exp(W[p + "lq1"] @ W[p + "lk1"]) - math.exp(W[p + "lq2"] @ W[p + "lk2"]) + 0.3
    o = (1 - lam) * v
    unit = o / np.sqrt((o * o).mean() + 1e-6) * 0.7
    assert np.allclose(P.difference_attention(h, W, p, m, 1e-6), np.concatenate([unit, unit], axis=1) @ W[p + "o"].T)
    # two tokens, written out for the second: map m of head a uses entries [m d, (m + 1) d) of the head's 2 d
    h = np.random.default_rng(1).normal(size=(2, 16))
    q = (h @ W[p + "q"].T).reshape(2, 2, 2, 4)
    k = (h @ W[p + "k"].T).reshape(2, 1, 2, 4)
    v = h @ W[p + "v"].T
    heads = []
    for a in range(2):
        maps = []
        for mm in range(2):
            s = np.array([q[1, a, mm] @ k[j, 0, mm] for j in range(2)]) * 0.5
            pr = np.exp(s) / np.exp(s).sum()
            maps.append(pr[0] * v[0] + pr[1] * v[1])
        o = maps[0] - lam * maps[1]
        heads.append(o / np.sqrt((o * o).mean() + 1e-6) * 0.7)
    assert np.allclose(P.difference_attention(h, W, p, m, 1e-6)[1], np.concatenate(heads) @ W[p + "o"].T)


def test_the_plain_attention_with_biases_turns_by_the_distance_alone_and_keeps_the_values_as_they_are():
    cfg = one_layer(kt.sinked(2, 1, 6, 4, 0.5, 4, 7.0, kt.yarn(3.0, 10, 2.0, 0.5)))
    W = kt.as_arrays(kt.make_weights(cfg, 4))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = np.random.default_rng(1).normal(size=(2, 16))
    f, mag = P.rotary_frequencies(m["rot"])
    q = (h[1] @ W[p + "q"].T + W[p + "q.b"]).reshape(2, 6)
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = h @ W[p + "v"].T + W[p + "v.b"]

    def turn(x, pos):
        out = np.array(x)
        for i in range(2):
            c, s = math.cos(pos * f[i]) * mag, math.sin(pos * f[i]) * mag
            out[i], out[i + 2] = x[i] * c - x[i + 2] * s, x[i + 2] * c + x[i] * s
        return out
    heads = []
    for a in range(2):
        s = np.array([turn(q[a], 1) @ turn(k[j], j) for j in range(2)]) * 0.5
        heads.append((math.exp(s[0]) * v[0] + math.exp(s[1]) * v[1]) / (1 + math.exp(s[0]) + math.exp(s[1])))
    assert np.allclose(P.sink_attention(h, W, p, m, 1e-6)[1], np.concatenate(heads) @ W[p + "o"].T)


def test_the_plain_stretches_start_at_multiples_of_their_size():
    cfg = one_layer(kt.chunked(2, 1, 6, 0.5, 4, 3, 20.0))
    w = kt.make_weights(cfg, 3)
    a = kt.plain_logits(cfg, w, [1, 2, 3, 4, 5, 6, 7, 8])
    b = kt.plain_logits(cfg, w, [1, 2, 9, 4, 5, 6, 7, 8])             # position 2 is the last of the first stretch
    assert np.allclose(a[3:], b[3:]) and not np.allclose(a[2], b[2], atol=1e-3)
    c = kt.plain_logits(cfg, w, [1, 2, 3, 9, 5, 6, 7, 8])             # position 3 opens the second: 4 and 5 see it, 6 does not
    assert not np.allclose(a[4], c[4], atol=1e-3) and not np.allclose(a[5], c[5], atol=1e-3) and np.allclose(a[6:], c[6:])
    # a stretch of one: a row depends on its token and nothing else, the position included (one key: the weight is one)
    cfg = one_layer(kt.chunked(2, 1, 6, 0.5, 4, 1, 20.0))
    w = kt.make_weights(cfg, 3)
    assert np.allclose(kt.plain_logits(cfg, w, [1, 2, 3, 4])[3], kt.plain_logits(cfg, w, [7, 4])[1])
    # one key: the value is the key as projected, without the norm (and the turn) that queries and keys get
    W = kt.as_arrays(w)
    h = np.random.default_rng(2).normal(size=(1, 16))
    k = h @ W["l0.mix.k"].T
    assert np.allclose(P.chunk_attention(h, W, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6), np.concatenate([k, k], axis=1) @ W["l0.mix.o"].T)


def expert_case(top, limit=10.0):
    """Three experts with router logits ln 1, ln 3, ln 1/3 for the input of ones (scores 1/2, 3/4, 1/4),
    gate rows that sum their input and up rows that give half of that; expert e's output is 10^e times
    its hidden unit in every entry."""
    D = 4
    W = {"router": np.log(np.array([1.0, 3.0, 1 / 3]))[:, None] * np.ones((3, D)) / D}
    for e in range(3):
        W.update({f"e{e}.gate": np.ones((1, D)), f"e{e}.up": 0.5 * np.ones((1, D)), f"e{e}.down": np.full((D, 1), 10.0 ** e)})
    return W, dict(router=dict(experts=3, top=top), expert=dict(ff=1, limit=limit))


def hidden_unit(g, u, limit):
    g, u = min(g, limit), max(-limit, min(u, limit))
    return g / (1 + math.exp(-1.702 * g)) * (u + 1)


def test_the_plain_router_weighs_an_experts_input_by_its_score():
    h = np.ones((1, 4))
    W, mlp = expert_case(1)
    assert np.allclose(P.router_scores(h, W, ""), [[0.5, 0.75, 0.25]])
    # expert 1 reads 3/4 h: g = 3, u = 1.5
    assert np.allclose(P.routed_experts(h, W, "", mlp), 10 * hidden_unit(3.0, 1.5, 10.0))
    assert np.allclose(P.router_margins(h, W, "", mlp), [0.25])
    W, mlp = expert_case(2)
    assert np.allclose(P.routed_experts(h, W, "", mlp), 10 * hidden_unit(3.0, 1.5, 10.0) + hidden_unit(2.0, 1.0, 10.0))
    # the scores are not shares of one: with every expert picked their inputs are still 1/2, 3/4 and 1/4 of h
    W, mlp = expert_case(3)
    assert np.allclose(P.routed_experts(h, W, "", mlp),
                       10 * hidden_unit(3.0, 1.5, 10.0) + hidden_unit(2.0, 1.0, 10.0) + 100 * hidden_unit(1.0, 0.5, 10.0))
    # the limit: the gate's product from above only, the other from both sides
    W, mlp = expert_case(1, limit=1.25)
    assert np.allclose(P.routed_experts(h, W, "", mlp), 10 * 1.25 / (1 + math.exp(-1.702 * 1.25)) * 2.25)
    # for -h the logits change sign: scores 1/2, 1/4, 3/4, so expert 2 is picked and reads -3/4 h: g = -3 stays, u = -1.5 becomes -1.25
    assert np.allclose(P.routed_experts(-h, W, "", mlp), 100 * -3.0 / (1 + math.exp(1.702 * 3.0)) * -0.25)


def test_the_passes_of_a_loop_add_the_embedding_again_and_a_vector_each():
    """A loop whose layers add nothing: x = x0, then + step[0], then + x0 + step[1], ..."""
    cfg = kt.config(40, 8, [kt.layer(kt.difference(1, 1, 2, 2, 0.5, 0.2), None)], loop=(0, 1, 3))
    w = kt.make_weights(cfg, 1)
    w["l0.mix.o"] = torch.zeros_like(w["l0.mix.o"])
    W = kt.as_arrays(w)
    _, layers = P.forward(cfg, W, [3, 7], return_layers=True)
    x0 = W["embed"][[3, 7]]
    assert np.allclose(layers[0], x0 + W["loop.step"][0])
    assert np.allclose(layers[1], 2 * x0 + W["loop.step"][0] + W["loop.step"][1])
    assert np.allclose(layers[2], 3 * x0 + W["loop.step"][:3].sum(axis=0))


def test_both_branches_of_a_layer_read_the_same_rows():
    cfg = one_layer(kt.sinked(2, 1, 6, 4, 0.5, 4), kt.moe(3, 2, 5, 0.9))
    W = kt.as_arrays(kt.make_weights(cfg, 2))
    tokens = [5, 9, 2]
    _, layers = P.forward(cfg, W, tokens, return_layers=True)
    x = W["embed"][tokens]
    mixed = P.sink_attention(P.offset_norm(x, W["l0.norm1"], 1e-6), W, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6)
    fed = P.routed_experts(P.offset_norm(x, W["l0.norm2"], 1e-6), W, "l0.mlp.", cfg["layers"][0]["mlp"])
    assert np.allclose(layers[0], x + mixed + fed)


def test_every_mechanism_shows_in_the_plain_model():
    """The tests of the engine would pass a model that ignored what they isolate, if the plain model did."""
    cfg = kt.CONFIGS["A"]
    w = kt.make_weights(cfg, 0)
    tokens = [int(t) for t in np.random.default_rng(3).integers(0, cfg["vocab"], size=80)]
    base = kt.plain_logits(cfg, w, tokens)
    for name in ("l0.norm1", "l0.norm2", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.v.b", "l1.mix.lq1", "l1.mix.lk2", "l1.mlp.router", "l1.mlp.e1.up",
                 "l2.mix.k", "l3.mlp.e0.gate", "l4.mix.lq2", "loop.step", "final.norm"):
        changed = dict(w)
        changed[name] = torch.zeros_like(w[name])
        assert kt.distance(kt.plain_logits(cfg, changed, tokens), base) > 0.003, name
    for path, value in ((("norm", "eps"), 0.3), (("layers", 0, "mixer", "scale"), 0.05), (("layers", 0, "mixer", "rot", "dims"), 4),
                        (("layers", 0, "mixer", "rot", "base"), 50.0), (("layers", 0, "mixer", "rot", "scaling", "factor"), 2.0),
                        (("layers", 0, "mixer", "rot", "scaling", "fast"), 4.0), (("layers", 1, "mixer", "diff"), 0.1),
                        (("layers", 1, "mixer", "scale"), 0.1), (("layers", 2, "mixer", "mask", "size"), 36),
                        (("layers", 2, "mixer", "rot", "dims"), 24), (("layers", 3, "mixer", "mask", "size"), 71),
                        (("layers", 0, "mlp", "router", "top"), 3), (("layers", 0, "mlp", "expert", "limit"), 0.4),
                        (("layers", 3, "mlp", "expert", "limit"), 1.2), (("loop", "times"), 2), (("loop", "start"), 2), (("loop", "stop"), 2)):
        other = copy.deepcopy(cfg)
        at = other
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        assert kt.distance(kt.plain_logits(other, w, tokens), base) > 1e-4, path
    no_scaling = copy.deepcopy(cfg)
    del no_scaling["layers"][0]["mixer"]["rot"]["scaling"]
    assert kt.distance(kt.plain_logits(no_scaling, w, tokens), base) > 1e-4
