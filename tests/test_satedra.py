"""Satedra without a GPU: the configuration's faults by key, the layer calls and the cache entries
they share, the rotation's tables against a case worked by hand, and closed forms that pin the
plain model of tests/plain/satedra_plain.py itself."""
import copy
import json
import math

import numpy as np
import pytest
import torch

import satedra_tiny as st
from picolm_amd.config import ConfigError, resolve
from picolm_amd.config.satedra import SatedraConfig
from picolm_amd.engine.builder import build_from_config_dict
from plain import satedra_plain as P


def test_the_registry_knows_the_name_and_the_configuration_round_trips():
    for cfg in st.CONFIGS.values():
        assert resolve(cfg).name == "Satedra"
        typed = SatedraConfig.from_dict(cfg)
        assert SatedraConfig.from_dict(typed.to_dict()) == typed
        assert SatedraConfig.from_dict(json.loads(json.dumps(typed.to_dict()))) == typed
        assert typed.vocab_size == cfg["vocab"] and typed.hidden_size == cfg["width"]


@pytest.mark.parametrize("path,value,names", [
    (("vocab",), None, "vocab"), (("width",), 0, "width"), (("norm", "eps"), 0.0, "norm.eps"),
    (("layers", 0, "type"), "conv", "layers[0].type"), (("layers", 0, "mixer", "heads"), None, "layers[0].mixer.heads"),
    (("layers", 0, "mixer", "rot_dim"), 11, "layers[0].mixer.rot"), (("layers", 2, "mixer", "rot", "dims"), 6, "layers[2].mixer.rot.dims"),
    (("layers", 2, "mixer", "kv_rank"), 2000, "layers[2].mixer.kv_rank"), (("layers", 3, "mixer", "scale"), None, "layers[3].mixer.scale"),
    (("layers", 3, "mixer", "scale"), 0.0, "layers[3].mixer.scale"), (("layers", 2, "mixer", "rot", "base"), 0.0, "layers[2].mixer.rot.base"),
    (("layers", 0, "mixer", "rot", "scaling", "factor"), None, "layers[0].mixer.rot.scaling.factor"),
    (("layers", 0, "mixer", "rot", "scaling", "slow"), 0.0, "layers[0].mixer.rot.scaling.slow"),
    (("layers", 0, "mlp", "kind"), "conv", "layers[0].mlp.kind"), (("layers", 0, "mlp", "ff"), None, "layers[0].mlp.ff"),
    (("layers", 1, "mlp", "router", "top"), 9, "layers[1].mlp.router.top"), (("layers", 1, "mlp", "shared"), 5, "layers[1].mlp.shared"),
    (("layers", 1, "mlp", "expert"), None, "layers[1].mlp.expert"),
    (("layers", 1, "mixer", "kv_from"), 1, "layers[1].mixer.kv_from"), (("layers", 1, "mixer", "kv_from"), 7, "layers[1].mixer.kv_from"),
    (("layers", 3, "mixer", "kv_from"), 1, "layers[3].mixer.kv_from"),        # layer 1 keeps no latents of its own
    (("layers", 4, "mixer", "kv_from"), 0, "layers[4].mixer.kv_from"),        # layer 0's latents are of another size
    (("layers", 1, "mixer", "rot", "base"), 300.0, "layers[1].mixer.kv_from"),        # and must turn as its reader's queries do
])
def test_a_fault_names_its_key(path, value, names):
    cfg = copy.deepcopy(st.CONFIG_A)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        SatedraConfig.from_dict(cfg)
    assert names in str(e.value)


def test_layers_that_read_latents_share_the_keepers_cache_entry():
    model = build_from_config_dict(st.CONFIG_A)
    assert len(model.blocks) == 5 and [c.block for c in model.order] == [0, 1, 2, 3, 4]
    assert [c.reads_cache_of for c in model.order] == [None, 0, None, 0, 2]
    b = model.bindings
    assert b[0].kv == b[1].kv == b[3].kv and b[2].kv == b[4].kv and b[0].kv != b[2].kv
    assert [x.writes for x in b] == [True, False, True, False, False]
    assert all(x.state is None for x in b)                    # nothing but keys and values is kept
    groups = {(g.head_dim, g.value_dim): g for g in model.cache_spec.kv_groups}
    # a key is [latent | rotated part], one head of them for all query heads; the value is the latent; the entry is laid out for the
    # widest window among the layers that use it (0: a layer sees every key) and keeps every key where it was written
    wide, small = groups[(40 + 12, 40)], groups[(24 + 8, 24)]
    assert (wide.n_entries, wide.n_kv_heads, wide.window, wide.keeps_all) == (1, 1, 70, True)
    assert (small.n_entries, small.n_kv_heads, small.window, small.keeps_all) == (1, 1, 0, True)
    # the tensors: a reader has no W_dkv and no norm of latents
    names = {s.name for s in model.tensor_specs() if not s.optional}
    assert "l0.mix.dkv" in names and "l0.mix.dkv.norm" in names and "l1.mix.dkv" not in names and "l1.mix.dkv.norm" not in names
    assert "l2.norm2" not in names and "l2.norm2.b" not in names          # a layer without a feed-forward
    assert names | {"head"} == set(st.tensor_shapes(st.CONFIG_A))          # (a model without a head of its own would use the embedding table)


def test_a_window_over_an_entry_laid_out_for_fewer_keys_is_refused():
    from picolm_amd.parts.latent_attention import RotatedLatentAttention
    from picolm_amd.parts.position import RotaryEmbedding
    with pytest.raises(ValueError):
        RotatedLatentAttention("l0.mix.", 16, 2, 4, 4, 4, 8, 0.5, 1e-6, RotaryEmbedding(4, 100.0, style="half"), window=9, cache_window=8)
    with pytest.raises(ValueError):
        RotatedLatentAttention("l0.mix.", 16, 2, 4, 4, 4, 8, 0.5, 1e-6, RotaryEmbedding(4, 100.0, style="half"), window=0, cache_window=8)


# ------------------------------------------------------------------------------ the rotation
def test_the_scaled_frequencies_of_a_case_worked_by_hand():
    """base e, eight entries, original = 2 pi e: a pair that turns t times within `original` positions
    is pair 4 (1 - ln t).  fast = e^0.7 gives 1.2, so the ramp starts at pair 1; slow = e^0.1 gives
    3.6, so it ends at pair 4: ramps 0, 0, 1/3, 2/3 for the four pairs."""
    rot = dict(base=math.e, dims=8, scaling=st.yarn(5.0, 2 * math.pi * math.e, math.exp(0.7), math.exp(0.1)))
    f = np.exp(-np.arange(4) / 4.0)
    want = f * np.array([1.0, 1.0, 1 - 1 / 3 + 1 / 15, 1 - 2 / 3 + 2 / 15])
    got, mag = P.rotary_frequencies(rot)
    assert np.allclose(got, want, rtol=1e-12) and math.isclose(mag, 1 + 0.1 * math.log(5.0))
    # the library's tables hold the same angles, cosines and sines times the same factor
    from picolm_amd.config.satedra import YarnScaling
    from picolm_amd.parts.base import Runtime
    from picolm_amd.parts.position import RotaryEmbedding
    part = RotaryEmbedding(8, math.e, YarnScaling.from_dict(rot["scaling"], ""), style="half")
    part.prepare(Runtime(torch.device("cpu"), torch.float32), 50)
    cos, sin, style = part.rotary_tables()
    pos = np.arange(50)[:, None]
    assert style == 1 and cos.shape == (50, 4)
    assert np.allclose(cos.numpy(), np.cos(pos * want) * mag, atol=2e-5) and np.allclose(sin.numpy(), np.sin(pos * want) * mag, atol=2e-5)
    # without scaling: the plain powers of the base, and no factor
    got, mag = P.rotary_frequencies(dict(base=100.0, dims=4, scaling=None))
    assert np.allclose(got, [1.0, 0.1]) and mag == 1.0


def test_the_ramp_of_a_degenerate_case():
    """Both ends fall on one pair: the ramp's width is the floor 0.001, so that pair keeps its
    frequency and every later one is divided."""
    rot = dict(base=math.e, dims=8, scaling=st.yarn(2.0, 2 * math.pi * math.e, math.exp(0.45), math.exp(0.55)))     # 2.2 and 1.8: lo = hi = 2
    got, _ = P.rotary_frequencies(rot)
    assert np.allclose(got, np.exp(-np.arange(4) / 4.0) * np.array([1.0, 1.0, 1.0, 0.5]))
    from picolm_amd.config.satedra import YarnScaling
    from picolm_amd.parts.position import rotary_inv_freq
    assert np.allclose(rotary_inv_freq(8, math.e, YarnScaling.from_dict(rot["scaling"], "")).numpy(), got)
    # ends beyond the pairs there are: the first pair at the earliest, the last entry's index at the latest
    rot = dict(base=math.e, dims=4, scaling=st.yarn(3.0, 2 * math.pi * math.e, math.exp(5.0), math.exp(-5.0)))      # -8 and 12: lo = 0, hi = 3
    got, _ = P.rotary_frequencies(rot)
    assert np.allclose(got, np.exp(-np.arange(2) / 2.0) * np.array([1.0, 1 - 1 / 3 + 1 / 9]))
    assert np.allclose(rotary_inv_freq(4, math.e, YarnScaling.from_dict(rot["scaling"], "")).numpy(), got)


def test_the_plain_rotation_pairs_an_entry_with_the_one_half_the_part_away():
    rot = dict(base=100.0, dims=4, scaling=None)
    x = np.array([[[1.0, 2.0, 3.0, 4.0, 9.0]]])                       # one token, one head; the fifth entry is not turned
    out = P.rotate(x, [3], rot)[0, 0]
    a0, a1 = 3.0, 0.3
    assert np.allclose(out, [math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                             3 * math.cos(a0) + math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 9.0])
    assert np.allclose(P.rotate(x, [0], rot), x)


# ------------------------------------------------------------------------------ closed forms of the plain model
def test_the_plain_norms():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    w, b = np.array([1.0, 2.0, 1.0, 0.5]), np.array([0.0, 1.0, 0.0, -1.0])
    dev = np.array([-2.0, -1.0, 0.0, 3.0])
    assert np.allclose(P.layer_norm(x, w, b, 0.5), dev / math.sqrt(3.5 + 0.5) * w + b)
    assert np.allclose(P.rms_norm(x, w, 0.5), x / math.sqrt(12.5 + 0.5) * w)


def tiny_attention(window, heads=2, T=9):
    cfg = st.config(50, 16, [st.layer(st.mixer(heads, 4, 2, 6, 8, 0.5, window), None)])
    return cfg, st.make_weights(cfg, 3)


def test_the_plain_window_shows_a_token_itself_and_the_ones_before_it_up_to_its_size():
    cfg, w = tiny_attention(3)
    a = st.plain_logits(cfg, w, [1, 2, 3, 4, 5, 6, 7])
    far = st.plain_logits(cfg, w, [1, 2, 3, 9, 5, 6, 7])            # three back from the last: outside
    edge = st.plain_logits(cfg, w, [1, 2, 3, 4, 9, 6, 7])           # two back: the last one inside
    later = st.plain_logits(cfg, w, [1, 2, 3, 4, 5, 6, 9])
    assert np.allclose(a[6], far[6]) and not np.allclose(a[5], far[5], atol=1e-3)
    assert not np.allclose(a[6], edge[6], atol=1e-3)
    assert np.allclose(a[:6], later[:6])
    # a window of one: a token sees itself alone, so a row depends on its token and its position only
    cfg, w = tiny_attention(1)
    assert np.allclose(st.plain_logits(cfg, w, [1, 2, 3, 4])[3], st.plain_logits(cfg, w, [7, 8, 9, 4])[3])


def test_the_plain_attention_with_one_key_is_the_gated_value():
    """The first token sees itself alone: out = W_o (sigmoid(W_g h) per head * W_uv c)."""
    cfg, w = tiny_attention(4)
    W = st.as_arrays(w)
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = np.random.default_rng(0).normal(size=(1, 16))
    low = h @ W[p + "dkv"].T
    c = low[:, :8] / np.sqrt((low[:, :8] ** 2).mean() + 1e-6) * W[p + "dkv.norm"]
    v = (c @ W[p + "uv"].T).reshape(2, 6) * (1 / (1 + np.exp(-(h @ W[p + "g"].T)))).reshape(2, 1)
    kv = P.latent_keys(h, W, p, m, 1e-6, [0])
    assert np.allclose(kv[0], c)
    assert np.allclose(P.latent_attention(h, W, p, m, 1e-6, kv, [0]), v.reshape(1, 12) @ W[p + "o"].T)


def test_the_plain_scores_use_the_scale_as_given_and_turn_by_the_distance_alone():
    """Two tokens: the weight of the first key for the second query, written out; moving both
    positions by the same number changes nothing."""
    cfg, w = tiny_attention(4, heads=1)
    W = st.as_arrays(w)
    m, p = dict(cfg["layers"][0]["mixer"]), "l0.mix."
    m["rot"] = dict(base=7.0, dims=2, scaling=st.yarn(3.0, 10, 2.0, 0.5))
    h = np.random.default_rng(1).normal(size=(2, 16))
    out = {}
    for at in (0, 11):
        pos = [at, at + 1]
        kv = P.latent_keys(h, W, p, m, 1e-6, pos)
        out[at] = P.latent_attention(h, W, p, m, 1e-6, kv, pos)
    assert np.allclose(out[0], out[11])
    f, mag = P.rotary_frequencies(m["rot"])
    q = h[1] @ W[p + "q"].T
    low = h @ W[p + "dkv"].T
    c = low[:, :8] / np.sqrt((low[:, :8] ** 2).mean(axis=1, keepdims=True) + 1e-6) * W[p + "dkv.norm"]
    k = c @ W[p + "uk"].T
    turn = lambda x, pos: np.array([x[0] * math.cos(pos * f[0]) - x[1] * math.sin(pos * f[0]),
                                    x[1] * math.cos(pos * f[0]) + x[0] * math.sin(pos * f[0])]) * mag
    s = np.array([q[:4] @ k[j] + turn(q[4:], 1) @ turn(low[j, 8:], j) for j in (0, 1)]) * m["scale"]
    pr = np.exp(s) / np.exp(s).sum()
    v = c @ W[p + "uv"].T
    want = ((pr[0] * v[0] + pr[1] * v[1]) / (1 + np.exp(-(h[1] @ W[p + "g"].T)))) @ W[p + "o"].T
    assert np.allclose(out[0][1], want)


def router_case(correction, top, identity=0, scale=1.0, shared=False):
    """Four router outputs with logits ln 1, ln 2, ln 3, ln 4 for the input of ones (scores 0.1 to
    0.4), experts whose outputs are 1, 10, 100, ... times a unit in every entry."""
    D, n = 3, 4
    W = {"router": np.log(np.arange(1.0, n + 1))[:, None] * np.ones((n, D)) / D, "correction": np.array(correction)}
    for e in range(n - identity):
        W.update({f"e{e}.gate": np.ones((1, D)), f"e{e}.up": np.ones((1, D)), f"e{e}.down": np.full((D, 1), 10.0 ** e)})
    mlp = dict(router=dict(experts=n - identity, top=top, identity=identity, scale=scale), expert=dict(ff=1), shared=None)
    if shared:
        mlp["shared"] = dict(ff=1)
        W.update({"shared.gate": np.ones((1, D)), "shared.up": np.ones((1, D)), "shared.down": np.full((D, 1), 0.5),
                  "shared.sg": np.full((1, D), math.log(3.0) / D)})
    return W, mlp, P.silu(3.0) * 3.0


def test_the_plain_router_weighs_by_the_scores_and_picks_by_the_corrected_ones():
    h = np.ones((1, 3))
    W, mlp, unit = router_case([0, 0, 0, 0], 2)
    assert np.allclose(P.router_scores(h, W, ""), [[0.1, 0.2, 0.3, 0.4]])
    assert np.allclose(P.routed_experts(h, W, "", mlp), unit * (3 / 7 * 100 + 4 / 7 * 1000))
    # a correction lifts the first expert over the others; its weight is still its own score's share
    W, mlp, unit = router_case([0.35, 0, 0, 0], 2)
    assert np.allclose(P.routed_experts(h, W, "", mlp), unit * (1 / 5 * 1 + 4 / 5 * 1000))
    W, mlp, unit = router_case([0.35, 0, 0, 0], 2, scale=2.5)
    assert np.allclose(P.routed_experts(h, W, "", mlp), 2.5 * unit * (1 / 5 * 1 + 4 / 5 * 1000))
    # one pick: its weight is one (times the scale), whatever its score
    W, mlp, unit = router_case([0, 0.5, 0, 0], 1, scale=3.0)
    assert np.allclose(P.routed_experts(h, W, "", mlp), 3.0 * unit * 10)
    assert np.allclose(P.router_margins(h, W, "", mlp), [0.7 - 0.4])


def test_the_plain_identity_picks_give_the_input_back_and_the_shared_expert_is_gated_per_token():
    h = np.ones((1, 3))
    # the last two router outputs are identity picks; they take part in the softmax and in the picks' sum
    W, mlp, unit = router_case([0, 0, 0, 0], 2, identity=2)
    assert np.allclose(P.routed_experts(h, W, "", mlp), (3 / 7 + 4 / 7) * h)
    W, mlp, unit = router_case([0, 0.25, 0, 0], 2, identity=2, scale=2.0)        # choice scores 0.1, 0.45, 0.3, 0.4
    assert np.allclose(P.routed_experts(h, W, "", mlp), 2.0 * (2 / 6 * unit * 10 + 4 / 6 * h))
    W, mlp, unit = router_case([0, 0, 0, 0], 1, identity=1, shared=True)
    assert np.allclose(P.routed_experts(h, W, "", mlp), h + 0.75 * unit * 0.5)           # sigmoid(ln 3) = 3/4
    # the shared expert's gate is a number per token
    two = np.stack([np.ones(3), 2 * np.ones(3)])
    out = P.routed_experts(two, W, "", mlp)
    gate2 = 1 / (1 + math.exp(-2 * math.log(3.0)))
    assert np.allclose(out[1] - two[1], gate2 * P.silu(6.0) * 6.0 * 0.5)


def test_every_mechanism_shows_in_the_plain_model():
    """The tests of the engine would pass a model that ignored what they isolate, if the plain model did."""
    cfg = st.CONFIGS["A"]
    w = st.make_weights(cfg, 0)
    tokens = [int(t) for t in np.random.default_rng(3).integers(0, cfg["vocab"], size=80)]
    base = st.plain_logits(cfg, w, tokens)
    for name in ("l0.norm1.b", "l0.mix.g", "l0.mix.dkv.norm", "l1.mix.uk", "l1.mix.uv", "l1.mlp.correction", "l1.mlp.shared.sg",
                 "l1.mlp.shared.down", "l1.mlp.e1.up", "l3.mlp.correction", "l4.mix.q", "l4.mlp.router", "final.norm.b"):
        changed = dict(w)
        changed[name] = torch.zeros_like(w[name])
        assert st.distance(st.plain_logits(cfg, changed, tokens), base) > 0.01, name
    for path, value in ((("logit_scale",), 1.0), (("norm", "eps"), 0.3), (("layers", 0, "mixer", "scale"), 0.05),
                        (("layers", 0, "mixer", "mask", "size"), 36), (("layers", 1, "mixer", "mask", "size"), 22),
                        (("layers", 3, "mixer", "mask", "size"), 69), (("layers", 4, "mixer", "mask", "size"), 10),
                        (("layers", 0, "mixer", "rot", "base"), 50.0), (("layers", 0, "mixer", "rot", "scaling"), None),
                        (("layers", 0, "mixer", "rot", "scaling", "factor"), 2.0), (("layers", 0, "mixer", "rot", "scaling", "fast"), 4.0),
                        (("layers", 1, "mlp", "router", "scale"), 1.0), (("layers", 1, "mlp", "router", "top"), 3)):
        other = copy.deepcopy(cfg)
        at = other
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        for l in other["layers"]:               # a layer that reads another's latents turns as that one does
            if l["mixer"].get("kv_from") == 0:
                l["mixer"]["rot"] = other["layers"][0]["mixer"]["rot"]
        assert st.distance(st.plain_logits(other, w, tokens), base) > 1e-4, path
    # a layer that reads another's latents has keys of its own if the configuration says so: another function
    own = copy.deepcopy(cfg)
    del own["layers"][1]["mixer"]["kv_from"]
    w2 = st.make_weights(own, 0)
    w2.update({k: v for k, v in w.items() if k in w2})
    assert st.distance(st.plain_logits(own, w2, tokens), base) > 0.01
