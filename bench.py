#!/usr/bin/env python3
"""Decode and prefill throughput of a Llama shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape llama31-8b|llama2-7b|llama31-70b|llama32-1b|heads96]
                    [--batch B] [--layers L]

The default run is the Llama-3.1-8B shape at batch 8 and a context of up to 4,096; the other
shapes are the other workloads the library is measured on (Llama-2-7B: batch 16, prompts of 64 to
1,024 tokens, 256 greedy steps; Llama-3.1-70B: 80 layers with 141 GB of weights made on the GPU,
decode at batch 8 and 1; Llama-3.2-1B: head size 64 and a tied head, batch 8, 1 and 64).  A step is one decode step of the generation loop's inner body: the model
step over the batch from the cache, the sampler, and the hand-over of the sampled tokens.  Weights
are random bf16 made on the GPU, prompts are seeded uniform-random token ids; they go through the
model as the generation loop sends them (one step, or the steps of its token budget).  Prints one
JSON line: tokens a second, the step's fraction of HBM's peak, a prefill of 2,048 tokens, further
batch sizes (each right after its prompts, and with every sequence near 2,000 tokens and near the
full context), whole generation loops (the library's own and the Python one), and for each class
of kernels (decode products, decode attention, prefill products, prefill attention) what it reaches against the nominal peak and against what a plain read or a
register-only MFMA loop reaches on the same GPU (picolm prints effective weight throughput of its
layers likewise, picolm/picolm.c:305-317; its harness discards a warm-up and takes medians,
picolm/bench.zsh:46, :272).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
LLAMA3_SCALING = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192)

SHAPES = {
    "llama31-8b": dict(
        name="Llama-3.1-8B shape", std=0.02, batch=8, steps=64, warmup=8, prompt_range=(128, 2048), points=(1, 64),
        config=dict(architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                    num_key_value_heads=8, num_hidden_layers=32, vocab_size=128256, head_dim=128, rms_norm_eps=1e-5,
                    rope_theta=500000.0, rope_scaling=LLAMA3_SCALING, tie_word_embeddings=False,
                    max_position_embeddings=131072, eos_token_id=128001, bos_token_id=128000)),
    "llama2-7b": dict(
        name="Llama-2-7B shape", std=0.02, batch=16, steps=256, warmup=4, prompt_range=(64, 1024), points=(),
        config=dict(architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=11008, num_attention_heads=32,
                    num_key_value_heads=32, num_hidden_layers=32, vocab_size=32000, head_dim=128, rms_norm_eps=1e-5,
                    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False, max_position_embeddings=4096,
                    eos_token_id=2, bos_token_id=1)),
    "llama32-1b": dict(
        name="Llama-3.2-1B shape", std=0.02, batch=8, steps=64, warmup=8, prompt_range=(128, 2048), points=(1, 64),
        config=dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=8192, num_attention_heads=32,
                    num_key_value_heads=8, num_hidden_layers=16, vocab_size=128256, head_dim=64, rms_norm_eps=1e-5,
                    rope_theta=500000.0, rope_scaling=dict(LLAMA3_SCALING, factor=32.0), tie_word_embeddings=True,
                    max_position_embeddings=131072, eos_token_id=128001, bos_token_id=128000)),
    # no checkpoint's shape: a head size that is no power of two (96), for the attention kernels at such sizes
    "heads96": dict(
        name="width 3072, heads of 96", std=0.02, batch=8, steps=64, warmup=8, prompt_range=(128, 2048), points=(1, 64),
        config=dict(architectures=["LlamaForCausalLM"], hidden_size=3072, intermediate_size=8192, num_attention_heads=32,
                    num_key_value_heads=8, num_hidden_layers=32, vocab_size=32064, head_dim=96, rms_norm_eps=1e-5,
                    rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False, max_position_embeddings=4096,
                    eos_token_id=2, bos_token_id=1)),
    "llama31-70b": dict(
        name="Llama-3.1-70B shape", std=0.01, batch=8, steps=16, warmup=3, prompt_range=(128, 2048), points=(1,),
        config=dict(architectures=["LlamaForCausalLM"], hidden_size=8192, intermediate_size=28672, num_attention_heads=64,
                    num_key_value_heads=8, num_hidden_layers=80, vocab_size=128256, head_dim=128, rms_norm_eps=1e-5,
                    rope_theta=500000.0, rope_scaling=LLAMA3_SCALING, tie_word_embeddings=False,
                    max_position_embeddings=131072, eos_token_id=128001, bos_token_id=128000)),
}
CONTEXT = 4096
PREFILL_TOKENS = 2048


def layer_weight_bytes(cfg, itemsize=2) -> int:
    D, F = cfg.hidden_size, cfg.intermediate_size
    return (D * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * D + 3 * D * F) * itemsize


def weight_bytes(cfg, itemsize=2) -> int:
    """What a decode step reads of the weights: every layer's matrices and the head once, the norms."""
    D, V, L = cfg.hidden_size, cfg.vocab_size, cfg.num_hidden_layers
    return L * layer_weight_bytes(cfg, itemsize) + V * D * itemsize + (L * 2 * D + D) * 4


def kv_bytes_per_token(cfg, itemsize=2) -> int:
    return 2 * cfg.num_hidden_layers * cfg.kv_size * itemsize


def product_flops(cfg, T: int) -> float:
    D, F = cfg.hidden_size, cfg.intermediate_size
    return cfg.num_hidden_layers * 2.0 * T * (D * (cfg.q_size + 2 * cfg.kv_size) + cfg.q_size * D + 3 * D * F)


def attention_flops(cfg, T: int) -> float:
    return cfg.num_hidden_layers * 4.0 * cfg.head_dim * cfg.num_attention_heads * (T * (T + 1) / 2)


def prefill_flops(cfg, T: int) -> float:
    return product_flops(cfg, T) + attention_flops(cfg, T) + 2.0 * cfg.hidden_size * cfg.vocab_size


def library_products(cfg, dev, prefill_rows: int) -> dict:
    """A layer's four products (qkv, o, gate and up, down) at decode and prefill row counts: this
    library's kernels with the epilogue each has in the model, and the vendor library's plain
    product of the same shape (torch.matmul), in microseconds.  Every measurement replays a
    recorded graph that walks copies of the weights in turn, more of them than the memory-side
    cache holds, so that neither the host's launches nor that cache decide it."""
    import torch

    from picolm_amd import kernels
    D, F = cfg.hidden_size, cfg.intermediate_size
    shapes = [("qkv", cfg.q_size + 2 * cfg.kv_size, D, kernels.EPI_STORE, torch.float32), ("o", D, cfg.q_size, kernels.EPI_ACCUMULATE, torch.float32),
              ("gate_up", 2 * F, D, kernels.EPI_SWIGLU, torch.bfloat16), ("down", D, F, kernels.EPI_ACCUMULATE, torch.float32)]

    def replayed(calls, reps=3):
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            for f in calls:
                f()
            stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                for f in calls:
                    f()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(reps):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end) / (reps * len(calls)) * 1e3

    out = {}
    for M in (1, 8, 64, prefill_rows):
        row = {}
        for name, N, K, epilogue, c_dtype in shapes:
            copies = max(3, int(1.5e9 // (N * K * 2)))
            a = torch.randn(M, K, device=dev).to(torch.bfloat16)
            ws = [(torch.randn(N, K, device=dev) * 0.02).to(torch.bfloat16) for _ in range(copies)]
            c = torch.zeros(M, N // 2 if epilogue == kernels.EPI_SWIGLU else N, device=dev, dtype=c_dtype)
            plain = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            row[name] = {"library_us": round(replayed([(lambda w=w: torch.matmul(a, w.t(), out=plain)) for w in ws]), 1),
                         "ours_us": round(replayed([(lambda w=w: kernels.gemm(a, w, c, epilogue)) for w in ws]), 1)}
            del ws
        row["layer"] = {k: round(sum(v[k] for v in row.values()), 1) for k in ("library_us", "ours_us")}
        out[f"rows_{M}"] = row
        print(f"[bench] {M} rows: the library's four products {row['layer']['library_us']} us, ours {row['layer']['ours_us']} us",
              file=sys.stderr, flush=True)
    return {"library_products": out, "model": "layer sizes of " + str(cfg.hidden_size) + " x " + str(cfg.intermediate_size)}


# ---- another design beside the closest Llama of equal size --------------------------------------------
def _begopel_pair(width: int, heads: int, kv_heads: int, ff: int, vocab: int, pairs: int, loop_times: int = 0):
    """A Begopel of `pairs` (parallel, mamba2) pairs of layers with heads of 128, and the Llama of the
    same width, heads, feed-forward width, vocabulary and number of layer runs."""
    att = dict(heads=heads, kv_heads=kv_heads, dim=128, vdim=128, scale=128 ** -0.5, bias_max=4096.0, bias_rows=64)
    delta = dict(heads=heads, kv_heads=max(heads // 2, 1), dim=128, vdim=128, conv=4)
    mamba = dict(heads=2 * width // 64, vdim=64, state=128, groups=max(heads // 4, 1), norm_groups=1, conv=4)
    mlp = dict(kind="dense", ff=ff)
    layers = []
    for _ in range(pairs):
        layers += [dict(type="parallel", mixer=dict(left=att, right=delta), mlp=mlp), dict(type="mamba2", mixer=mamba, mlp=mlp)]
    beg = dict(architecture="Begopel", vocab=vocab, width=width, embedding=dict(scale=1.0), norm=dict(eps=1e-6), layers=layers,
               logit_softcap=30.0)
    runs = 2 * pairs
    if loop_times:
        beg["loop"] = dict(start=0, stop=2, times=loop_times)
        runs += 2 * (loop_times - 1)
    llama = dict(architectures=["LlamaForCausalLM"], hidden_size=width, intermediate_size=ff, num_attention_heads=heads,
                 num_key_value_heads=kv_heads, num_hidden_layers=runs, vocab_size=vocab, head_dim=128, rms_norm_eps=1e-6,
                 rope_theta=500000.0, rope_scaling=None, tie_word_embeddings=True, max_position_embeddings=131072, eos_token_id=2)
    return beg, llama


def _begopel_rooflines(cfg: dict, T: int, n_seq: int, context: int) -> dict:
    """Per label of operation, the seconds that the work of one prefill step of T tokens and of one
    decode step of n_seq sequences at `context` would take at the peak that binds it: products and
    softmax attention in a prefill at the bf16 matrix peak, the walk of a matrix state at the 32-bit
    vector peak (its state is 32-bit and its recurrence is no product), everything in a decode step
    and every row-wise operation at HBM's peak over the bytes it must move."""
    runs = []
    loop = cfg.get("loop")
    for i, layer in enumerate(cfg["layers"]):
        runs += [layer] * (loop["times"] if loop and loop["start"] <= i < loop["stop"] else 1)
    mfma, valu, hbm = PEAK_TFLOPS["bf16"] * 1e12, PEAK_TFLOPS["fp32"] * 1e12, HBM_PEAK_GBS * 1e9
    pre = {"sink_attention": 0.0, "state_scan": 0.0}
    dec = {"sink_attention": 0.0, "state_scan": 0.0}
    for layer in runs:
        m = layer["mixer"]
        if layer["type"] == "parallel":
            l, r = m["left"], m["right"]
            pre["sink_attention"] += 2.0 * l["heads"] * (l["dim"] + l["vdim"]) * (T * (T + 1) / 2) / mfma
            dec["sink_attention"] += n_seq * context * l["kv_heads"] * (l["dim"] + l["vdim"]) * 2 / hbm
            pre["state_scan"] += 7.0 * T * r["heads"] * r["dim"] * r["vdim"] / valu
            dec["state_scan"] += n_seq * 2 * r["heads"] * r["dim"] * r["vdim"] * 4 / hbm
        else:
            pre["state_scan"] += 5.0 * T * m["heads"] * m["state"] * m["vdim"] / valu
            dec["state_scan"] += n_seq * 2 * m["heads"] * m["state"] * m["vdim"] * 4 / hbm
    return {"prefill": pre, "decode": dec}


def _zarinex_pair(width: int, heads: int, kv_rank: int, experts: int, top: int, vocab: int, runs: int):
    """A Zarinex of `runs` layers in the order (hgrn2, mamba1, latent attention, mamba1) with heads of
    128, a selective scan of twice the width with a state of 16, and `experts` experts as wide as the
    model of which a token uses `top` beside a shared one; and the Begopel of the same width, heads,
    vocabulary and number of layer runs whose dense feed-forward is as wide as the experts a token uses."""
    mlp = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=width), shared=dict(ff=width))
    kinds = [("hgrn2", dict(heads=heads, dim=128, vdim=128)),
             ("mamba1", dict(inner=2 * width, state=16, dt_rank=width // 16, conv=4)),
             ("latent_attention", dict(heads=heads, dim=128, vdim=128, kv_rank=kv_rank, q_rank=3 * kv_rank, scale=128 ** -0.5)),
             ("mamba1", dict(inner=2 * width, state=16, dt_rank=width // 16, conv=4))]
    if runs < 4:
        kinds = kinds[1:3]
    layers = [dict(type=t, mixer=m, mlp=mlp) for t, m in kinds[:runs]]
    zar = dict(architecture="Zarinex", vocab=vocab, width=width, norm=dict(eps=1e-6), postln_alpha=1.0, layers=layers)
    beg, _ = _begopel_pair(width, heads, max(heads // 4, 1), (top + 1) * width, vocab, runs // 2)
    return zar, beg


def _satedra_pair(width: int, heads: int, kv_rank: int, rot_dim: int, window: int, experts: int, top: int, vocab: int, runs: int):
    """A Satedra of `runs` layers with query heads of 128 (of which `rot_dim` entries turn), values of
    128 read out of latents of `kv_rank`, every second layer reading the latents of the one before it,
    windows of `window` keys in the layers that keep latents and of half as many in those that read
    them, `experts` experts as wide as the model of which a token uses `top` (two more router outputs
    give the input back) beside a shared one; and the Zarinex of as many latent-attention layers of the
    same width, heads, vocabulary, experts and a cached key as long (kv_rank + rot_dim)."""
    scaling = dict(factor=8.0, original=4096, fast=32.0, slow=1.0)
    mlp = dict(kind="moe", router=dict(experts=experts, top=top, identity=2, scale=1.0), expert=dict(ff=width), shared=dict(ff=width))
    layers = []
    for i in range(runs):
        m = dict(heads=heads, dim=128 - rot_dim, rot_dim=rot_dim, vdim=128, kv_rank=kv_rank, scale=128 ** -0.5,
                 mask=dict(size=window if i % 2 == 0 else max(window // 2, 1)), rot=dict(base=10000.0, dims=rot_dim, scaling=scaling))
        if i % 2:
            m["kv_from"] = i - 1
        layers.append(dict(type="latent_attention", mixer=m, mlp=mlp))
    sat = dict(architecture="Satedra", vocab=vocab, width=width, norm=dict(eps=1e-6), logit_scale=1.0, layers=layers)
    key = kv_rank + rot_dim
    zmlp = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=width), shared=dict(ff=width))
    zar = dict(architecture="Zarinex", vocab=vocab, width=width, norm=dict(eps=1e-6), postln_alpha=1.0,
               layers=[dict(type="latent_attention", mixer=dict(heads=heads, dim=128, vdim=128, kv_rank=key, q_rank=3 * key, scale=128 ** -0.5),
                            mlp=zmlp) for _ in range(runs)])
    return sat, zar


def _satedra_rooflines(cfg: dict, T: int, n_seq: int, context: int) -> dict:
    """As _zarinex_rooflines: the attention over the keys a window lets a query see, [latent | rotated
    part] as the key and the latent as the value, at the bf16 matrix peak; the picked experts' products
    at the bf16 matrix peak (every pick counted as a real expert); in a decode step a window's keys
    and values once per sequence and the weights of the experts that the step's tokens can pick at
    most, at HBM's peak."""
    mfma, hbm = PEAK_TFLOPS["bf16"] * 1e12, HBM_PEAK_GBS * 1e9
    names = ("sink_attention", "routed_experts")
    pre, dec = {k: 0.0 for k in names}, {k: 0.0 for k in names}
    D = cfg["width"]
    for layer in cfg["layers"]:
        m = layer["mixer"]
        window = (m.get("mask") or {}).get("size", 0) or T + context
        seen = sum(min(i + 1, window) for i in range(T))
        pre["sink_attention"] += 2.0 * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"]) * seen / mfma
        dec["sink_attention"] += n_seq * min(context, window) * (2 * m["kv_rank"] + m["rot_dim"]) * 2 / hbm
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "moe":
            E, top, F = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            pre["routed_experts"] += 2.0 * 3 * T * top * D * F / mfma
            dec["routed_experts"] += min(n_seq * top, E) * 3 * D * F * 2 / hbm
    return {"prefill": pre, "decode": dec}


def _kekelix_pair(width: int, heads: int, stretch: int, experts: int, top: int, vocab: int, runs: int):
    """A Kekelix of `runs` layer runs with heads of 128: a layer of two attention maps a head (keys of
    64 each, so a cached key of 128) that a loop runs twice, a layer whose values are its keys and whose
    queries see stretches of `stretch` positions, and from four runs on a layer with biases, half of
    every head turned (YaRN-scaled) and one more in the softmax's denominator; a KV head for four query
    heads; `experts` experts as wide as the model of which a token uses `top`.  And the Satedra of as
    many layer runs of the same width, heads, vocabulary, experts and a cached key as long, whose
    windows are `stretch` keys."""
    mlp = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=width, limit=7.0))
    G = max(heads // 4, 1)
    kinds = [dict(type="attention", mixer=dict(heads=heads, kv_heads=G, dim=64, vdim=128, scale=64 ** -0.5, diff=0.25), mlp=mlp),
             dict(type="attention_3", mixer=dict(heads=heads, kv_heads=G, dim=128, vdim=128, scale=128 ** -0.5,
                                                 rot=dict(base=500000.0, dims=64), mask=dict(size=stretch)), mlp=mlp),
             dict(type="attention_2", mixer=dict(heads=heads, kv_heads=G, dim=128, vdim=128, scale=128 ** -0.5,
                                                 rot=dict(base=10000.0, dims=64, scaling=dict(factor=8.0, original=4096, fast=32.0, slow=1.0))),
                  mlp=mlp)]
    layers = kinds[:runs - 1]
    kek = dict(architecture="Kekelix", vocab=vocab, width=width, norm=dict(eps=1e-6), layers=layers, loop=dict(start=0, stop=1, times=2))
    sat, _ = _satedra_pair(width, heads, 96, 32, stretch, experts, top, vocab, runs)
    return kek, sat


def _kekelix_rooflines(cfg: dict, T: int, n_seq: int, context: int) -> dict:
    """As _satedra_rooflines: the attention over the keys a query sees (both maps of a layer with two,
    each with keys of its own and the same values) and the picked experts' products at the bf16 matrix
    peak; in a decode step the keys and values that the new token sees once per sequence and the
    weights of the experts that the step's tokens can pick at most, at HBM's peak."""
    mfma, hbm = PEAK_TFLOPS["bf16"] * 1e12, HBM_PEAK_GBS * 1e9
    names = ("sink_attention", "routed_experts")
    pre, dec = {k: 0.0 for k in names}, {k: 0.0 for k in names}
    D, loop = cfg["width"], cfg.get("loop")
    for i, layer in enumerate(cfg["layers"]):
        times = loop["times"] if loop and loop["start"] <= i < loop["stop"] else 1
        m = layer["mixer"]
        maps = 2 if layer["type"] == "attention" else 1
        size = (m.get("mask") or {}).get("size", 0) or T + context + 1
        seen = sum(j % size + 1 for j in range(T))
        pre["sink_attention"] += times * 2.0 * m["heads"] * maps * (m["dim"] + m["vdim"]) * seen / mfma
        dec["sink_attention"] += times * n_seq * (context % size + 1) * m["kv_heads"] * (maps * m["dim"] + m["vdim"]) * 2 / hbm
        mlp = layer.get("mlp")
        if mlp:
            E, top, F = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            pre["routed_experts"] += times * 2.0 * 3 * T * top * D * F / mfma
            dec["routed_experts"] += times * min(n_seq * top, E) * 3 * D * F * 2 / hbm
    return {"prefill": pre, "decode": dec}


DESIGN_SIZES = {
    "kekelix": [("width 1024", (1024, 8, 1536, 8, 2, 32000, 4)), ("width 2048", (2048, 16, 1536, 8, 2, 32000, 4)),
                ("width 4096", (4096, 32, 1536, 16, 2, 128256, 3))],
    "begopel": [("width 1024", (1024, 8, 2, 4096, 32000, 2, 2)), ("width 2048", (2048, 16, 4, 8192, 32000, 2, 0)),
                ("width 4096", (4096, 32, 8, 14336, 128256, 1, 0))],
    "zarinex": [("width 1024", (1024, 8, 128, 8, 2, 32000, 4)), ("width 2048", (2048, 16, 128, 8, 2, 32000, 4)),
                ("width 4096", (4096, 32, 128, 16, 2, 128256, 2)), ("width 4096, latents of 512", (4096, 32, 512, 16, 2, 128256, 2))],
    "satedra": [("width 1024", (1024, 8, 96, 32, 1024, 8, 2, 32000, 4)), ("width 2048", (2048, 16, 96, 32, 1024, 8, 2, 32000, 4)),
                ("width 4096", (4096, 32, 96, 32, 4096, 16, 2, 128256, 2)),
                ("width 4096, latents of 512", (4096, 32, 512, 64, 4096, 16, 2, 128256, 2))],
}


def _zarinex_rooflines(cfg: dict, T: int, n_seq: int, context: int) -> dict:
    """As _begopel_rooflines, for the operations of a Zarinex: the attention over latents (keys and
    values are both the latent) at the bf16 matrix peak, the walk of the states at the 32-bit vector
    peak (6 flops per state element and token with a decay per element, 5 with one per row), the
    picked experts' products at the bf16 matrix peak; in a decode step the latents twice (the cache
    keeps them in the keys' and in the values' layout), twice the states, and the weights of the
    experts that the step's tokens can pick at most, at HBM's peak."""
    mfma, valu, hbm = PEAK_TFLOPS["bf16"] * 1e12, PEAK_TFLOPS["fp32"] * 1e12, HBM_PEAK_GBS * 1e9
    names = ("sink_attention", "decay_scan", "routed_experts")
    pre, dec = {k: 0.0 for k in names}, {k: 0.0 for k in names}
    D = cfg["width"]
    for layer in cfg["layers"]:
        m = layer["mixer"]
        if layer["type"] == "latent_attention":
            pre["sink_attention"] += 2.0 * m["heads"] * 2 * m["kv_rank"] * (T * (T + 1) / 2) / mfma
            dec["sink_attention"] += n_seq * context * 2 * m["kv_rank"] * 2 / hbm
        elif layer["type"] == "mamba1":
            pre["decay_scan"] += 6.0 * T * m["inner"] * m["state"] / valu
            dec["decay_scan"] += n_seq * 2 * m["inner"] * m["state"] * 4 / hbm
        else:
            pre["decay_scan"] += 5.0 * T * m["heads"] * m["dim"] * m["vdim"] / valu
            dec["decay_scan"] += n_seq * 2 * m["heads"] * m["dim"] * m["vdim"] * 4 / hbm
        mlp = layer.get("mlp")
        if mlp:
            E, top, F = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            pre["routed_experts"] += 2.0 * 3 * T * top * D * F / mfma
            dec["routed_experts"] += min(n_seq * top, E) * 3 * D * F * 2 / hbm
    return {"prefill": pre, "decode": dec}


def design_comparison(design: str, T: int, n_seq: int, context: int, steps: int) -> dict:
    """Prefill and decode throughput of `design` at a few sizes that resemble real layers (random
    weights), beside the closest model the library has at equal size (for Begopel the Llama, for
    Zarinex the Begopel, for Satedra the Zarinex, for Kekelix the Satedra), and the GPU time of one prefill step and one decode step by operation."""
    import torch

    from picolm_amd.config import LlamaConfig, resolve
    from picolm_amd.engine import Session, random_model
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    out = {"design": design, "prefill_tokens": T, "decode_batch": n_seq, "decode_context": context, "dtype": "bf16",
           "data": "synthetic", "sizes": []}

    def measure(cfg, vocab):
        model = random_model(cfg, seed=0, std=0.02, dtype="bfloat16", device=dev)
        prompt = [int(t) for t in rng.integers(0, vocab, size=T)]
        res = {}
        for timed in (False, True):
            sess = Session(model, max_tokens=(T + 64) + n_seq * (context + 2 * steps + 64), n_slots=n_seq + 1, time_ops=timed)
            times = []
            for _ in range(4):
                [s] = sess.begin(1)
                torch.cuda.synchronize()
                if timed:
                    sess.engine.op_times()
                t0 = time.perf_counter()
                sess.step([s], [prompt])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                if timed:
                    res["prefill_ops_ms"] = sess.engine.op_times_by_label()
                sess.release([s])
            if not timed:
                res["prefill_tok_s"] = T / float(np.median(times[1:]))
            slots = sess.begin(n_seq)
            sess.step(slots, [[int(t) for t in rng.integers(0, vocab, size=context)] for _ in range(n_seq)])
            toks = [[int(t)] for t in rng.integers(0, vocab, size=n_seq)]
            for _ in range(4):
                sess.step(slots, toks)
            torch.cuda.synchronize()
            if timed:
                sess.engine.op_times()
                sess.step(slots, toks)
                res["decode_ops_ms"] = sess.engine.op_times_by_label()
            else:
                t0 = time.perf_counter()
                for _ in range(steps):
                    sess.step(slots, toks)
                torch.cuda.synchronize()
                res["decode_tok_s"] = n_seq * steps / (time.perf_counter() - t0)
            sess.release(slots)
            del sess
            torch.cuda.empty_cache()
        del model
        torch.cuda.empty_cache()
        return res

    def fractions_of(roof, res):
        return {phase: {k: roof[phase][k] / (res[phase + "_ops_ms"][k] * 1e-3) for k in roof[phase] if res[phase + "_ops_ms"].get(k)}
                for phase in ("prefill", "decode")}

    for name, size in DESIGN_SIZES[design]:
        print(f"[bench] {design} {name}", file=sys.stderr, flush=True)
        if design == "kekelix":
            kek, sat = _kekelix_pair(*size)
            a = measure(resolve(kek).parse_config(kek), kek["vocab"])
            b = measure(resolve(sat).parse_config(sat), sat["vocab"])
            out["sizes"].append({"size": name, "layer_runs": size[-1], design: a, "satedra": b,
                                 "fraction_of_roofline": fractions_of(_kekelix_rooflines(kek, T, n_seq, context), a),
                                 "satedra_fraction_of_roofline": fractions_of(_satedra_rooflines(sat, T, n_seq, context), b)})
            continue
        if design == "satedra":
            sat, zar = _satedra_pair(*size)
            a = measure(resolve(sat).parse_config(sat), sat["vocab"])
            b = measure(resolve(zar).parse_config(zar), zar["vocab"])
            out["sizes"].append({"size": name, "layer_runs": len(sat["layers"]), design: a, "zarinex": b,
                                 "fraction_of_roofline": fractions_of(_satedra_rooflines(sat, T, n_seq, context), a),
                                 "zarinex_fraction_of_roofline": fractions_of(_zarinex_rooflines(zar, T, n_seq, context), b)})
            continue
        if design == "zarinex":
            zar, beg = _zarinex_pair(*size)
            a = measure(resolve(zar).parse_config(zar), zar["vocab"])
            b = measure(resolve(beg).parse_config(beg), beg["vocab"])
            out["sizes"].append({"size": name, "layer_runs": len(zar["layers"]), design: a, "begopel": b,
                                 "fraction_of_roofline": fractions_of(_zarinex_rooflines(zar, T, n_seq, context), a),
                                 "begopel_fraction_of_roofline": fractions_of(_begopel_rooflines(beg, T, n_seq, context), b)})
            continue
        beg, llama = _begopel_pair(*size)
        a = measure(resolve(beg).parse_config(beg), beg["vocab"])
        b = measure(LlamaConfig.from_dict(llama), llama["vocab_size"])
        lc = LlamaConfig.from_dict(llama)
        like = {"prefill": attention_flops(lc, T) / (PEAK_TFLOPS["bf16"] * 1e12),
                "decode": n_seq * context * kv_bytes_per_token(lc) / (HBM_PEAK_GBS * 1e9)}
        fractions = fractions_of(_begopel_rooflines(beg, T, n_seq, context), a)
        for phase in ("prefill", "decode"):
            fractions[phase]["llama attention"] = like[phase] / (b[phase + "_ops_ms"]["attention"] * 1e-3)
        out["sizes"].append({"size": name, "layer_runs": llama["num_hidden_layers"], design: a, "llama": b,
                             "fraction_of_roofline": fractions})
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="llama31-8b")
    ap.add_argument("--steps", type=int, default=0, help="timed decode steps (default: the shape's, 64 for the 8B shape)")
    ap.add_argument("--warmup", type=int, default=-1)
    ap.add_argument("--batch", type=int, default=0, help="sequences of the timed decode (default: the shape's, 8 for the 8B shape)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--no-points", action="store_true", help="skip the further batch sizes, the prefill and the kernel classes")
    ap.add_argument("--prefill-only", action="store_true", help="run only the prefill (for profiling)")
    ap.add_argument("--batch-only", action="store_true", help="run only the decode at --batch (for profiling)")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the record: prefill of 128 to 32,768 tokens and decode at contexts of 16,384 to 131,072 "
                         "tokens, as one JSON line")
    ap.add_argument("--sampling", choices=["greedy", "picolm"], default="greedy",
                    help="greedy (the measured default) or picolm's command-line defaults: temperature 0.8, top_k 40, top_p 0.9, min_p 0.05")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="with --prefill-only: a prompt of another length than the 2,048 of the record")
    ap.add_argument("--prompt-range", default="",
                    help="prompt lengths of the decode runs, uniform in LO,HI (default: the shape's, 128,2048 for the 8B shape)")
    ap.add_argument("--context", type=int, default=CONTEXT, help="longest sequence the cache is laid out for")
    ap.add_argument("--weight-std", type=float, default=None,
                    help="standard deviation of the random weights (default: the shape's); 0 makes every operand of "
                         "every product zero, which shows what the GPU's power limit costs the same kernels on real data")
    ap.add_argument("--library-products", action="store_true",
                    help="time a layer's four products at 1, 8 and 64 rows and at the prefill's rows, this library's kernels "
                         "(with their epilogues) beside torch.matmul (the vendor library's plain product), both replayed "
                         "from a recorded graph over copies of the weights taken in turn; prints one JSON line")
    ap.add_argument("--steps-ahead", type=int, choices=[0, 1], default=1,
                    help="1 (the generation loop's way): the next step is launched before this step's tokens are "
                         "read on the host; 0: the host reads every step's tokens first")
    ap.add_argument("--design", choices=sorted(DESIGN_SIZES), default="",
                    help="instead of the record: prefill and decode throughput of another design at a few sizes beside the "
                         "closest model of equal size, with the GPU time of a step by operation, as one JSON line")
    args = ap.parse_args()
    if args.design:
        print(json.dumps(design_comparison(args.design, args.prefill_tokens, args.batch or 8, 1024, args.steps or 32)))
        return 0
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2

    import torch

    from picolm_amd import LlamaConfig, kernels
    from picolm_amd.engine import Session, random_model
    from picolm_amd.generation import SessionStepper, generate
    from picolm_amd.sampling import Sampler, SamplingParams
    from picolm_amd.sampling.params import CLI_DEFAULTS

    shape = SHAPES[args.shape]
    steps = args.steps or shape["steps"]
    warmup = args.warmup if args.warmup >= 0 else shape["warmup"]
    batch = args.batch or shape["batch"]
    full_layers = shape["config"]["num_hidden_layers"]
    cfg_dict = dict(shape["config"])
    if args.layers:
        cfg_dict["num_hidden_layers"] = args.layers
    cfg = LlamaConfig.from_dict(cfg_dict)
    dev = torch.device("cuda:0")
    if args.library_products:
        print(json.dumps(library_products(cfg, dev, args.prefill_tokens)))
        return 0
    t0 = time.time()
    if args.weight_std is not None:
        shape = dict(shape, std=args.weight_std)
    model = random_model(cfg, seed=0, std=shape["std"], dtype="bfloat16", device=dev)
    torch.cuda.synchronize()
    print(f"[bench] {shape['name']}: {cfg.num_hidden_layers} layers, {weight_bytes(cfg) / 1e9:.1f} GB of weights ready in "
          f"{time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    prompt_lo, prompt_hi = (int(x) for x in args.prompt_range.split(",")) if args.prompt_range else shape["prompt_range"]
    context = args.context

    def decode_run(n_seq: int, n_steps: int, n_warm: int, time_ops: bool = False, prompt_len: int = 0, seq_len: int = 0):
        """Decode steps of `n_seq` sequences after prompts of random lengths in the shape's range, or
        of `prompt_len` tokens each: (tokens a second, seconds a step, live context summed over the
        sequences in the middle of the timed steps, op times)."""
        seq_len = seq_len or context
        lens = [prompt_len] * n_seq if prompt_len else [int(x) for x in rng.integers(prompt_lo, prompt_hi + 1, size=n_seq)]
        prompts = [[int(t) for t in rng.integers(0, cfg.vocab_size, size=n)] for n in lens]
        pages = sum((min(n + n_steps + n_warm + 1, seq_len) + 63) // 64 for n in lens)
        sess = Session(model, max_tokens=pages * 64, max_seq_len=seq_len, n_slots=n_seq, time_ops=time_ops)
        sampler = Sampler(CLI_DEFAULTS if args.sampling == "picolm" else SamplingParams(), n_seq, dev)
        slots = sess.begin(n_seq)
        logits = SessionStepper(sess).step(slots, prompts)          # the prompts, as the generation loop sends them
        idx = list(range(n_seq))

        if args.steps_ahead:
            # as the generation loop runs: a step takes its tokens on the device from the draw
            # before it, and the host reads a step's tokens while the next step runs
            def one_step(pending):
                lg = sess.step_tokens_on_device(slots, pending.on_device())
                nxt = sampler.launch(lg, idx)
                pending.wait()
                return nxt

            state = sampler.launch(logits, idx)
        else:
            def one_step(lg):
                toks = sampler.sample(lg, idx)
                return sess.step(slots, [[t] for t in toks])

            state = logits
        for _ in range(n_warm):
            state = one_step(state)
        torch.cuda.synchronize()
        if time_ops:
            sess.engine.op_times()
        t = time.perf_counter()
        for _ in range(n_steps):
            state = one_step(state)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ops = sess.engine.op_times() if time_ops else None
        ctx = sum(sess.length(s) for s in slots) - n_seq * n_steps / 2.0     # live context, summed, in the middle of the timed steps
        sess.release(slots)
        del sess
        torch.cuda.empty_cache()
        return n_seq * n_steps / dt, dt / n_steps, ctx, ops

    def generation_loops(n_seq: int, few: int = 8, many: int = 104):
        """Tokens a second of whole generation loops over a batch of `n_seq` prompts: the library's
        own (picolm_engine_generate, one wait a step) and the Python loop (one step ahead), each as
        the time that `many - few` more tokens a sequence take."""
        lens = [int(x) for x in rng.integers(prompt_lo, prompt_hi + 1, size=n_seq)]
        prompts = [[int(t) for t in rng.integers(0, cfg.vocab_size, size=n)] for n in lens]
        pages = sum((min(n + many + 1, context) + 63) // 64 for n in lens)
        sess = Session(model, max_tokens=pages * 64, max_seq_len=context, n_slots=n_seq)
        params = CLI_DEFAULTS if args.sampling == "picolm" else SamplingParams()
        out = {}
        for name, run in (("c_api", lambda n: sess.engine.generate(prompts, n, params, [], batch_size=n_seq)),
                          ("python", lambda n: generate(sess, prompts, n, params, stop_ids=[], batch_size=n_seq))):
            run(few)                                  # the shapes' first uses (recordings) lie outside the clock
            times = []
            for n in (few, many):
                best = None
                for _ in range(3):                    # the prompts' time, which the difference removes, varies by more than a step
                    torch.cuda.synchronize()
                    t = time.perf_counter()
                    run(n)
                    torch.cuda.synchronize()
                    dt = time.perf_counter() - t
                    best = dt if best is None else min(best, dt)
                times.append(best)
            out[name] = n_seq * (many - few) / (times[1] - times[0])
        del sess
        torch.cuda.empty_cache()
        return out

    def prefill_run(T: int, reps: int = 3, time_ops: bool = False):
        sess = Session(model, max_tokens=T + 64, max_seq_len=max(context, T + 64), n_slots=1, time_ops=time_ops)
        toks = [int(t) for t in rng.integers(0, cfg.vocab_size, size=T)]
        times, ops = [], []
        for _ in range(reps + 1):
            [s] = sess.begin(1)
            torch.cuda.synchronize()
            t = time.perf_counter()
            sess.step([s], [toks])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            if time_ops:
                ops.append(sess.engine.op_times())
            sess.release([s])
        del sess
        torch.cuda.empty_cache()
        if time_ops:
            return {k: float(np.median([o[k] for o in ops[1:]])) for k in ops[0]}
        return float(np.median(times[1:]))

    def ceilings():
        """What a plain read of 4 GiB and a register-only MFMA loop reach on this GPU, each the best
        of a few launch shapes: (GB/s, TFLOP/s)."""
        src = torch.empty(4 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        sink = torch.zeros(1 << 20, dtype=torch.int32, device=dev)
        fsink = torch.zeros(4, device=dev)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def timed(f):
            f()
            out = []
            for _ in range(5):
                start.record()
                f()
                stop.record()
                torch.cuda.synchronize()
                out.append(start.elapsed_time(stop) * 1e-3)
            return float(np.median(out))
        read = max(kernels.read_probe(src, sink, b) / timed(lambda b=b: kernels.read_probe(src, sink, b)) / 1e9
                   for b in (2048, 1024, 512))
        mfma = max(kernels.mfma_probe(fsink, b, 2000) / timed(lambda b=b: kernels.mfma_probe(fsink, b, 2000)) / 1e12
                   for b in (512, 1024, 2048))
        # the same loop on operands like real data: the power limit then sets the clock
        mfma_real = max(kernels.mfma_probe(fsink, b, 16000, True) / timed(lambda b=b: kernels.mfma_probe(fsink, b, 16000, True)) / 1e12
                        for b in (512, 1024, 2048))
        del src
        torch.cuda.empty_cache()
        return read, mfma, mfma_real

    def kernel_classes(n_seq: int):
        """Each class of kernels against the nominal peak and against the measured ceiling, from
        events around every operation of launched (not replayed) steps."""
        read_gbs, mfma_tflops, mfma_real_tflops = ceilings()
        n = 12
        _, _, ctx, ops = decode_run(n_seq, n, 3, time_ops=True)
        out = {"read_ceiling_gbs": round(read_gbs, 1), "mfma_ceiling_tflops": round(mfma_tflops, 1),
               "mfma_ceiling_random_operands_tflops": round(mfma_real_tflops, 1), "decode_batch": n_seq}

        def put(name, achieved, unit, ceiling, peak):
            out[f"{name}_{unit}"] = round(achieved, 1)
            out[f"{name}_of_ceiling"] = round(achieved / ceiling, 4)
            out[f"{name}_of_peak"] = round(achieved / peak, 4)
        put("decode_products", cfg.num_hidden_layers * layer_weight_bytes(cfg) / (ops["products"] / n * 1e-3) / 1e9, "gbs", read_gbs, HBM_PEAK_GBS)
        put("decode_head", cfg.vocab_size * cfg.hidden_size * 2 / (ops["head"] / n * 1e-3) / 1e9, "gbs", read_gbs, HBM_PEAK_GBS)
        put("decode_attention", ctx * kv_bytes_per_token(cfg) / (ops["attention"] / n * 1e-3) / 1e9, "gbs", read_gbs, HBM_PEAK_GBS)
        pre = prefill_run(PREFILL_TOKENS, time_ops=True)
        put("prefill_products", product_flops(cfg, PREFILL_TOKENS) / (pre["products"] * 1e-3) / 1e12, "tflops", mfma_tflops, PEAK_TFLOPS["bf16"])
        put("prefill_attention", attention_flops(cfg, PREFILL_TOKENS) / (pre["attention"] * 1e-3) / 1e12, "tflops", mfma_tflops, PEAK_TFLOPS["bf16"])
        out["prefill_products_of_ceiling_random_operands"] = round(out["prefill_products_tflops"] / mfma_real_tflops, 4)
        return out

    if args.sweep:
        # further sizes and contexts: each prefill is one prompt from an empty cache; each decode
        # point has every sequence at the named context
        big = cfg.hidden_size >= 8192
        out = {"model": shape["name"], "layers": cfg.num_hidden_layers, "prefill": {}, "decode": {}}
        for T in ((2048, 8192) if big else (128, 512, 1024, 2048, 4096, 8192, 16384, 32768)):
            sec = prefill_run(T, reps=2)
            out["prefill"][str(T)] = {"ms": round(sec * 1e3, 3), "tok_s": round(T / sec, 1),
                                      "frac": round(prefill_flops(cfg, T) / sec / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
            print(f"[bench] prefill {T}: {sec * 1e3:.2f} ms", file=sys.stderr, flush=True)
        for b, ctx_len in (((8, 32768), (1, 32768)) if big else ((8, 16384), (4, 65536), (1, 131072))):
            n, warm = 12, 3
            tps, sps, ctx, _ = decode_run(b, n, warm, prompt_len=ctx_len - warm - n - 1, seq_len=ctx_len)
            gbs = (weight_bytes(cfg) + ctx * kv_bytes_per_token(cfg)) / sps / 1e9
            out["decode"][f"b{b}_ctx{ctx_len}"] = {"tok_s": round(tps, 2), "ms_per_step": round(sps * 1e3, 4),
                                                   "mean_context": round(ctx / b, 1), "gb_s": round(gbs, 1),
                                                   "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}
            print(f"[bench] decode b{b} at {ctx_len}: {sps * 1e3:.2f} ms a step", file=sys.stderr, flush=True)
        print(json.dumps(out))
        return 0
    if args.prefill_only:
        sec = prefill_run(args.prefill_tokens)
        print(json.dumps({"prefill_ms": round(sec * 1e3, 3), "tokens": args.prefill_tokens, "layers": cfg.num_hidden_layers}))
        return 0
    tok_s, s_per_step, ctx_tokens, _ = decode_run(batch, steps, warmup)
    step_bytes = weight_bytes(cfg) + ctx_tokens * kv_bytes_per_token(cfg)
    achieved = step_bytes / s_per_step / 1e9
    scaling = cfg.rope_scaling
    record = {
        "metric": f"decode tok/s at batch {batch} ({shape['name']}, bf16, context <= {context})",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(s_per_step * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": f"synthetic: random bf16 weights N(0,{shape['std']}), seeded uniform-random token ids, prompt lengths uniform in [{prompt_lo},{prompt_hi}]",
        "config": {
            "model": shape["name"], "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta,
            "rope_scaling": (f"llama3 factor {scaling.factor:g} low {scaling.low_freq_factor:g} high {scaling.high_freq_factor:g} "
                             f"original {scaling.original_max_position_embeddings}") if scaling else "none",
            "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings, "global_batch": batch,
            "seq_len": context, "prompt_lengths": f"uniform[{prompt_lo},{prompt_hi}]", "mean_context": round(ctx_tokens / batch, 1),
            "sampling": args.sampling, "steps_ahead": args.steps_ahead, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not (args.no_points or args.batch_only):
        sec = prefill_run(PREFILL_TOKENS)
        fl = prefill_flops(cfg, PREFILL_TOKENS)
        record["prefill"] = {"value": round(PREFILL_TOKENS / sec, 1), "tokens": PREFILL_TOKENS, "ms": round(sec * 1e3, 3),
                             "frac": round(fl / sec / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
        points = {}
        for b in shape["points"]:
            tps, sps, ctx, _ = decode_run(b, min(steps, 32 if b == 1 else 16), min(warmup, 4 if b == 1 else 2))
            points[f"decode_b{b}"] = round(tps, 2)
            points[f"decode_b{b}_ms_per_step"] = round(sps * 1e3, 4)
            points[f"decode_b{b}_mean_context"] = round(ctx / b, 1)
            points[f"decode_b{b}_hbm_frac"] = round((weight_bytes(cfg) + ctx * kv_bytes_per_token(cfg)) / sps / 1e9 / HBM_PEAK_GBS, 4)
        # the stated workload goes up to a total of `context` tokens: the same batches where the cache
        # weighs most, every sequence near 2,000 and near the full context
        for b in sorted(set(shape["points"]) | {batch}):
            for ctx_len in (2000, context - 96):
                n, warm = (16, 2) if b > 1 else (24, 3)
                tps, sps, ctx, _ = decode_run(b, n, warm, prompt_len=ctx_len - warm - n // 2)
                key = f"decode_b{b}_ctx{ctx_len}"
                points[key] = round(tps, 2)
                points[key + "_ms_per_step"] = round(sps * 1e3, 4)
                points[key + "_mean_context"] = round(ctx / b, 1)
                points[key + "_hbm_frac"] = round((weight_bytes(cfg) + ctx * kv_bytes_per_token(cfg)) / sps / 1e9 / HBM_PEAK_GBS, 4)
        loops = generation_loops(batch)
        points[f"generate_c_api_b{batch}"] = round(loops["c_api"], 2)
        points[f"generate_python_b{batch}"] = round(loops["python"], 2)
        record["points"] = points
        record["kernel_classes"] = kernel_classes(batch)
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
