"""Causal softmax attention whose every refinement is an option: biases of the projections, a
rotation of part of every head, an RMS norm of queries and keys per head (with a weight, or to unit
root mean square without one), a learned bias by distance, one more term in the softmax's
denominator (a sink, learned per head or a constant), values of a size of their own or the keys
themselves as values, stretches of positions that bound what a query sees, and a gate on the heads
before the output projection.

    q, k, v, g = W h (+ b);  q, k <- turned by the position;  q <- rms(q) w_q,  k <- rms(k) w_k     per head
    s_ij = scale (q_i . k_j) + rel[bucket(i - j)][head]                j <= i, and floor(i / chunk) = floor(j / chunk)
    p_ij = exp(s_ij) / (exp(sink_head) + sum_j' exp(s_ij'))            the sink is a term of the denominator only
    out  = W_o (concat_heads(sum_j p_ij v_j) * sigmoid(g))

The bias table has B rows: one per distance below B/2, then rows spaced evenly in the logarithm of
the distance up to `bias_max`, the last row for everything beyond.  It is expanded once, at load,
into one entry per distance up to `bias_max` and per head; the attention kernels index that by
min(distance, last).
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import KVRequest, Mixer, Runtime
from .calls import SinkAttentionArgs, emit_library_call
from .linear import Linear


def distance_rows(n_rows: int, bias_max: float) -> list[int]:
    """For every distance 0 .. ceil(bias_max) the row of a table of `n_rows` that holds its bias."""
    half = n_rows // 2
    last = int(math.ceil(bias_max))
    if n_rows > 1 and not bias_max > half:
        raise ValueError(f"a bias table of {n_rows} rows needs bias_max above {half}, got {bias_max}")
    rows = []
    for n in range(last + 1):
        if n < half or n_rows == 1:
            rows.append(min(n, n_rows - 1))
        else:
            steps = math.log(n / half) / math.log(bias_max / half) * (n_rows - half)
            rows.append(min(n_rows - 1, half + int(math.floor(steps))))
    return rows


class SinkAttention(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, eps: float, bias_rows: int | None = None, bias_max: float = 0.0, has_bias: bool = False,
                 qk_norm: bool = True, sink: bool = True, gate: bool = True, proj_bias: bool = False, position=None,
                 unit_qk: bool = False, fixed_sink: float | None = None, chunk: int = 0, values_are_keys: bool = False):
        """`has_bias`: scores get the bias by distance, from a table of `bias_rows` rows (None: as many
        as the checkpoint's tensor has) that reaches to `bias_max`.  `proj_bias`: q, k and v have
        biases, the tensors `<name>.b`.  `position`: a `RotaryEmbedding` over the first entries of
        every query and key head (as many as it was made for).  `unit_qk` (without `qk_norm`): queries
        and keys are divided by their root mean square, after the rotation.  `fixed_sink` (without
        `sink`): the denominator's extra term is exp(fixed_sink) for every head, and no tensor holds
        it.  `chunk` > 0: a query sees the keys of its own stretch of `chunk` positions, counted from
        the sequence's first.  `values_are_keys`: there is no value projection; a token's value is its
        key as projected, before rotation and norm."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not split over {n_kv_heads} KV heads")
        self.prefix, self.D = prefix, hidden_size
        self.H, self.G, self.d, self.dv = n_heads, n_kv_heads, head_dim, v_head_dim
        self.scale, self.eps = float(scale), float(eps)
        self.has_bias = bool(has_bias or bias_rows)
        self.bias_rows, self.bias_max = (None if bias_rows is None else int(bias_rows)), float(bias_max)
        if self.has_bias and not self.bias_max > 0:
            raise ValueError("a bias by distance needs bias_max, the distance its last row starts at")
        self.qk_norm, self.has_sink, self.has_gate = qk_norm, sink, gate
        if values_are_keys and v_head_dim != head_dim:
            raise ValueError(f"values that are the keys have the keys' size {head_dim}, not {v_head_dim}")
        if position is not None and not 0 < position.head_dim <= head_dim:
            raise ValueError(f"a rotation of {position.head_dim} entries of a head of {head_dim}")
        if chunk < 0:
            raise ValueError(f"stretches of {chunk} positions")
        self.proj_bias, self.position, self.unit_qk = bool(proj_bias), position, bool(unit_qk) and not qk_norm
        self.fixed_sink = None if sink or fixed_sink is None else float(fixed_sink)
        self.chunk, self.values_are_keys = int(chunk), bool(values_are_keys)
        names = [prefix + "q", prefix + "k"] + ([] if values_are_keys else [prefix + "v"]) + ([prefix + "g"] if gate else [])
        sizes = ([n_heads * head_dim, n_kv_heads * head_dim] + ([] if values_are_keys else [n_kv_heads * v_head_dim]) +
                 ([n_heads * v_head_dim] if gate else []))
        self.proj = Linear(names, sizes, hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], n_heads * v_head_dim)
        self.q_norm = self.k_norm = self.bias = self.sink = self.in_bias = None

    def children(self):
        return [self.proj, self.o] + ([self.position] if self.position is not None else [])

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        if self.position is not None:
            self.position.prepare(runtime, max_positions)

    def tensor_specs(self):
        specs = []
        if self.qk_norm:
            specs += [TensorSpec(self.prefix + "q.norm", (self.d,), init="ones"), TensorSpec(self.prefix + "k.norm", (self.d,), init="ones")]
        if self.has_bias:       # (-1: any number of rows; random weights need the number)
            specs.append(TensorSpec(self.prefix + "rel", (self.bias_rows if self.bias_rows is not None else -1, self.H)))
        if self.has_sink:
            specs.append(TensorSpec(self.prefix + "sink", (self.H,)))
        if self.proj_bias:
            specs += [TensorSpec(n + ".b", (size,)) for n, size in zip(self.proj.names[:2 if self.values_are_keys else 3], self.proj.out_sizes)]
        return specs

    def load(self, fetch, runtime: Runtime) -> None:
        f32 = lambda name: fetch.get(self.prefix + name).to(torch.float32).contiguous()
        if self.qk_norm:
            self.q_norm, self.k_norm = f32("q.norm"), f32("k.norm")
        if self.has_bias:
            rel = f32("rel")
            rows = distance_rows(rel.shape[0], self.bias_max)
            self.bias = rel[torch.tensor(rows, device=rel.device)].t().contiguous()   # [H, distances]
        if self.has_sink:
            self.sink = f32("sink")
        elif self.fixed_sink is not None:
            self.sink = torch.full((self.H,), self.fixed_sink, dtype=torch.float32, device=runtime.device)
        if self.proj_bias:          # one entry per column of the stacked product; the gate's columns get none
            parts = [fetch.get(n + ".b").to(torch.float32) for n in self.proj.names[:2 if self.values_are_keys else 3]]
            parts.append(torch.zeros(self.proj.out_size - sum(p.numel() for p in parts), dtype=torch.float32, device=parts[0].device))
            self.in_bias = torch.cat(parts).contiguous()

    def cache_requests(self):
        return KVRequest(self.G, self.d, 0, self.dv), None

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(gate * attention) for the rows h of `src`, as operations of a launch program."""
        H, G, d, dv = self.H, self.G, self.d, self.dv
        width = self.proj.out_size
        rows = b.buffer("sink_attn.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        q = b.buffer("sink_attn.q", H * d, b.dtype)
        out = b.buffer("sink_attn.out", H * dv, b.dtype)
        q_off, k_off = 0, H * d
        v_off = k_off if self.values_are_keys else k_off + G * d
        gate_off = (k_off + G * d if self.values_are_keys else v_off + G * dv) if self.has_gate else -1
        args = SinkAttentionArgs(H, G, d, dv, width, q_off, k_off, v_off, gate_off, self.scale, self.eps,
                                 b._ptr(self.q_norm), b._ptr(self.k_norm), b._ptr(self.bias),
                                 0 if self.bias is None else self.bias.shape[1], b._ptr(self.sink))
        args.chunk, args.unit_qk, args.in_bias = self.chunk, int(self.unit_qk), b._ptr(self.in_bias)
        if self.position is not None:
            cos, sin, style = self.position.rotary_tables()
            if cos is None:
                raise ValueError(f"the rotation of {self.prefix} has no tables laid out (prepare)")
            args.cos_table, args.sin_table, args.table_positions = b._ptr(cos), b._ptr(sin), cos.shape[0]
            args.rot_dims, args.rot_half = self.position.head_dim, style
        lib = kernels.lib()
        on_matrix_cores = b.dtype == torch.bfloat16 and lib.picolm_attn_plain_mfma_takes(d, dv)
        emit_library_call(b, "sink_attention", args, out, inp=rows, extra=[q], uses_kv=True, attends=True,
                          tile_rows=lib.picolm_attn_plain_mfma_tile_rows() if on_matrix_cores else kernels.attn_prefill_tile_rows(),
                          partial_floats=H * (dv + 2))
        if accumulate:
            self.o.emit(b, out, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)
        else:
            self.o.emit(b, out, x, kernels.EPI_STORE)
