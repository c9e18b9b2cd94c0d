"""Causal softmax attention in which every head holds two attention maps over the same values and
gives their difference:

    q [H][2][d], k [G][2][d], v [G][dv] = W h                       map m of a head lies behind map m - 1
    a_m  = softmax_j(scale q_m,i . k_m,j) v_j                       j <= i, for m = 1, 2
    lam  = exp(lq1 . lk1) - exp(lq2 . lk2) + diff                   one number for the layer
    o    = (a_1 - lam a_2) / sqrt(mean((a_1 - lam a_2)^2) + eps) * (1 - diff)     over the head's dv values
    out  = W_o concat_heads(o)

Positions do not enter the scores.  The cache keeps a token's two keys side by side as one key of
2 d entries; the attention operation runs 2 H queries of which query m is zero outside part m, so
that its product with the cached key is the product with key m, and leaves both maps as float rows
for the step that takes the difference."""
from __future__ import annotations

import math

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import KVRequest, Mixer, Runtime
from .calls import MapDifferenceArgs, SinkAttentionArgs, emit_library_call
from .linear import Linear


class DifferenceAttention(Mixer):
    graph_safe = True      # launches depend on device memory only
    LAMBDA_NAMES = ("lq1", "lk1", "lq2", "lk2")

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int, scale: float,
                 eps: float, diff: float):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not split over {n_kv_heads} KV heads")
        self.prefix, self.D = prefix, hidden_size
        self.H, self.G, self.d, self.dv = n_heads, n_kv_heads, head_dim, v_head_dim
        self.scale, self.eps, self.diff = float(scale), float(eps), float(diff)
        self.proj = Linear([prefix + "q", prefix + "k", prefix + "v"],
                           [n_heads * 2 * head_dim, n_kv_heads * 2 * head_dim, n_kv_heads * v_head_dim], hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], n_heads * v_head_dim)
        self.lam = None

    def children(self):
        return [self.proj, self.o]

    def tensor_specs(self):
        return [TensorSpec(self.prefix + n, (self.d,)) for n in self.LAMBDA_NAMES]

    def load(self, fetch, runtime: Runtime) -> None:
        lq1, lk1, lq2, lk2 = (fetch.get(self.prefix + n).to(torch.float32) for n in self.LAMBDA_NAMES)
        # float arithmetic, as the maps themselves
        self.lam = float(torch.exp(torch.sum(lq1 * lk1)) - torch.exp(torch.sum(lq2 * lk2)) + torch.tensor(self.diff, dtype=torch.float32))

    def cache_requests(self):
        return KVRequest(self.G, 2 * self.d, 0, self.dv), None

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(the normed difference of the two maps) for the rows h of `src`."""
        from ..engine.program import _DT
        if self.lam is None:
            raise ValueError(f"the attention of {self.prefix} has no weights loaded")
        H, G, d2, dv = self.H, self.G, 2 * self.d, self.dv
        width = self.proj.out_size
        rows = b.buffer("sink_attn.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        q = b.buffer("sink_attn.q", 2 * H * d2, b.dtype)
        maps = b.buffer("diff_attn.maps", 2 * H * dv, torch.float32)
        args = SinkAttentionArgs(H, G, d2, dv, width, 0, H * d2, H * d2 + G * d2, -1, self.scale, self.eps, None, None, None, 0, None)
        args.maps, args.out_float = 2, 1
        lib = kernels.lib()
        on_matrix_cores = b.dtype == torch.bfloat16 and lib.picolm_attn_plain_mfma_takes(d2, dv)
        emit_library_call(b, "sink_attention", args, maps, inp=rows, extra=[q], uses_kv=True, attends=True,
                          tile_rows=lib.picolm_attn_plain_mfma_tile_rows() if on_matrix_cores else kernels.attn_prefill_tile_rows(),
                          partial_floats=2 * H * (dv + 2))
        out = b.buffer("sink_attn.out", H * dv, b.dtype)
        emit_library_call(b, "map_difference", MapDifferenceArgs(H, dv, _DT[b.dtype], self.lam, self.eps, 1.0 - self.diff), out, inp=maps)
        self.o.emit(b, out, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))
