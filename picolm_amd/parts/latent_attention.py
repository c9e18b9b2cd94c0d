"""Causal softmax attention whose keys and values are read out of one small latent per token, so
that only the latent is cached; queries pass a latent of their own; no positions.

    c_q = rms(W_dq h) w_dq;  q = W_uq c_q                       [heads, dim]
    c   = rms(W_dkv h) w_dkv                                    [kv_rank]: what the cache keeps
    k_j = W_uk c_j, v_j = W_uv c_j per head;  s_ij = scale (q_i . k_j),  j <= i;  p = softmax(s)
    out = W_o (concat_heads(sum_j p_ij v_j) * sigmoid(W_g h))

The products with W_uk and W_uv are moved off the cached side: q_i . (W_uk c_j) = (W_uk^T q_i) . c_j
and sum_j p_ij W_uv c_j = W_uv (sum_j p_ij c_j), so the attention runs over the latents themselves,
all heads sharing one key head whose keys and values are both c, and a token costs two small
products per head instead of two per head and cached token.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import KVRequest, Mixer, Runtime
from .calls import GATE_NONE, GATE_SIGMOID, HeadLinearArgs, SinkAttentionArgs, SliceNormArgs, emit_library_call
from .linear import Linear


class LatentAttention(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, head_dim: int, v_head_dim: int, kv_rank: int, q_rank: int,
                 scale: float, eps: float, gate: bool = True):
        self.prefix, self.D = prefix, hidden_size
        self.H, self.d, self.dv, self.r, self.rq = n_heads, head_dim, v_head_dim, kv_rank, q_rank
        self.scale, self.eps, self.has_gate = float(scale), float(eps), bool(gate)
        names = [prefix + "dq", prefix + "dkv"] + ([prefix + "g"] if gate else [])
        self.proj = Linear(names, [q_rank, kv_rank] + ([n_heads * v_head_dim] if gate else []), hidden_size)
        self.uq = Linear([prefix + "uq"], [n_heads * head_dim], q_rank)
        self.o = Linear([prefix + "o"], [hidden_size], n_heads * v_head_dim)
        self.uk = self.uv = self.q_norm = self.c_norm = None
        self.uk_transposed = False

    def children(self):
        return [self.proj, self.uq, self.o]

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "dq.norm", (self.rq,), init="ones"), TensorSpec(p + "dkv.norm", (self.r,), init="ones"),
                TensorSpec(p + "uk", (self.H * self.d, self.r)), TensorSpec(p + "uv", (self.H * self.dv, self.r))]

    def load(self, fetch, runtime: Runtime) -> None:
        kept = lambda name: (lambda t: t.to(torch.float32) if runtime.is_f32 else t)(fetch.get(self.prefix + name)).contiguous()
        self.uk, self.uv = kept("uk"), kept("uv")
        # the bfloat16 runtime keeps W_uk transposed per head, [heads][kv_rank][dim]: q' = W_uk^T q is then a plain product
        # per head, which the matrix cores take; the 32-bit runtime multiplies with the tensor as it is stored
        self.uk_transposed = not runtime.is_f32
        if self.uk_transposed:
            self.uk = self.uk.view(self.H, self.d, self.r).transpose(1, 2).contiguous().view(self.H * self.r, self.d)
        self.q_norm = fetch.get(self.prefix + "dq.norm").to(torch.float32).contiguous()
        self.c_norm = fetch.get(self.prefix + "dkv.norm").to(torch.float32).contiguous()

    def cache_requests(self):
        return KVRequest(1, self.r, 0, self.r), None

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(gate * attention) for the rows h of `src`, as operations of a launch program."""
        from ..engine.program import _DT, F32
        H, d, dv, r, rq = self.H, self.d, self.dv, self.r, self.rq
        width = self.proj.out_size
        engine_dt = _DT[b.dtype]
        rows = b.buffer("latent.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        cq = b.buffer("latent.cq", rq, b.dtype)
        emit_library_call(b, "slice_norm", SliceNormArgs(b._ptr(self.q_norm), rq, width, 0, rq, 0, engine_dt, self.eps), cq, inp=rows)
        q = b.buffer("latent.q", H * d, torch.float32)
        self.uq.emit(b, cq, q, kernels.EPI_STORE)
        # [W_uk^T q per head | c]: the attention's queries, and its one key and value
        qc = b.buffer("latent.qc", H * r + r, torch.float32)
        weight_dt = _DT[self.uk.dtype]
        emit_library_call(b, "head_linear", HeadLinearArgs(b._ptr(self.uk), weight_dt, H, d, r, 0 if self.uk_transposed else 1, H * d, 0, F32,
                                                           H * r + r, 0, F32,
                                                           GATE_NONE, 0, 0), qc, inp=q)
        emit_library_call(b, "slice_norm", SliceNormArgs(b._ptr(self.c_norm), r, width, rq, H * r + r, H * r, F32, self.eps), qc, inp=rows)
        scratch = b.buffer("latent.q.rows", H * r, b.dtype)
        att = b.buffer("latent.att", H * r, b.dtype)
        args = SinkAttentionArgs(H, 1, r, r, H * r + r, 0, H * r, H * r, -1, self.scale, self.eps, None, None, None, 0, None)
        lib = kernels.lib()
        on_matrix_cores = b.dtype == torch.bfloat16 and lib.picolm_attn_plain_mfma_takes(r, r)
        emit_library_call(b, "sink_attention", args, att, inp=qc, extra=[scratch], uses_kv=True, attends=True,
                          tile_rows=lib.picolm_attn_plain_mfma_tile_rows() if on_matrix_cores else kernels.attn_prefill_tile_rows(),
                          partial_floats=H * (r + 2))
        heads = b.buffer("latent.heads", H * dv, b.dtype)
        emit_library_call(b, "head_linear", HeadLinearArgs(b._ptr(self.uv), weight_dt, H, r, dv, 0, H * r, 0, engine_dt, H * dv, 0, engine_dt,
                                                           GATE_SIGMOID if self.has_gate else GATE_NONE, width, rq + r), heads, inp=att,
                          extra=[rows] if self.has_gate else [])
        self.o.emit(b, heads, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))


class RotatedLatentAttention(Mixer):
    """Attention over cached latents with a rotated key part beside them, a window and a gate per head:

        q = W_q h, per head [dim unrotated | rot_dim rotated by the position]
        [c_raw | k_raw] = W_dkv h;  c = rms(c_raw) w_c  [kv_rank];  k_rot = rotated(k_raw)  [rot_dim], one for all heads
        s_ij = scale (q_plain_i . (W_uk c_j) + q_rot_i . k_rot_j)  for  0 <= i - j < window;  p = softmax(s)
        out = W_o concat_heads(sigmoid((W_g h)_head) * sum_j p_ij W_uv c_j)

    What a token leaves in the cache is [c | k_rot], a key of kv_rank + rot_dim, and c once more as
    the value.  As in `LatentAttention` the products with W_uk and W_uv are moved off the cached
    side: the query of a head is [W_uk^T q_plain | q_rot], the attention runs over one key head for
    all query heads, and W_uv meets the weighted sum of latents.  `reads_latents=True`: the layer
    has no W_dkv and reads the cache entry of another layer call (whose latents, rotated parts and
    rotation are of the same kind); its window is its own.  `cache_window`: the window that the
    cache entry is laid out for where several layers with windows of their own read it (the widest
    of them, 0 for all keys; None: this layer's).  `position`: the rotation, a `PositionEncoding` with tables over `rot_dim` entries."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, kv_rank: int,
                 scale: float, eps: float, position, window: int = 0, reads_latents: bool = False, cache_window: int | None = None,
                 gate: bool = True):
        self.prefix, self.D = prefix, hidden_size
        self.H, self.d, self.dr, self.dv, self.r = n_heads, head_dim, rot_dim, v_head_dim, kv_rank
        self.scale, self.eps, self.window = float(scale), float(eps), int(window)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        if self.cache_window and (not self.window or self.window > self.cache_window):
            raise ValueError(f"a window of {self.window or 'all'} keys over a cache entry laid out for {self.cache_window}")
        self.reads_latents, self.has_gate, self.position = bool(reads_latents), bool(gate), position
        names = [prefix + "q"] + ([] if reads_latents else [prefix + "dkv"]) + ([prefix + "g"] if gate else [])
        sizes = [n_heads * (head_dim + rot_dim)] + ([] if reads_latents else [kv_rank + rot_dim]) + ([n_heads] if gate else [])
        self.proj = Linear(names, sizes, hidden_size)
        self.o = Linear([prefix + "o"], [hidden_size], n_heads * v_head_dim)
        self.uk = self.uv = self.c_norm = None
        self.uk_transposed = False

    def children(self):
        return [self.proj, self.o, self.position]

    def tensor_specs(self):
        p = self.prefix
        specs = [TensorSpec(p + "uk", (self.H * self.d, self.r)), TensorSpec(p + "uv", (self.H * self.dv, self.r))]
        if not self.reads_latents:
            specs.append(TensorSpec(p + "dkv.norm", (self.r,), init="ones"))
        return specs

    def load(self, fetch, runtime: Runtime) -> None:
        kept = lambda name: (lambda t: t.to(torch.float32) if runtime.is_f32 else t)(fetch.get(self.prefix + name)).contiguous()
        self.uk, self.uv = kept("uk"), kept("uv")
        # the bfloat16 runtime keeps W_uk transposed per head, [heads][kv_rank][dim]: q' = W_uk^T q is then a plain product
        # per head, which the matrix cores take; the 32-bit runtime multiplies with the tensor as it is stored
        self.uk_transposed = not runtime.is_f32
        if self.uk_transposed:
            self.uk = self.uk.view(self.H, self.d, self.r).transpose(1, 2).contiguous().view(self.H * self.r, self.d)
        if not self.reads_latents:
            self.c_norm = fetch.get(self.prefix + "dkv.norm").to(torch.float32).contiguous()

    def cache_requests(self):
        # every key stays in its page: a layer that reads the entry may look further back than the one that writes it
        return KVRequest(1, self.r + self.dr, self.cache_window, self.r, keeps_all=True), None

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        self.position.prepare(runtime, max_positions)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= o(gate * attention) for the rows h of `src`, as operations of a launch program."""
        from ..engine.program import _DT, F32
        from .calls import RotateHeadsArgs
        H, d, dr, dv, r = self.H, self.d, self.dr, self.dv, self.r
        if b.binding is not None and bool(b.binding.writes) == self.reads_latents:
            raise ValueError(f"{self.prefix}: a layer that keeps latents of its own writes its cache entry, one that reads another's does not")
        tables = self.position.rotary_tables()
        if tables is None:
            raise ValueError(f"{self.prefix}: the rotated part needs a rotation with tables")
        cos, sin, style = tables
        if cos.shape[1] * 2 != dr:
            raise ValueError(f"{self.prefix}: the rotation's tables turn {cos.shape[1] * 2} entries, the rotated part has {dr}")
        width = self.proj.out_size
        q_size, key = H * (d + dr), r + dr
        c_at = q_size                                    # [c_raw | k_raw] in the projected rows (a layer with latents of its own)
        g_at = q_size + (0 if self.reads_latents else key)
        engine_dt = _DT[b.dtype]
        rows = b.buffer("rla.in", width, torch.float32)
        self.proj.emit(b, src, rows, kernels.EPI_STORE)
        # [per head: W_uk^T q_plain | rotated q] and then the token's key [c | rotated k]; the value is the key's first kv_rank entries
        q_wide = H * key
        qc = b.buffer("rla.qc", q_wide + key, torch.float32)
        weight_dt = _DT[self.uk.dtype]
        emit_library_call(b, "head_linear", HeadLinearArgs(b._ptr(self.uk), weight_dt, H, d, r, 0 if self.uk_transposed else 1, width, 0, F32,
                                                           q_wide + key, 0, F32, GATE_NONE, 0, 0, d + dr, key, 0), qc, inp=rows)
        # one pass over a token's row: the queries' rotated parts behind each head's W_uk^T q, and for a layer with latents of its own
        # the normed latent and the rotated key part behind the queries
        own = (1, c_at + r, 0, q_wide + r, 0, b._ptr(self.c_norm), r, c_at, q_wide, self.eps) if not self.reads_latents else ()
        emit_library_call(b, "rotate_heads", RotateHeadsArgs(b._ptr(cos), b._ptr(sin), cos.shape[0], dr, style, H, dr, width, d, d + dr,
                                                             q_wide + key, r, key, *own), qc, inp=rows)
        scratch = b.buffer("rla.q.rows", q_wide, b.dtype)
        att = b.buffer("rla.att", H * r, b.dtype)
        args = SinkAttentionArgs(H, 1, key, r, q_wide + key, 0, q_wide, q_wide, -1, self.scale, self.eps, None, None, None, 0, None,
                                 self.window if self.window != self.cache_window else 0)
        lib = kernels.lib()
        on_matrix_cores = b.dtype == torch.bfloat16 and lib.picolm_attn_plain_mfma_takes(key, r)
        emit_library_call(b, "sink_attention", args, att, inp=qc, extra=[scratch], uses_kv=True, attends=True,
                          tile_rows=lib.picolm_attn_plain_mfma_tile_rows() if on_matrix_cores else kernels.attn_prefill_tile_rows(),
                          partial_floats=H * (r + 2))
        heads = b.buffer("rla.heads", H * dv, b.dtype)
        emit_library_call(b, "head_linear", HeadLinearArgs(b._ptr(self.uv), weight_dt, H, r, dv, 0, H * r, 0, engine_dt, H * dv, 0, engine_dt,
                                                           GATE_SIGMOID if self.has_gate else GATE_NONE, width, g_at, 0, 0, 1), heads, inp=att,
                          extra=[rows] if self.has_gate else [])
        self.o.emit(b, heads, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE,
                    **({"out_norm": out_norm, "out_norm_when": out_norm_when} if accumulate else {}))
