"""Token embedding and the output head.  x = table[token] widened to float, no scaling
(picolm/model_core.c:1785-1786); logits = W_out h, where W_out is the embedding table when
the checkpoint has no `lm_head.weight` (picolm/safetensors.c:248-251) or the configuration
ties them."""
from __future__ import annotations

import torch

from .. import kernels
from ..weights import TensorSpec
from .base import Part, Runtime


class TokenEmbedding(Part):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, name: str, vocab_size: int, hidden_size: int, scale: float = 1.0, keeps_output: bool = False,
                 positions: "SinusoidalPositions | None" = None):
        """`scale`: the rows are multiplied by it (in float).  `keeps_output`: the output is also
        left in a buffer of its own (`embed.out`), for parts that read it again later.  `positions`:
        a vector per position that is added to the rows."""
        self.name, self.V, self.D = name, vocab_size, hidden_size
        self.scale, self.keeps_output = float(scale), bool(keeps_output)
        self.positions = positions
        self.table = None

    def children(self):
        return [self.positions] if self.positions is not None else []

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.V, self.D))]

    def load(self, fetch, runtime: Runtime) -> None:
        t = fetch.get(self.name)
        self.table = (t.to(torch.float32) if runtime.is_f32 else t).contiguous()

    def emit(self, b) -> int:
        """The lookup as an operation of a launch program; returns the buffer of the residual rows."""
        if self.table is None:
            raise ValueError(f"embedding {self.name} has no table loaded")
        x = b.buffer("residual", self.D, torch.float32)
        b.embed(self.table, x, self.scale)
        if self.positions is not None:
            self.positions.emit(b, x)
        if self.keeps_output:
            b.embed(self.table, b.buffer("embed.out", self.D, torch.float32), self.scale)
        return x

    def forward(self, tokens: torch.Tensor, x: torch.Tensor) -> None:
        """The same on tensors, now: rows of the table for `tokens`, widened to float, into x."""
        kernels.embed(self.table, tokens, x)
        if self.scale != 1.0:
            x.mul_(self.scale)


class SinusoidalPositions(Part):
    """A fixed vector per position, added to the embedding: entry 2i is sin(p f_i), entry 2i+1 is
    cos(p f_i) with f_i = base^(-2i / width).  The frequencies are laid out once, in double; the
    angle of a token is taken in double from its position in the step's arrays, so the part has no
    table that a longest sequence would size."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, width: int, base: float = 10000.0):
        self.width, self.base = int(width), float(base)
        self.freq = None

    def load(self, fetch, runtime: Runtime) -> None:
        i = torch.arange((self.width + 1) // 2, dtype=torch.float64)
        self.freq = torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / self.width).to(runtime.device).contiguous()

    def emit(self, b, x: int) -> None:
        from .calls import AddPositionsArgs, emit_library_call
        if self.freq is None:
            raise ValueError("the positions have no frequencies laid out (load)")
        emit_library_call(b, "add_positions", AddPositionsArgs(b._ptr(self.freq), self.width), x)


class LMHead(Part):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, name: str, vocab_size: int, hidden_size: int, embedding: TokenEmbedding, tied: bool,
                 softcap: float = 0.0, scale: float = 1.0):
        """`scale`: the logits are multiplied by it; `softcap` c > 0: then logits <- c tanh(logits / c)."""
        self.name, self.V, self.D, self.embedding, self.tied = name, vocab_size, hidden_size, embedding, tied
        self.softcap, self.scale = float(softcap or 0.0), float(scale)
        self.weight = None

    def tensor_specs(self):
        # optional either way: absent -> the embedding table serves; a tied model's stray
        # copy is ignored
        return [TensorSpec(self.name, (self.V, self.D), optional=True, init=None if self.tied else "normal")]

    def load(self, fetch, runtime: Runtime) -> None:
        if self.tied or not fetch.has(self.name):
            self.weight = self.embedding.table
        else:
            t = fetch.get(self.name)
            self.weight = (t.to(torch.float32) if runtime.is_f32 else t).contiguous()

    def emit(self, b, src) -> None:
        """logits = W h for the wanted rows h of `src`, as an operation of a launch program."""
        from ..engine.program import ROWS_WANTED
        if self.weight is None:
            raise ValueError(f"head {self.name} has no weights loaded")
        logits = b.buffer("logits", self.V, torch.float32, ROWS_WANTED)
        b.linear(self.weight, src, logits, kernels.EPI_STORE, rows=ROWS_WANTED)
        if self.scale != 1.0:
            from .calls import MAP_SCALE, MapRowsArgs, emit_library_call
            from ..engine.program import F32
            emit_library_call(b, "map_rows", MapRowsArgs(MAP_SCALE, self.V, F32, F32, self.scale), logits, rows=ROWS_WANTED)
        if self.softcap > 0:
            from .calls import MAP_SOFTCAP, MapRowsArgs, emit_library_call
            from ..engine.program import F32
            emit_library_call(b, "map_rows", MapRowsArgs(MAP_SOFTCAP, self.V, F32, F32, self.softcap), logits, rows=ROWS_WANTED)
        b.logits_buffer = logits

    def forward(self, h: torch.Tensor, logits: torch.Tensor) -> None:
        """The same on tensors, now."""
        kernels.gemm(h, self.weight, logits, kernels.EPI_STORE)
        if self.scale != 1.0:
            logits.mul_(self.scale)
        if self.softcap > 0:
            logits.copy_(self.softcap * torch.tanh(logits / self.softcap))
