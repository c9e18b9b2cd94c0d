"""Arrangements of norm, mixer and feed-forward in a layer.  PreNormBlock is picolm's
(picolm/model_core.c:1841, :2151, :2160, :2204): x += mixer(norm(x)); x += ffn(norm(x));
a block without a feed-forward skips the second half, as picolm does when the three
matrices are absent (:2159)."""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm


def norm_ref_of(norm):
    """The norm as the product before it may prepare it, or None for a norm of another kind."""
    f = getattr(norm, "norm_ref", None)
    return f() if f is not None else None


class PreNormBlock(Block):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def first_norm(self):
        """The norm this block applies to the residual stream on entry: the block before may
        have it prepared."""
        return self.mixer_norm

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        """x += mixer(norm(x)); x += ffn(norm(x)) over the residual rows in buffer `x`, as operations
        of a launch program.  `after`: the RMSNorm that meets x after this block (after_when = 1: only
        in steps that want every row's logits), so that the block's last product can prepare it.
        Every part emits what it is: the engine's operations, or a call of its `forward`."""
        if type(self).forward is not Block.forward and type(self).emit is PreNormBlock.emit:
            return Block.emit(self, b, x, after, after_when)       # a subclass with an arrangement of its own
        src = self.mixer_norm.emit(b, x)
        if self.ffn is None:
            self.mixer.emit(b, src, x, after, after_when)
            return
        self.mixer.emit(b, src, x, norm_ref_of(self.ffn_norm), 0)
        self.ffn.emit(b, self.ffn_norm.emit(b, x), x, after, after_when)


class _NoMixer(Mixer):
    """The mixer of a block that has none: it asks nothing of the cache."""


class ParallelBlock(Block):
    """Mixer and feed-forward as two branches of the same rows, each behind a norm of its own:
        x <- x + mixer(norm1(x)) + ffn(norm2(x))
    A block without a feed-forward is x <- x + mixer(norm1(x)).  Both norms are taken before the
    mixer's output joins x (two RMS norms with one eps in one pass over the rows, `rms_pair`: they
    share the root); the two branches then add to x one after the other."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def _shared_root(self):
        """The two norms as (NormRef, NormRef) if they are RMS norms with one eps over the same width,
        so that one pass over a row serves both; else None."""
        if self.ffn is None:
            return None
        a, c = norm_ref_of(self.mixer_norm), norm_ref_of(self.ffn_norm)
        if a is None or c is None or a.eps != c.eps or a.weight.shape != c.weight.shape:
            return None
        return a, c

    def first_norm(self):
        """The norm that the block before may have prepared: the mixer's, unless one kernel takes
        both norms of this block."""
        return None if self._shared_root() else self.mixer_norm

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        from ..engine.program import _DT, Rows
        from .calls import RmsPairArgs, emit_library_call
        if self.ffn is None:
            self.mixer.emit(b, self.mixer_norm.emit(b, x), x, after, after_when)
            return
        pair = self._shared_root()
        if pair is not None:
            first = b.buffer("norm.out", self.mixer_norm.size, b.dtype)
            second = b.buffer("norm.out.second", self.ffn_norm.size, b.dtype)
            emit_library_call(b, "rms_pair", RmsPairArgs(b._ptr(pair[0].weight), b._ptr(pair[1].weight), self.mixer_norm.size, _DT[b.dtype],
                                                        pair[0].eps), first, inp=x, extra=[second])
            self.mixer.emit(b, Rows(first), x, None, 0)
            self.ffn.emit(b, Rows(second), x, after, after_when)
            return
        src = self.mixer_norm.emit(b, x)
        second = self.ffn_norm.emit(b, x)
        if second.norm is not None:         # rows of their own: the first norm's place is in use until the mixer has read it
            second = Rows(b.buffer("norm.out.second", self.ffn_norm.size, b.dtype), second.norm, second.x)
        held = Rows(b.materialize(second))
        self.mixer.emit(b, src, x, None, 0)
        self.ffn.emit(b, held, x, after, after_when)


class _WithRowState(Mixer):
    """A mixer as the cache sees it when its block keeps `row_floats` floats of its own per
    sequence in front of the mixer's state: one state entry holds both."""

    def __init__(self, inner: Mixer, row_floats: int):
        self.inner, self.row_floats = inner, int(row_floats)
        if self.row_floats and hasattr(inner, "state_base"):
            inner.state_base = self.row_floats

    def cache_requests(self):
        import torch
        from .base import StateRequest
        kv, st = self.inner.cache_requests()
        if not self.row_floats:
            return kv, st
        if st is not None and (len(st.shape) != 1 or st.dtype != torch.float32 or not hasattr(self.inner, "state_base")):
            raise ValueError(f"{type(self.inner).__name__} keeps a state that a row cannot be put in front of")
        return kv, StateRequest((self.row_floats + (st.shape[0] if st is not None else 0),), torch.float32)

    def prepare(self, runtime, max_positions: int) -> None:
        self.inner.prepare(runtime, max_positions)


class PostNormBlock(Block):
    """Norm after the sum, each branch reading the residual rows themselves:
        x <- norm1(alpha x + gate1(x) * mixer(shifted(x)));   x <- norm2(alpha x + gate2(x) * ffn(x))
    shifted(x)[t] = x[t] + (x[t-1] - x[t]) * mu (`shift_name`: the tensor mu; None: the mixer reads x),
    with the row before a step's first one kept in the layer call's state; gate(x) = sigmoid(W x + b)
    (`gate_names`: the two matrices, their biases at `<name>.b`; None: no gates).  A block without a
    feed-forward has the first half only."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, hidden_size: int, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, ffn: FeedForward | None,
                 alpha: float = 1.0, shift_name: str | None = None, gate_names=None):
        from .linear import Linear
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.D, self.alpha = hidden_size, float(alpha)
        self.mixer_norm, self.inner, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.shift_name = shift_name
        self.mixer = _WithRowState(mixer, hidden_size if shift_name else 0)
        self.gate_names = tuple(gate_names) if gate_names else None
        self.gates = [Linear([n], [hidden_size], hidden_size) for n in self.gate_names[:2 if ffn is not None else 1]] if gate_names else []
        self.mu = None
        self.gate_bias = []

    def children(self):
        return [p for p in (self.mixer_norm, self.inner, self.ffn_norm, self.ffn, *self.gates) if p is not None]

    def tensor_specs(self):
        from ..weights import TensorSpec
        specs = [TensorSpec(self.shift_name, (self.D,))] if self.shift_name else []
        specs += [TensorSpec(g.names[0] + ".b", (self.D,), init="zeros") for g in self.gates]
        if self.gate_names and len(self.gates) < len(self.gate_names):      # a block without a feed-forward may carry its gate all the same
            specs += [TensorSpec(n + s, shape, optional=True, init=None) for n in self.gate_names[len(self.gates):]
                      for s, shape in (("", (self.D, self.D)), (".b", (self.D,)))]
        return specs

    def load(self, fetch, runtime) -> None:
        import torch
        if self.shift_name:
            self.mu = fetch.get(self.shift_name).to(torch.float32).contiguous()
        self.gate_bias = [fetch.get(g.names[0] + ".b").to(torch.float32).contiguous() for g in self.gates]

    def _join(self, b, x: int, branch: int, plain: int, which: int, norm, leaves_plain: bool = False) -> None:
        """x <- norm(alpha x + branch * gate(plain)); leaves_plain: and the new x in `plain`, in the
        dtype that products read."""
        import torch
        from .. import kernels
        from .calls import GatedPostnormArgs, emit_library_call
        extra, bias = [-1], None
        if self.gates:
            g = b.buffer("postnorm.gate", self.D, torch.float32)
            self.gates[which].emit(b, plain, g, kernels.EPI_STORE)
            extra, bias = [g], self.gate_bias[which]
        if leaves_plain:
            extra.append(plain)
        ref = norm.norm_ref()
        if ref is None:
            raise ValueError("a block that norms after the sum takes RMS norms")
        emit_library_call(b, "gated_postnorm", GatedPostnormArgs(b._ptr(ref.weight), b._ptr(bias), self.D, self.alpha, ref.eps), x,
                          inp=branch, extra=extra)

    def _plain_rows(self, b, x: int) -> int:
        """The residual rows in the dtype that products read."""
        import torch
        from ..engine.program import _DT, F32
        from .calls import GATE_NONE, GateRowsArgs, emit_library_call
        plain = b.buffer("postnorm.plain", self.D, b.dtype)
        emit_library_call(b, "gate_rows", GateRowsArgs(self.D, GATE_NONE, self.D, 0, F32, 0, 0, _DT[b.dtype], None), plain, inp=x)
        return plain

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        import torch
        from ..engine.program import Rows
        from .calls import TokenShiftArgs, emit_library_call
        D = self.D
        if self.shift_name:
            if self.mu is None:
                raise ValueError(f"{self.shift_name} is not loaded")
            plain = b.buffer("postnorm.plain", D, b.dtype)
            reads = b.buffer("postnorm.shifted", D, b.dtype)
            emit_library_call(b, "token_shift", TokenShiftArgs(b._ptr(self.mu), D, 0), reads, inp=x, extra=[plain] if self.gates else [],
                              uses_state=True)
        else:
            plain = reads = self._plain_rows(b, x)
        branch = b.buffer("postnorm.branch", D, torch.float32)
        self.inner.emit(b, Rows(reads), branch, accumulate=False)
        self._join(b, x, branch, plain, 0, self.mixer_norm, leaves_plain=self.ffn is not None)
        if self.ffn is not None:
            self.ffn.emit(b, Rows(plain), branch, accumulate=False)
            self._join(b, x, branch, plain, 1, self.ffn_norm)




class LoopSum(Block):
    """What runs before pass `number` over a looped stretch of layers where the pass is entered by
    sums alone:  x <- x + x0 (every pass but the first) + step[number], with x0 the embedding's
    output (which the embedding keeps, `TokenEmbedding(keeps_output=True)`) and step [passes, D]."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, step_name: str, hidden_size: int, passes: int, number: int):
        if not 0 <= number < passes:
            raise ValueError(f"pass {number} of {passes}")
        self.D, self.passes, self.number = hidden_size, passes, number
        self.step_name = step_name
        self.mixer = _NoMixer()
        self.step = None

    def tensor_specs(self):
        from ..weights import TensorSpec
        return [TensorSpec(self.step_name, (self.passes, self.D))]

    def load(self, fetch, runtime) -> None:
        import torch
        self.step = fetch.get(self.step_name).to(torch.float32).contiguous()

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        import torch
        from .calls import AddRowsArgs, emit_library_call
        if self.step is None:
            raise ValueError(f"loop entry {self.step_name} has no weights loaded")
        first = b.buffer("embed.out", self.D, torch.float32) if self.number > 0 else -1
        emit_library_call(b, "add_rows", AddRowsArgs(b._ptr(self.step[self.number]), self.D), x, inp=first)


class LoopEntry(Block):
    """What runs before pass `number` over a looped stretch of layers:
    x <- W_in [x ; x0] + step[number], with x0 the embedding's output (which the embedding keeps,
    `TokenEmbedding(keeps_output=True)`), W_in [D, 2 D] and step [passes, D].  The passes of one
    loop share the two tensors; each pass is a part of its own because its vector differs."""
    graph_safe = True      # launches depend on device memory only

    def __init__(self, w_in, step_name: str, hidden_size: int, passes: int, number: int):
        """`w_in`: the `Linear` [D, 2 D] that the passes share."""
        if not 0 <= number < passes:
            raise ValueError(f"pass {number} of {passes}")
        self.D, self.passes, self.number = hidden_size, passes, number
        self.step_name = step_name
        self.w_in = w_in
        self.mixer = _NoMixer()
        self.step = None

    def children(self):
        return [self.w_in]

    def tensor_specs(self):
        from ..weights import TensorSpec
        return [TensorSpec(self.step_name, (self.passes, self.D))]

    def load(self, fetch, runtime) -> None:
        import torch
        self.step = fetch.get(self.step_name).to(torch.float32).contiguous()

    def emit(self, b, x: int, after=None, after_when: int = 0) -> None:
        import torch
        from .. import kernels
        from .calls import LoopInputArgs, emit_library_call
        if self.step is None:
            raise ValueError(f"loop entry {self.step_name} has no weights loaded")
        first = b.buffer("embed.out", self.D, torch.float32)
        joined = b.buffer("loop.joined", 2 * self.D, b.dtype)
        row = self.step[self.number]
        emit_library_call(b, "loop_input", LoopInputArgs(b._ptr(row), self.D), x, inp=first, extra=[joined])
        self.w_in.emit(b, joined, x, kernels.EPI_ACCUMULATE, out_norm=after, out_norm_when=after_when)
