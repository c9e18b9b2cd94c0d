"""Gated feed-forward: down(silu(gate x) * (up x)), no bias (picolm/model_core.c:2182-2204,
silu picolm/tensor.c:3306-3315).  gate and up are one product over row-interleaved weights
whose epilogue applies silu(g) * u; the down product adds into the residual."""
from __future__ import annotations

from .. import kernels
from .base import FeedForward, StepContext, keeps_forward
from .linear import Linear


class SwiGLU(FeedForward):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        self.D, self.F = hidden_size, intermediate_size
        self.gate_up = Linear([prefix + names[0], prefix + names[1]], [intermediate_size] * 2, hidden_size,
                              interleave=True)
        self.down = Linear([prefix + names[2]], [hidden_size], intermediate_size)

    def children(self):
        return [self.gate_up, self.down]

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += down(silu(gate h) * (up h)) for the rows h of `src`, as operations of a launch program."""
        if not keeps_forward(self, SwiGLU):
            return FeedForward.emit(self, b, src, x, out_norm, out_norm_when)
        act = b.buffer("ffn.act", self.F, b.dtype)
        self.gate_up.emit(b, src, act, kernels.EPI_SWIGLU)
        self.down.emit(b, act, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)

    def forward(self, ctx: StepContext, h, residual) -> None:
        """The same on tensors, now: for parts that run from Python (a routed feed-forward calls
        its experts on the rows it sends them)."""
        act = ctx.ws.get("ffn.act", (h.shape[0], self.F), ctx.dtype)
        self.gate_up.forward(h, act, kernels.EPI_SWIGLU)
        self.down.forward(act, residual, kernels.EPI_ACCUMULATE)


class ActivatedMLP(FeedForward):
    """Two matrices with an activation between them: down(act(up h)), no bias.  `activation`:
    "relu_squared" is max(z, 0)^2.  The up product leaves float rows, the activation is taken in
    float and rounded once to the dtype the down product reads."""
    graph_safe = True      # launches depend on device memory only
    ACTIVATIONS = {"relu_squared": 1}

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "relu_squared",
                 names=("up", "down")):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation '{activation}': known are {', '.join(self.ACTIVATIONS)}")
        self.D, self.F, self.activation = hidden_size, intermediate_size, activation
        self.up = Linear([prefix + names[0]], [intermediate_size], hidden_size)
        self.down = Linear([prefix + names[1]], [hidden_size], intermediate_size)

    def children(self):
        return [self.up, self.down]

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += down(act(up h)) for the rows h of `src`, as operations of a launch program."""
        import torch
        from ..engine.program import _DT, F32
        from .calls import MapRowsArgs, emit_library_call
        pre = b.buffer("ffn.pre", self.F, torch.float32)
        act = b.buffer("ffn.act", self.F, b.dtype)
        self.up.emit(b, src, pre, kernels.EPI_STORE)
        emit_library_call(b, "map_rows", MapRowsArgs(self.ACTIVATIONS[self.activation], self.F, F32, _DT[b.dtype], 0.0), act, inp=pre)
        self.down.emit(b, act, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)


class RoutedExperts(FeedForward):
    """A feed-forward of many small gated experts of which every row uses a few:
        z = W_router h;  out = sum_k w_k expert_k(h)  (+ shared(h)) over the row's `top` picks k
    scoring "picked_softmax": the largest z + b are picked (ties: the lower index) and w is the
    softmax over the picked z + b alone.  scoring "softmax_all": s = softmax(z) over every router
    output, the largest s + b are picked, and w = s_k / (sum of the picked s + 1e-20) * weight_scale.
    expert(h) = down(silu(gate h) * (up h)), no biases; the last `identity` router outputs have no
    tensors and stand for experts that give h back; `shared_size` > 0 adds one more expert of that
    inner width that every row passes, multiplied by sigmoid(w_sg . h), one number a row, where
    `shared_gate` names that vector's tensor.  `bias_name`: the tensor b, one entry per router
    output.  The router's logits, the picks and their weights are float; only the picked experts'
    weights are read."""
    graph_safe = True      # launches depend on device memory only
    SCORINGS = {"picked_softmax": 0, "softmax_all": 1, "sigmoid": 2}
    ACTIVATIONS = {"silu_gated": 0, "clamped": 1}

    def __init__(self, prefix: str, hidden_size: int, n_experts: int, top: int, expert_size: int, shared_size: int = 0,
                 names=("gate", "up", "down"), scoring: str = "picked_softmax", identity: int = 0, weight_scale: float = 1.0,
                 bias_name: str | None = "router.b", shared_gate: str | None = None, activation: str = "silu_gated",
                 limit: float = 0.0, alpha: float = 1.0, weight_on_input: bool = False):
        """`bias_name` None: the router has no bias tensor."""
        if scoring not in self.SCORINGS:
            raise ValueError(f"scoring '{scoring}': known are {', '.join(self.SCORINGS)}")
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation '{activation}': known are {', '.join(self.ACTIVATIONS)}")
        if activation == "clamped" and not limit > 0:
            raise ValueError(f"the clamped activation needs a positive limit, got {limit}")
        if weight_on_input and identity:
            raise ValueError("weights on the experts' input and router outputs that give the input back do not go together")
        self.activation, self.limit, self.alpha, self.weight_on_input = activation, float(limit), float(alpha), bool(weight_on_input)
        if n_experts < 1 or identity < 0 or not 1 <= top <= n_experts + identity:
            raise ValueError(f"{top} picks among {n_experts} experts and {identity} that give their input back")
        if shared_gate and not shared_size:
            raise ValueError("a gate of the shared expert needs a shared expert")
        self.prefix, self.D, self.E, self.top, self.F, self.names = prefix, hidden_size, n_experts, top, expert_size, tuple(names)
        self.scoring, self.identity, self.weight_scale = scoring, int(identity), float(weight_scale)
        self.bias_name, self.shared_gate = bias_name, shared_gate
        self.outputs = n_experts + self.identity           # what the router gives a row
        # the shared expert's gate is one more row of the router's product: both read h
        self.router = Linear([prefix + "router"] + ([prefix + shared_gate] if shared_gate else []),
                             [self.outputs] + ([1] if shared_gate else []), hidden_size)
        self.shared_gate_up = self.shared_down = None
        if shared_size:
            self.shared_gate_up = Linear([prefix + "shared." + names[0], prefix + "shared." + names[1]], [shared_size] * 2, hidden_size,
                                         interleave=True)
            self.shared_down = Linear([prefix + "shared." + names[2]], [hidden_size], shared_size)
        self.shared_size = shared_size
        self.gate = self.up = self.down = self.router_bias = None

    def children(self):
        return [p for p in (self.router, self.shared_gate_up, self.shared_down) if p is not None]

    def tensor_specs(self):
        from ..weights import TensorSpec
        specs = [TensorSpec(self.prefix + self.bias_name, (self.outputs,), init="zeros")] if self.bias_name else []
        for e in range(self.E):
            p = f"{self.prefix}e{e}."
            specs += [TensorSpec(p + self.names[0], (self.F, self.D)), TensorSpec(p + self.names[1], (self.F, self.D)),
                      TensorSpec(p + self.names[2], (self.D, self.F))]
        return specs

    def load(self, fetch, runtime) -> None:
        import torch

        def stacked(name):      # [experts][out][in], in the dtype the runtime multiplies in
            ws = [fetch.get(f"{self.prefix}e{e}.{name}") for e in range(self.E)]
            if runtime.is_f32 or any(w.dtype == torch.float32 for w in ws):
                ws = [w.to(torch.float32) for w in ws]
            return torch.stack(ws, dim=0).contiguous()
        self.gate, self.up, self.down = (stacked(n) for n in self.names)
        self.router_bias = fetch.get(self.prefix + self.bias_name).to(torch.float32).contiguous() if self.bias_name else None

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0, accumulate: bool = True) -> None:
        """x (+)= the picked experts' weighted sum (+ the shared expert) for the rows h of `src`."""
        import torch
        from ..engine.program import _DT
        from .calls import GATE_SIGMOID, GateRowsArgs, RoutedExpertsArgs, RouteTopArgs, emit_library_call
        if self.gate is None:
            raise ValueError(f"the experts of {self.prefix} have no weights loaded")
        h = b.materialize(src)
        n_logits = self.router.out_size
        logits = b.buffer("moe.logits", n_logits, torch.float32)
        self.router.emit(b, h, logits, kernels.EPI_STORE)
        picks = b.buffer("moe.picks", 2 * self.top, torch.float32)
        emit_library_call(b, "route_top", RouteTopArgs(b._ptr(self.router_bias), self.outputs, self.top, self.SCORINGS[self.scoring], n_logits,
                                                       self.weight_scale), picks, inp=logits)
        written = accumulate
        if self.shared_size:
            act = b.buffer("ffn.act", self.shared_size, b.dtype)
            self.shared_gate_up.emit(b, h, act, kernels.EPI_SWIGLU)
            if self.shared_gate:
                # down(act) * s = down(act * s) for a number s a row: the hidden units take the gate
                gated = b.buffer("ffn.act.gated", self.shared_size, b.dtype)
                emit_library_call(b, "gate_rows", GateRowsArgs(self.shared_size, GATE_SIGMOID, self.shared_size, 0, _DT[b.dtype], n_logits,
                                                               self.outputs, _DT[b.dtype], None, 1), gated, inp=act, extra=[logits])
                act = gated
            self.shared_down.emit(b, act, x, kernels.EPI_ACCUMULATE if accumulate else kernels.EPI_STORE)
            written = True
        hidden = b.buffer("moe.hidden", self.top * self.F, torch.float32)
        args = RoutedExpertsArgs(b._ptr(self.gate), b._ptr(self.up), b._ptr(self.down), _DT[self.gate.dtype], self.E, self.top, self.D,
                                 self.F, int(written), self.identity, self.ACTIVATIONS[self.activation], self.limit, self.alpha,
                                 int(self.weight_on_input))
        pair_out = b.buffer("moe.pairs", self.top * self.D, torch.float32)
        plan = b.buffer("moe.plan", self.top + self.E + 1, torch.float32)
        emit_library_call(b, "routed_experts", args, x, inp=h, extra=[picks, hidden, pair_out, plan])
