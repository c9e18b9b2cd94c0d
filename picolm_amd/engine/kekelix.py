"""The Kekelix decoder as a list of parts, and its entry in the architecture registry.

Layers whose mixer and feed-forward are two branches of the same rows, each behind an RMS norm
whose weight is an offset from one; three kinds of attention (two softmax maps a head whose normed
difference is the output; projections with biases, a partly rotated head and a softmax with one more
in its denominator; keys that are also the values, unit-RMS queries and keys, and stretches of
positions that bound what a query sees); routed experts picked by sigmoid scores that multiply what
the expert reads, with clamped hidden units; a stretch of layers that runs several times in a row,
every pass entered by adding the embedding's output again and a vector of the pass; a head tied to
the embedding table."""
from __future__ import annotations

from ..config import register_architecture
from ..config.kekelix import KekelixConfig
from ..parts import LMHead, RMSNorm, TokenEmbedding
from ..parts.block import LoopSum, ParallelBlock
from ..parts.difference_attention import DifferenceAttention
from ..parts.feedforward import RoutedExperts
from ..parts.position import RotaryEmbedding
from ..parts.sink_attention import SinkAttention
from ..weights import TensorSpec
from .begopel import _UnusedTensors
from .model import DecoderModel, LayerCall

EXPERT_SIGMOID_SLOPE = 1.702      # the design's constant in g sigmoid(1.702 g)


def _mixer(prefix: str, m, D: int, eps: float, rotations: dict):
    if m.kind == "attention":
        return DifferenceAttention(prefix, D, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, eps, m.diff)
    position = rotations.setdefault((m.rot.dims, m.rot.base, m.rot.scaling),
                                    RotaryEmbedding(m.rot.dims, m.rot.base, m.rot.scaling, style="half"))
    if m.kind == "attention_2":
        return SinkAttention(prefix, D, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, eps, qk_norm=False, sink=False, gate=False,
                             proj_bias=True, position=position, fixed_sink=0.0)
    return SinkAttention(prefix, D, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, eps, qk_norm=False, sink=False, gate=False,
                         position=position, unit_qk=True, chunk=m.chunk, values_are_keys=True)


def build_kekelix(cfg: KekelixConfig) -> DecoderModel:
    D, eps = cfg.width, cfg.norm_eps
    rotations = {}                       # one set of tables for the layers that turn alike
    blocks, unused = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mixer = _mixer(p + "mix.", layer.mixer, D, eps, rotations)
        ffn = None
        if layer.mlp is not None:
            ffn = RoutedExperts(p + "mlp.", D, layer.mlp.experts, layer.mlp.top, layer.mlp.ff, scoring="sigmoid", bias_name=None,
                                activation="clamped", limit=layer.mlp.limit, alpha=EXPERT_SIGMOID_SLOPE, weight_on_input=True)
        else:
            unused.append(TensorSpec(p + "norm2", (D,), optional=True, init=None))
        blocks.append(ParallelBlock(RMSNorm(p + "norm1", D, eps, weight_offset=1.0), mixer,
                                    RMSNorm(p + "norm2", D, eps, weight_offset=1.0) if ffn is not None else None, ffn))
    n_layers = len(blocks)
    if cfg.loop is not None:
        blocks += [LoopSum("loop.step", D, cfg.loop.times, t) for t in range(cfg.loop.times)]
    else:
        unused.append(TensorSpec("loop.step", (-1, D), optional=True, init=None))       # a checkpoint may carry the passes' vectors all the same
    order = []
    for i, t, first in cfg.layer_runs():
        if first:
            order.append(LayerCall(n_layers + t))
        order.append(LayerCall(i))
    emb = TokenEmbedding("embed", cfg.vocab, D, keeps_output=cfg.loop is not None and cfg.loop.times > 1)
    model = DecoderModel(cfg, emb, blocks, RMSNorm("final.norm", D, eps, weight_offset=1.0), LMHead("head", cfg.vocab, D, emb, tied=True),
                         order)
    model.extra_parts = [_UnusedTensors(unused)]
    return model


register_architecture("Kekelix", KekelixConfig.from_dict, build_kekelix, replace=True)
