"""The Satedra decoder as a list of parts, and its entry in the architecture registry.

Pre-norm layers with layer norms (weight and bias); every mixer an attention over cached latents
with a rotated key part shared by the heads (YaRN-scaled rotation), a sliding window and a gate per
head, some layers reading the latents that an earlier layer cached; a dense gated feed-forward, or
routed experts picked by softmax scores plus a correction, some of which give their input back,
beside a shared expert with a gate per token; a final layer norm and a head whose logits are
multiplied by a constant."""
from __future__ import annotations

from ..config import register_architecture
from ..config.satedra import SatedraConfig
from ..parts import LMHead, TokenEmbedding
from ..parts.block import PreNormBlock
from ..parts.feedforward import RoutedExperts, SwiGLU
from ..parts.latent_attention import RotatedLatentAttention
from ..parts.norm import LayerNorm
from ..parts.position import RotaryEmbedding
from ..weights import TensorSpec
from .begopel import _UnusedTensors
from .model import DecoderModel, LayerCall


def _feed_forward(prefix: str, mlp, D: int):
    if mlp.kind == "dense":
        return SwiGLU(prefix, D, mlp.ff, names=("gate", "up", "down"))
    return RoutedExperts(prefix, D, mlp.experts, mlp.top, mlp.ff, mlp.shared_ff, scoring="softmax_all", identity=mlp.identity,
                         weight_scale=mlp.scale, bias_name="correction", shared_gate="shared.sg" if mlp.shared_ff else None)


def build_satedra(cfg: SatedraConfig) -> DecoderModel:
    D, eps = cfg.width, cfg.norm_eps
    # a cache entry is laid out for the widest window among the layer that writes it and those that read it (0: all keys)
    windows = {}
    for i, layer in enumerate(cfg.layers):
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        windows.setdefault(owner, []).append(layer.mixer.window)
    cache_window = {owner: 0 if 0 in ws else max(ws) for owner, ws in windows.items()}
    rotations = {}                       # one set of tables for the layers that turn alike
    blocks, order, unused = [], [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        owner = i if m.kv_from is None else m.kv_from
        position = rotations.setdefault((m.rot_dim, m.rot_base, m.rot_scaling),
                                        RotaryEmbedding(m.rot_dim, m.rot_base, m.rot_scaling, style="half"))
        mixer = RotatedLatentAttention(p + "mix.", D, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, eps, position,
                                       window=m.window, reads_latents=m.kv_from is not None, cache_window=cache_window[owner])
        ffn = _feed_forward(p + "mlp.", layer.mlp, D) if layer.mlp is not None else None
        if ffn is None:
            unused += [TensorSpec(p + "norm2", (D,), optional=True, init=None), TensorSpec(p + "norm2.b", (D,), optional=True, init=None)]
        blocks.append(PreNormBlock(LayerNorm(p + "norm1", D, eps), mixer, LayerNorm(p + "norm2", D, eps) if ffn is not None else None, ffn))
        order.append(LayerCall(i, reads_cache_of=m.kv_from))
    emb = TokenEmbedding("embed", cfg.vocab, D)
    model = DecoderModel(cfg, emb, blocks, LayerNorm("final.norm", D, eps),
                         LMHead("head", cfg.vocab, D, emb, tied=False, scale=cfg.logit_scale), order)
    model.extra_parts = [_UnusedTensors(unused)]
    return model


register_architecture("Satedra", SatedraConfig.from_dict, build_satedra, replace=True)
