"""Typed configuration of the Kekelix decoder, read from the keys of its config.json.

    architecture        "Kekelix"
    vocab, width        sizes of the embedding table (the head is the table itself)
    norm.eps            eps of every RMS norm (the layers', the final one, and the weightless ones inside mixers)
    layers[i]           {"type": "attention" | "attention_2" | "attention_3", "mixer": {...}, "mlp": {...} | null}
        attention       mixer {heads, kv_heads, dim, vdim, scale, diff}: two softmax maps a head, their difference normed
        attention_2     mixer {heads, kv_heads, dim, vdim, scale, rot: {base, dims, scaling: {factor, original, fast,
                        slow} | absent}}: biases on q, k, v, a rotation of the first rot.dims entries of a head, a
                        softmax with one more in its denominator
        attention_3     mixer {heads, kv_heads, dim, vdim, scale, rot: {base, dims}, mask: {size}}: the values are the
                        keys, q and k of unit RMS after the rotation, a query sees its own stretch of mask.size positions
        mlp             {"kind": "moe", "router": {experts, top}, "expert": {ff, limit}}
    loop                {start, stop, times}: layers start .. stop-1 run `times` times in a row (absent: no loop)

Every size the model uses comes from an instance of `KekelixConfig`.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .begopel import MAX_HEAD_DIM, LoopConfig, _integer, _number, _object
from .llama import ConfigError
from .satedra import YarnScaling

MIXER_TYPES = ("attention", "attention_2", "attention_3")


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: YarnScaling | None = None

    @staticmethod
    def from_dict(d: dict, where: str) -> "RotationConfig":
        scaling = d.get("scaling")
        if scaling is not None and not isinstance(scaling, dict):
            raise ConfigError(f"{where}scaling: expected an object or null")
        c = RotationConfig(_number(d, where, "base"), _integer(d, where, "dims"),
                           YarnScaling.from_dict(scaling, where + "scaling.") if scaling else None)
        if c.dims % 2:
            raise ConfigError(f"{where}dims: {c.dims} is odd, the rotation pairs entries")
        if not c.base > 0 or c.base == 1.0:
            raise ConfigError(f"{where}base: must be positive and not 1")
        return c

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class KekelixMixer:
    kind: str                        # one of MIXER_TYPES
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float = 0.0                # attention: the constant of the maps' difference
    rot: RotationConfig | None = None
    chunk: int = 0                   # attention_3: positions a stretch

    @staticmethod
    def from_dict(kind: str, d: dict, where: str) -> "KekelixMixer":
        rot = mask = None
        diff = 0.0
        if kind == "attention":
            diff = _number(d, where, "diff")
        else:
            rot = RotationConfig.from_dict(_object(d, where, "rot"), where + "rot.")
        if kind == "attention_3":
            mask = _integer(_object(d, where, "mask"), where + "mask.", "size")
        dim = _integer(d, where, "dim")
        # where the values are the keys they have the keys' size, whatever `vdim` says
        heads = _integer(d, where, "heads")
        # (a configuration that leaves them out: a KV head a head, and the usual 1 / sqrt(dim))
        c = KekelixMixer(kind, heads, _integer(d, where, "kv_heads", heads), dim,
                         dim if kind == "attention_3" else _integer(d, where, "vdim"), _number(d, where, "scale", dim ** -0.5), diff, rot,
                         mask or 0)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}kv_heads: {c.kv_heads} does not divide heads = {c.heads}")
        key = 2 * c.dim if kind == "attention" else c.dim          # both maps' keys of a token are cached side by side
        if key > MAX_HEAD_DIM:
            raise ConfigError(f"{where}dim: a cached key of {key} entries exceeds {MAX_HEAD_DIM}, the largest the attention kernels take")
        if c.vdim > MAX_HEAD_DIM:
            raise ConfigError(f"{where}vdim: {c.vdim} exceeds {MAX_HEAD_DIM}, the largest head the attention kernels take")
        if not c.scale > 0:
            raise ConfigError(f"{where}scale: must be positive")
        if rot is not None and rot.dims > c.dim:
            raise ConfigError(f"{where}rot.dims: {rot.dims} entries of a head of {c.dim}")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.kind == "attention":
            d["diff"] = self.diff
        else:
            d["rot"] = self.rot.to_dict()
        if self.kind == "attention_3":
            d["mask"] = {"size": self.chunk}
        return d


@dataclass(frozen=True)
class KekelixMLP:
    experts: int
    top: int
    ff: int
    limit: float

    @staticmethod
    def from_dict(d: dict, where: str) -> "KekelixMLP":
        kind = d.get("kind")
        if kind != "moe":
            raise ConfigError(f"{where}kind: '{kind}' is not supported (known: moe)")
        router, expert = _object(d, where, "router"), _object(d, where, "expert")
        c = KekelixMLP(_integer(router, where + "router.", "experts"), _integer(router, where + "router.", "top"),
                       _integer(expert, where + "expert.", "ff"), _number(expert, where + "expert.", "limit"))
        if c.top > c.experts:
            raise ConfigError(f"{where}router.top: {c.top} exceeds the {c.experts} experts")
        if not c.limit > 0:
            raise ConfigError(f"{where}expert.limit: must be positive")
        return c

    def to_dict(self) -> dict:
        return {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff, "limit": self.limit}}


@dataclass(frozen=True)
class KekelixLayer:
    mixer: KekelixMixer
    mlp: KekelixMLP | None           # None: the layer has no feed-forward

    @staticmethod
    def from_dict(d: dict, where: str) -> "KekelixLayer":
        if not isinstance(d, dict):
            raise ConfigError(f"{where[:-1]}: expected an object")
        kind = d.get("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}type: '{kind}' is not a known mixer (known: {', '.join(MIXER_TYPES)})")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}mlp: expected an object or null")
        return KekelixLayer(KekelixMixer.from_dict(kind, _object(d, where, "mixer"), where + "mixer."),
                            KekelixMLP.from_dict(mlp, where + "mlp.") if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.mixer.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class KekelixConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float = 1e-6
    loop: LoopConfig | None = None
    torch_dtype: str = "bfloat16"
    max_position_embeddings: int | None = None       # rotary tables are laid out for what the cache holds
    bos_token_id: int | None = None
    eos_token_ids: tuple = field(default=())

    @staticmethod
    def from_dict(root: dict) -> "KekelixConfig":
        if not isinstance(root, dict):
            raise ConfigError("config.json: expected an object")
        layers = root.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("layers: expected a list of at least one layer")
        norm = root.get("norm") or {}
        loop = root.get("loop")
        if loop is not None and not isinstance(loop, dict):
            raise ConfigError("loop: expected an object or null")
        eos = root.get("eos_token_id")
        cfg = KekelixConfig(
            vocab=_integer(root, "", "vocab"), width=_integer(root, "", "width"),
            layers=tuple(KekelixLayer.from_dict(l, f"layers[{i}].") for i, l in enumerate(layers)),
            norm_eps=_number(norm, "norm.", "eps", 1e-6),
            loop=(LoopConfig(_integer(loop, "loop.", "start", least=0), _integer(loop, "loop.", "stop", least=0),
                             _integer(loop, "loop.", "times")) if loop is not None else None),
            torch_dtype=str(root.get("torch_dtype", "bfloat16")),
            max_position_embeddings=(_integer(root, "", "max_position_embeddings")
                                     if root.get("max_position_embeddings") is not None else None),
            bos_token_id=None if root.get("bos_token_id") is None else int(root["bos_token_id"]),
            eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps: must be positive")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"torch_dtype: '{self.torch_dtype}' is not one of bfloat16, float32, float16")
        if self.loop is not None and not 0 <= self.loop.start <= self.loop.stop <= len(self.layers):
            raise ConfigError(f"loop: layers {self.loop.start} .. {self.loop.stop - 1} are not a stretch of the {len(self.layers)} layers")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"eos_token_id: {e} is outside the vocabulary of {self.vocab}")

    def to_dict(self) -> dict:
        d = {"architecture": "Kekelix", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [l.to_dict() for l in self.layers], "torch_dtype": self.torch_dtype}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    # -- derived ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    def layer_runs(self) -> list:
        """The layers in the order they run, as (layer, pass number or None, first of its pass):
        the looped stretch `times` times in a row, then the rest."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None, False) for i in range(n)]
        lp = self.loop
        runs = [(i, None, False) for i in range(lp.start)]
        for t in range(lp.times):
            runs += [(i, t, i == lp.start) for i in range(lp.start, lp.stop)]
        return runs + [(i, None, False) for i in range(lp.stop, n)]
