"""Typed configuration of the Satedra decoder, read from the keys of its config.json.

    architecture        "Satedra"
    vocab, width        sizes of the embedding table
    norm.eps            eps of every norm (the layer norms and the RMS norm of the latents)
    logit_scale         the logits are multiplied by it
    layers[i]           {"type": "latent_attention", "mixer": {...}, "mlp": {...} | null}
        mixer           {heads, dim, rot_dim, vdim, kv_rank, scale, mask: {size}, rot: {base, dims, scaling: {factor,
                         original, fast, slow} | null}, kv_from: j}     kv_from: the layer reads layer j's latents and
                         rotated key parts instead of making its own
        mlp             {"kind": "dense", "ff"} or
                        {"kind": "moe", "router": {experts, top, identity, scale}, "expert": {ff}, "shared": {ff} | null}

Every size the model uses comes from an instance of `SatedraConfig`.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .begopel import MAX_HEAD_DIM, _integer, _number, _object
from .llama import ConfigError


@dataclass(frozen=True)
class YarnScaling:
    """Frequencies whose wavelength fits `slow` turns or fewer into `original` positions are divided
    by `factor`, those that fit `fast` turns or more stay, with a ramp over the pairs between."""
    factor: float
    original: float
    fast: float
    slow: float

    @staticmethod
    def from_dict(d: dict, where: str) -> "YarnScaling":
        c = YarnScaling(_number(d, where, "factor"), _number(d, where, "original"), _number(d, where, "fast"), _number(d, where, "slow"))
        for key in ("factor", "original", "fast", "slow"):
            if not getattr(c, key) > 0:
                raise ConfigError(f"{where}{key}: must be positive")
        return c

    def to_dict(self) -> dict:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class RotatedLatentAttentionConfig:
    heads: int
    dim: int                         # unrotated query/key entries a head
    rot_dim: int                     # rotated ones; the rotated key part is shared by the heads
    vdim: int
    kv_rank: int
    scale: float
    window: int                      # a query sees itself and the window - 1 tokens before it; 0: all
    rot_base: float
    rot_scaling: YarnScaling | None = None
    kv_from: int | None = None

    @staticmethod
    def from_dict(d: dict, where: str) -> "RotatedLatentAttentionConfig":
        rot = _object(d, where, "rot")
        mask = d.get("mask")
        if mask is not None and not isinstance(mask, dict):
            raise ConfigError(f"{where}mask: expected an object")
        scaling = rot.get("scaling")
        if scaling is not None and not isinstance(scaling, dict):
            raise ConfigError(f"{where}rot.scaling: expected an object or null")
        source = d.get("kv_from")
        c = RotatedLatentAttentionConfig(
            _integer(d, where, "heads"), _integer(d, where, "dim"), _integer(d, where, "rot_dim"), _integer(d, where, "vdim"),
            _integer(d, where, "kv_rank"), _number(d, where, "scale"), _integer(mask, where + "mask.", "size") if mask else 0,
            _number(rot, where + "rot.", "base"), YarnScaling.from_dict(scaling, where + "rot.scaling.") if scaling else None,
            None if source is None else _integer(d, where, "kv_from", least=0))
        if _integer(rot, where + "rot.", "dims") != c.rot_dim:
            raise ConfigError(f"{where}rot.dims: {rot['dims']} is not rot_dim = {c.rot_dim}, the part of a head that is rotated")
        if c.rot_dim % 2:
            raise ConfigError(f"{where}rot_dim: {c.rot_dim} is odd, the rotation pairs entries")
        if not c.scale > 0:
            raise ConfigError(f"{where}scale: must be positive")
        if not c.rot_base > 0:
            raise ConfigError(f"{where}rot.base: must be positive")
        if c.kv_rank + c.rot_dim > MAX_HEAD_DIM:        # the attention runs over [latent | rotated part]: that is its key
            raise ConfigError(f"{where}kv_rank: {c.kv_rank} + rot_dim = {c.rot_dim} exceed {MAX_HEAD_DIM}, the largest key the "
                              "attention kernels take")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale,
             "rot": {"base": self.rot_base, "dims": self.rot_dim, "scaling": self.rot_scaling.to_dict() if self.rot_scaling else None}}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d

    def cached_like(self, other: "RotatedLatentAttentionConfig") -> bool:
        """Whether what this layer caches is what `other` reads."""
        return (self.kv_rank, self.rot_dim, self.rot_base, self.rot_scaling) == (other.kv_rank, other.rot_dim, other.rot_base,
                                                                                  other.rot_scaling)


@dataclass(frozen=True)
class SatedraMLP:
    kind: str                        # "dense" | "moe"
    ff: int                          # inner width of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    identity: int = 0                # router outputs beyond the experts that stand for "the input itself"
    scale: float = 1.0               # the picks' weights are multiplied by it
    shared_ff: int = 0               # 0: no shared expert

    @staticmethod
    def from_dict(d: dict, where: str) -> "SatedraMLP":
        kind = d.get("kind")
        if kind == "dense":
            return SatedraMLP("dense", _integer(d, where, "ff"))
        if kind != "moe":
            raise ConfigError(f"{where}kind: '{kind}' is not supported (known: dense, moe)")
        router = _object(d, where, "router")
        shared = d.get("shared")
        if shared is not None and not isinstance(shared, dict):
            raise ConfigError(f"{where}shared: expected an object or null")
        c = SatedraMLP("moe", _integer(_object(d, where, "expert"), where + "expert.", "ff"),
                       _integer(router, where + "router.", "experts"), _integer(router, where + "router.", "top"),
                       _integer(router, where + "router.", "identity", 0, least=0), _number(router, where + "router.", "scale", 1.0),
                       _integer(shared, where + "shared.", "ff") if shared else 0)
        if c.top > c.experts + c.identity:
            raise ConfigError(f"{where}router.top: {c.top} exceeds the {c.experts + c.identity} router outputs")
        return c

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "router": {"experts": self.experts, "top": self.top, "identity": self.identity, "scale": self.scale},
                "expert": {"ff": self.ff}, "shared": {"ff": self.shared_ff} if self.shared_ff else None}


@dataclass(frozen=True)
class SatedraLayer:
    mixer: RotatedLatentAttentionConfig
    mlp: SatedraMLP | None           # None: the layer has no feed-forward

    @staticmethod
    def from_dict(d: dict, where: str) -> "SatedraLayer":
        if not isinstance(d, dict):
            raise ConfigError(f"{where[:-1]}: expected an object")
        if d.get("type") != "latent_attention":
            raise ConfigError(f"{where}type: '{d.get('type')}' is not a known mixer (known: latent_attention)")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}mlp: expected an object or null")
        return SatedraLayer(RotatedLatentAttentionConfig.from_dict(_object(d, where, "mixer"), where + "mixer."),
                            SatedraMLP.from_dict(mlp, where + "mlp.") if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": "latent_attention", "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class SatedraConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    torch_dtype: str = "bfloat16"
    max_position_embeddings: int | None = None       # rotary tables are laid out for what the cache holds
    bos_token_id: int | None = None
    eos_token_ids: tuple = field(default=())

    @staticmethod
    def from_dict(root: dict) -> "SatedraConfig":
        if not isinstance(root, dict):
            raise ConfigError("config.json: expected an object")
        layers = root.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("layers: expected a list of at least one layer")
        norm = root.get("norm") or {}
        eos = root.get("eos_token_id")
        cfg = SatedraConfig(
            vocab=_integer(root, "", "vocab"), width=_integer(root, "", "width"),
            layers=tuple(SatedraLayer.from_dict(l, f"layers[{i}].") for i, l in enumerate(layers)),
            norm_eps=_number(norm, "norm.", "eps", 1e-6), logit_scale=_number(root, "", "logit_scale", 1.0),
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
        for i, layer in enumerate(self.layers):
            j = layer.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < i:
                raise ConfigError(f"layers[{i}].mixer.kv_from: {j} is no earlier layer")
            if self.layers[j].mixer.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from: layer {j} keeps no latents of its own")
            if not self.layers[j].mixer.cached_like(layer.mixer):
                raise ConfigError(f"layers[{i}].mixer.kv_from: layer {j} keeps latents or rotated parts of another size or rotation")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"eos_token_id: {e} is outside the vocabulary of {self.vocab}")

    def to_dict(self) -> dict:
        d = {"architecture": "Satedra", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "logit_scale": self.logit_scale, "layers": [l.to_dict() for l in self.layers], "torch_dtype": self.torch_dtype}
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
