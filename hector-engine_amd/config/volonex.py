"""Typed configuration of the Volonex decoder, read from its config.json.

The file is nested: 'vocab', 'width', 'residual_mult', 'embedding' {scale}, 'norm' {eps},
'loop' {start, stop, times} and a list 'layers' whose entries give 'type' (the mixer's kind),
'mixer' (its sizes and constants) and 'mlp' (the feed-forward, or null for none). Every layer
carries its own sizes, so layers of one model may differ. A key that a layer leaves out switches
its mechanism off: no 'mask' is plain causal attention, no 'rot' no rotation, no 'scaling' the
unscaled frequencies, no 'loop' a single pass.
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig, architecture_name, read_field, read_object


@dataclasses.dataclass
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self) -> dict:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclasses.dataclass
class VolonexRotary:
    base: float
    dims: int
    scaling: RotaryScaling | None = None

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclasses.dataclass
class VolonexAttention:
    heads: int
    kv_heads: int
    dim: int            # of a query and of a key
    vdim: int           # of a value
    scale: float        # on q . k
    chunk: int = 0      # mask.size: a query sees its own chunk only (0: every earlier key)
    rot: VolonexRotary | None = None

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
             "vdim": self.vdim}
        if self.chunk:
            d["mask"] = {"size": self.chunk}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclasses.dataclass
class VolonexMLP:
    kind: str
    ff: int
    limit: float

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": self.kind, "limit": self.limit}


@dataclasses.dataclass
class VolonexLayer:
    type: str
    mixer: VolonexAttention
    mlp: VolonexMLP | None

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.type}


def _attention(data: dict, where: str) -> VolonexAttention:
    heads = read_field(data, "heads", int)
    dim = read_field(data, "dim", int)
    mask = read_object(data, "mask", None)
    rot = read_object(data, "rot", None)
    rotary = None
    if rot is not None:
        sc = read_object(rot, "scaling", None)
        scaling = None if sc is None else RotaryScaling(
            factor=read_field(sc, "factor", float), original=read_field(sc, "original", float),
            fast=read_field(sc, "fast", float), slow=read_field(sc, "slow", float))
        rotary = VolonexRotary(base=read_field(rot, "base", float), dims=read_field(rot, "dims", int),
                               scaling=scaling)
    a = VolonexAttention(heads=heads, kv_heads=read_field(data, "kv_heads", int, heads), dim=dim,
                         vdim=read_field(data, "vdim", int, dim), scale=read_field(data, "scale", float),
                         chunk=0 if mask is None else read_field(mask, "size", int), rot=rotary)
    if min(a.heads, a.kv_heads, a.dim, a.vdim) <= 0:
        raise ConfigError(f"{where}: 'heads', 'kv_heads', 'dim' and 'vdim' must be positive")
    if a.heads % a.kv_heads:
        raise ConfigError(f"{where}: 'kv_heads' ({a.kv_heads}) must divide 'heads' ({a.heads})")
    if a.chunk < 0 or (mask is not None and a.chunk == 0):
        raise ConfigError(f"{where}: 'mask.size' must be positive")
    if a.scale <= 0:
        raise ConfigError(f"{where}: 'scale' must be positive")
    if rotary is not None:
        if rotary.dims <= 0 or rotary.dims % 2 or rotary.dims > a.dim:
            raise ConfigError(f"{where}: 'rot.dims' ({rotary.dims}) must be even, positive and at most 'dim' ({a.dim})")
        if rotary.base <= 1:
            raise ConfigError(f"{where}: 'rot.base' must exceed 1")
        s = rotary.scaling
        if s is not None and (s.factor <= 0 or s.original <= 0 or s.fast <= 0 or s.slow <= 0):
            raise ConfigError(f"{where}: 'rot.scaling' needs positive factor, original, fast and slow")
    return a


@dataclasses.dataclass
class VolonexConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: list = dataclasses.field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    embedding_scale: float = 1.0
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, data: dict) -> "VolonexConfig":
        raw_layers = data.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"config key 'layers[{i}]'"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}: expected an object")
            kind = read_field(entry, "type", str)
            if kind != "attention":
                raise ConfigError(f"{where}: unknown mixer type '{kind}'")
            mixer = _attention(read_object(entry, "mixer"), where + ".mixer")
            raw_mlp = read_object(entry, "mlp", None)
            mlp = None
            if raw_mlp is not None:
                mlp = VolonexMLP(kind=read_field(raw_mlp, "kind", str, "dense"), ff=read_field(raw_mlp, "ff", int),
                                 limit=read_field(raw_mlp, "limit", float))
                if mlp.kind != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind '{mlp.kind}'")
                if mlp.ff <= 0 or mlp.limit <= 0:
                    raise ConfigError(f"{where}.mlp: 'ff' and 'limit' must be positive")
            layers.append(VolonexLayer(kind, mixer, mlp))
        loop = read_object(data, "loop", None) or {}
        cfg = cls(
            architecture=architecture_name(data),
            vocab=read_field(data, "vocab", int),
            width=read_field(data, "width", int),
            layers=layers,
            loop_start=read_field(loop, "start", int, 0),
            loop_stop=read_field(loop, "stop", int, 0),
            loop_times=read_field(loop, "times", int, 1),
            norm_eps=read_field(read_object(data, "norm", None) or {}, "eps", float, 1e-6),
            residual_mult=read_field(data, "residual_mult", float, 1.0),
            embedding_scale=read_field(read_object(data, "embedding", None) or {}, "scale", float, 1.0),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config keys 'vocab' and 'width' must be positive")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers):
            raise ConfigError(f"config key 'loop': start {self.loop_start} and stop {self.loop_stop} must lie "
                              f"in order within the {len(self.layers)} layers")
        if self.loop_times < 1:
            raise ConfigError("config key 'loop.times' must be at least 1")

    def runs(self) -> list[tuple[int, bool]]:
        """The layers in the order they run, as (layer, first of a repeated pass): the layers
        start .. stop-1 run `times` times in a row with the same weights, the others once."""
        order = [(l, False) for l in range(self.loop_start)]
        for t in range(self.loop_times if self.loop_stop > self.loop_start else 0):
            order += [(l, t > 0 and l == self.loop_start) for l in range(self.loop_start, self.loop_stop)]
        return order + [(l, False) for l in range(self.loop_stop, len(self.layers))]

    def to_dict(self) -> dict:
        return {
            "architecture": self.architecture,
            "embedding": {"scale": self.embedding_scale},
            "layers": [l.to_dict() for l in self.layers],
            "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times},
            "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult,
            "vocab": self.vocab,
            "width": self.width,
        }
