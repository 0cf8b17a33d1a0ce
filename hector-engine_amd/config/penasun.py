"""Typed configuration of the Penasun decoder, read from its config.json.

The file is nested: 'vocab', 'width', 'norm' {eps} and a list 'layers' whose entries give 'type'
(the mixer's kind: 'mamba2' or 'attention'), 'mixer' (its sizes and constants) and 'mlp' (the
routed feed-forward, or null for none). Every layer carries its own sizes, so layers of one model
may differ in kind, in order and in every size.

  mamba2 mixer:    heads, vdim, state, groups, conv, norm_groups
  attention mixer: heads, kv_heads, dim, vdim, scale, diff, q_temp {coef, every}
  mlp:             kind 'moe', expert {ff, limit}, router {experts, identity, top, scale,
                   groups {count, keep}}
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig, architecture_name, read_field, read_object


@dataclasses.dataclass
class PenasunScan:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    def to_dict(self) -> dict:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclasses.dataclass
class PenasunAttention:
    heads: int
    kv_heads: int
    dim: int            # of a query and of a key, per score map
    vdim: int           # of a value
    scale: float        # on q . k
    diff: float         # the constant of the two maps' difference
    q_temp_coef: float = 0.0
    q_temp_every: int = 0       # 0: no query temperature

    def to_dict(self) -> dict:
        d = {"diff": self.diff, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
             "scale": self.scale, "vdim": self.vdim}
        if self.q_temp_every:
            d["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return d


@dataclasses.dataclass
class PenasunMoE:
    ff: int
    limit: float
    experts: int        # experts with weights
    identity: int       # router outputs behind them whose expert is the identity
    top: int
    scale: float
    group_count: int
    group_keep: int

    def to_dict(self) -> dict:
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                "router": {"experts": self.experts, "groups": {"count": self.group_count, "keep": self.group_keep},
                           "identity": self.identity, "scale": self.scale, "top": self.top}}


@dataclasses.dataclass
class PenasunLayer:
    type: str
    mixer: PenasunScan | PenasunAttention
    mlp: PenasunMoE | None

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.type}


def _scan(data: dict, where: str) -> PenasunScan:
    m = PenasunScan(heads=read_field(data, "heads", int), vdim=read_field(data, "vdim", int),
                    state=read_field(data, "state", int), groups=read_field(data, "groups", int, 1),
                    conv=read_field(data, "conv", int), norm_groups=read_field(data, "norm_groups", int, 1))
    if min(m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups) <= 0:
        raise ConfigError(f"{where}: 'heads', 'vdim', 'state', 'groups', 'conv' and 'norm_groups' must be positive")
    if m.heads % m.groups:
        raise ConfigError(f"{where}: 'groups' ({m.groups}) must divide 'heads' ({m.heads})")
    if (m.heads * m.vdim) % m.norm_groups:
        raise ConfigError(f"{where}: 'norm_groups' ({m.norm_groups}) must divide heads * vdim ({m.heads * m.vdim})")
    return m


def _attention(data: dict, where: str) -> PenasunAttention:
    heads = read_field(data, "heads", int)
    dim = read_field(data, "dim", int)
    qt = read_object(data, "q_temp", None)
    a = PenasunAttention(heads=heads, kv_heads=read_field(data, "kv_heads", int, heads), dim=dim,
                         vdim=read_field(data, "vdim", int, dim), scale=read_field(data, "scale", float),
                         diff=read_field(data, "diff", float),
                         q_temp_coef=0.0 if qt is None else read_field(qt, "coef", float),
                         q_temp_every=0 if qt is None else read_field(qt, "every", int))
    if min(a.heads, a.kv_heads, a.dim, a.vdim) <= 0:
        raise ConfigError(f"{where}: 'heads', 'kv_heads', 'dim' and 'vdim' must be positive")
    if a.heads % a.kv_heads:
        raise ConfigError(f"{where}: 'kv_heads' ({a.kv_heads}) must divide 'heads' ({a.heads})")
    if a.scale <= 0:
        raise ConfigError(f"{where}: 'scale' must be positive")
    if qt is not None and a.q_temp_every <= 0:
        raise ConfigError(f"{where}: 'q_temp.every' must be positive")
    return a


def _moe(data: dict, where: str) -> PenasunMoE:
    kind = read_field(data, "kind", str, "moe")
    if kind != "moe":
        raise ConfigError(f"{where}: unknown kind '{kind}'")
    expert = read_object(data, "expert")
    router = read_object(data, "router")
    groups = read_object(router, "groups", None) or {}
    m = PenasunMoE(ff=read_field(expert, "ff", int), limit=read_field(expert, "limit", float),
                   experts=read_field(router, "experts", int), identity=read_field(router, "identity", int, 0),
                   top=read_field(router, "top", int), scale=read_field(router, "scale", float, 1.0),
                   group_count=read_field(groups, "count", int, 1), group_keep=read_field(groups, "keep", int, 0))
    if m.group_keep == 0:
        m.group_keep = m.group_count
    outputs = m.experts + m.identity
    if m.ff <= 0 or m.limit <= 0 or m.experts <= 0 or m.identity < 0:
        raise ConfigError(f"{where}: 'expert.ff', 'expert.limit' and 'router.experts' must be positive, "
                          "'router.identity' not negative")
    if m.group_count <= 0 or outputs % m.group_count or not 0 < m.group_keep <= m.group_count:
        raise ConfigError(f"{where}: the {outputs} router outputs must form 'groups.count' ({m.group_count}) equal "
                          f"groups of which 'groups.keep' ({m.group_keep}) are kept")
    if not 0 < m.top <= m.group_keep * (outputs // m.group_count):
        raise ConfigError(f"{where}: 'router.top' ({m.top}) must be positive and at most the "
                          f"{m.group_keep * (outputs // m.group_count)} outputs of the kept groups")
    return m


@dataclasses.dataclass
class PenasunConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: list = dataclasses.field(default_factory=list)
    norm_eps: float = 1e-6
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, data: dict) -> "PenasunConfig":
        raw_layers = data.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"config key 'layers[{i}]'"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}: expected an object")
            kind = read_field(entry, "type", str)
            if kind == "mamba2":
                mixer = _scan(read_object(entry, "mixer"), where + ".mixer")
            elif kind == "attention":
                mixer = _attention(read_object(entry, "mixer"), where + ".mixer")
            else:
                raise ConfigError(f"{where}: unknown mixer type '{kind}'")
            raw_mlp = read_object(entry, "mlp", None)
            layers.append(PenasunLayer(kind, mixer, None if raw_mlp is None else _moe(raw_mlp, where + ".mlp")))
        cfg = cls(architecture=architecture_name(data), vocab=read_field(data, "vocab", int),
                  width=read_field(data, "width", int), layers=layers,
                  norm_eps=read_field(read_object(data, "norm", None) or {}, "eps", float, 1e-6))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config keys 'vocab' and 'width' must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("config key 'norm.eps' must be positive")

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
