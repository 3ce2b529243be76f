"""Typed configuration of the Butolorn decoder, read from its config.json.

The file is nested: 'vocab', 'width', 'norm' {eps}, 'embedding' {scale}, 'token_side' {dim},
'loop' {start, stop, times} and a list 'layers' whose entries give 'type' (the mixer's kind:
'attention' or 'parallel'), 'mixer' (its sizes and constants) and 'mlp' (the feed-forward, or null
for none). Every layer carries its own sizes, so layers of one model may differ in kind, in order
and in every size.

  attention mixer: heads, kv_heads, dim, vdim, scale, rot {base, dims}
  parallel mixer:  left (an attention mixer's keys), right {heads, dim, vdim, gate_cap},
                   left_scale, right_scale
  mlp:             kind 'dense', ff
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig, architecture_name, read_field, read_object


@dataclasses.dataclass
class ButolornAttention:
    heads: int
    kv_heads: int
    dim: int            # of a query and of a key
    vdim: int           # of a value
    scale: float        # on q . k
    rot_base: float = 0.0
    rot_dims: int = 0   # 0: no rotation

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return d


@dataclasses.dataclass
class ButolornMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def to_dict(self) -> dict:
        return {"dim": self.dim, "gate_cap": self.gate_cap, "heads": self.heads, "vdim": self.vdim}


@dataclasses.dataclass
class ButolornParallel:
    left: ButolornAttention
    right: ButolornMemory
    left_scale: float
    right_scale: float

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclasses.dataclass
class ButolornMLP:
    ff: int
    kind: str = "dense"

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": self.kind}


@dataclasses.dataclass
class ButolornLayer:
    type: str
    mixer: ButolornAttention | ButolornParallel
    mlp: ButolornMLP | None

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.type}


def _attention(data: dict, where: str) -> ButolornAttention:
    heads = read_field(data, "heads", int)
    dim = read_field(data, "dim", int)
    rot = read_object(data, "rot", None)
    if rot is not None and read_field(rot, "dims", int, dim) == 0:
        rot = None          # no dimension is rotated
    a = ButolornAttention(heads=heads, kv_heads=read_field(data, "kv_heads", int, heads), dim=dim,
                          vdim=read_field(data, "vdim", int, dim), scale=read_field(data, "scale", float),
                          rot_base=0.0 if rot is None else read_field(rot, "base", float),
                          rot_dims=0 if rot is None else read_field(rot, "dims", int, dim))
    if min(a.heads, a.kv_heads, a.dim, a.vdim) <= 0:
        raise ConfigError(f"{where}: 'heads', 'kv_heads', 'dim' and 'vdim' must be positive")
    if a.heads % a.kv_heads:
        raise ConfigError(f"{where}: 'kv_heads' ({a.kv_heads}) must divide 'heads' ({a.heads})")
    if a.scale <= 0:
        raise ConfigError(f"{where}: 'scale' must be positive")
    if rot is not None:
        if a.rot_dims <= 0 or a.rot_dims % 2 or a.rot_dims > a.dim:
            raise ConfigError(f"{where}: 'rot.dims' ({a.rot_dims}) must be even, positive and at most 'dim' ({a.dim})")
        if a.rot_base <= 1:
            raise ConfigError(f"{where}: 'rot.base' must exceed 1")
    return a


def _memory(data: dict, where: str) -> ButolornMemory:
    dim = read_field(data, "dim", int)
    m = ButolornMemory(heads=read_field(data, "heads", int), dim=dim, vdim=read_field(data, "vdim", int, dim),
                       gate_cap=read_field(data, "gate_cap", float))
    if min(m.heads, m.dim, m.vdim) <= 0 or m.gate_cap <= 0:
        raise ConfigError(f"{where}: 'heads', 'dim', 'vdim' and 'gate_cap' must be positive")
    if m.dim > 512:
        raise ConfigError(f"{where}: 'dim' ({m.dim}) above 512")
    return m


@dataclasses.dataclass
class ButolornConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: list = dataclasses.field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    side_dim: int = 0           # columns of the second embedding table a layer reads; 0: no token input
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, data: dict) -> "ButolornConfig":
        raw_layers = data.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"config key 'layers[{i}]'"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}: expected an object")
            kind = read_field(entry, "type", str)
            raw = read_object(entry, "mixer")
            if kind == "attention":
                mixer = _attention(raw, where + ".mixer")
            elif kind == "parallel":
                mixer = ButolornParallel(left=_attention(read_object(raw, "left"), where + ".mixer.left"),
                                         right=_memory(read_object(raw, "right"), where + ".mixer.right"),
                                         left_scale=read_field(raw, "left_scale", float, 1.0),
                                         right_scale=read_field(raw, "right_scale", float, 1.0))
            else:
                raise ConfigError(f"{where}: unknown mixer type '{kind}'")
            raw_mlp = read_object(entry, "mlp", None)
            mlp = None
            if raw_mlp is not None:
                mlp = ButolornMLP(ff=read_field(raw_mlp, "ff", int), kind=read_field(raw_mlp, "kind", str, "dense"))
                if mlp.kind != "dense":
                    raise ConfigError(f"{where}.mlp: unknown kind '{mlp.kind}'")
                if mlp.ff <= 0:
                    raise ConfigError(f"{where}.mlp: 'ff' must be positive")
            layers.append(ButolornLayer(kind, mixer, mlp))
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
            embedding_scale=read_field(read_object(data, "embedding", None) or {}, "scale", float, 1.0),
            side_dim=read_field(read_object(data, "token_side", None) or {}, "dim", int, 0),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("config keys 'vocab' and 'width' must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("config key 'norm.eps' must be positive")
        if self.side_dim < 0:
            raise ConfigError("config key 'token_side.dim' must not be negative")
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
        d = {
            "architecture": self.architecture,
            "embedding": {"scale": self.embedding_scale},
            "layers": [l.to_dict() for l in self.layers],
            "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times},
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab,
            "width": self.width,
        }
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        return d
