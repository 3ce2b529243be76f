"""Typed configuration of the Domorax decoder, read from its config.json.

The file is nested: 'vocab', 'width', 'residual_mult', 'norm' {eps, groups} and a list 'layers' whose entries
give 'type' (the mixer's kind: 'latent_attention', 'attention' or 'delta'), 'mixer' (its sizes and constants)
and 'mlp' (the feed-forward, or null for none). Every layer carries its own sizes, so layers of one model may
differ in kind, in order and in every size.

  latent_attention: heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, mask {size} (or none: every earlier
                    position), rot {base, dims, scaling {factor, original, fast, slow} (or none)}
  attention:        heads, kv_heads, dim, vdim, conv, scale
  delta:            heads, kv_heads, dim, vdim, conv
  mlp:              kind 'dense' {ff}, or kind 'moe' {expert {ff}, router {experts, top}, shared {ff} (or none)}
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig, architecture_name, read_field, read_object


@dataclasses.dataclass
class DomoraxLatent:
    heads: int
    dim: int            # unrotated dims of a head's query and key
    rot_dim: int        # rotated dims
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    window: int = 0             # 0: every earlier position
    rot_base: float = 10000.0
    rot_dims: int = 0
    rot_scaling: dict | None = None

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
             "rot": {"base": self.rot_base, "dims": self.rot_dims}, "rot_dim": self.rot_dim, "scale": self.scale,
             "vdim": self.vdim}
        if self.rot_scaling:
            d["rot"]["scaling"] = dict(self.rot_scaling)
        if self.window:
            d["mask"] = {"size": self.window}
        return d


@dataclasses.dataclass
class DomoraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float

    def to_dict(self) -> dict:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                "vdim": self.vdim}


@dataclasses.dataclass
class DomoraxDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    def to_dict(self) -> dict:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclasses.dataclass
class DomoraxMLP:
    kind: str                   # 'dense' or 'moe'
    ff: int = 0                 # dense: the intermediate width; moe: an expert's
    experts: int = 0
    top: int = 0
    shared_ff: int = 0          # 0: no shared expert

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        d = {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclasses.dataclass
class DomoraxLayer:
    type: str
    mixer: DomoraxLatent | DomoraxAttention | DomoraxDelta
    mlp: DomoraxMLP | None

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


def _positive(where: str, **values) -> None:
    for key, v in values.items():
        if v <= 0:
            raise ConfigError(f"config key '{where}.{key}' must be positive, got {v}")


def _mixer(where: str, kind: str, m: dict):
    if kind == "latent_attention":
        rot = read_object(m, "rot", {})
        mask = read_object(m, "mask", {})
        rot_dim = read_field(m, "rot_dim", int, 0)
        out = DomoraxLatent(
            heads=read_field(m, "heads", int), dim=read_field(m, "dim", int), rot_dim=rot_dim,
            vdim=read_field(m, "vdim", int), kv_rank=read_field(m, "kv_rank", int), q_rank=read_field(m, "q_rank", int),
            scale=read_field(m, "scale", float), window=read_field(mask, "size", int, 0),
            rot_base=read_field(rot, "base", float, 10000.0), rot_dims=read_field(rot, "dims", int, rot_dim),
            rot_scaling=read_object(rot, "scaling", None))
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, kv_rank=out.kv_rank, q_rank=out.q_rank)
        if out.rot_dim < 0 or out.rot_dim % 2 or out.rot_dims != out.rot_dim:
            raise ConfigError(f"config key '{where}.rot_dim' must be even and equal to rot.dims, got {out.rot_dim} and {out.rot_dims}")
        if out.window < 0:
            raise ConfigError(f"config key '{where}.mask.size' must not be negative")
        if out.rot_scaling is not None:
            for key in ("factor", "original", "fast", "slow"):
                read_field(out.rot_scaling, key, float)
        return out
    if kind == "attention":
        out = DomoraxAttention(heads=read_field(m, "heads", int), kv_heads=read_field(m, "kv_heads", int),
                               dim=read_field(m, "dim", int), vdim=read_field(m, "vdim", int),
                               conv=read_field(m, "conv", int), scale=read_field(m, "scale", float))
        _positive(where, heads=out.heads, kv_heads=out.kv_heads, dim=out.dim, conv=out.conv)
        if out.vdim != out.dim:
            raise ConfigError(f"config key '{where}.vdim' must equal dim (the values are the keys), got {out.vdim} and {out.dim}")
    elif kind == "delta":
        out = DomoraxDelta(heads=read_field(m, "heads", int), kv_heads=read_field(m, "kv_heads", int),
                           dim=read_field(m, "dim", int), vdim=read_field(m, "vdim", int), conv=read_field(m, "conv", int))
        _positive(where, heads=out.heads, kv_heads=out.kv_heads, dim=out.dim, vdim=out.vdim, conv=out.conv)
    else:
        raise ConfigError(f"config key '{where[:-6]}.type': unknown mixer '{kind}'")
    if out.heads % out.kv_heads:
        raise ConfigError(f"config key '{where}.heads' ({out.heads}) must be a multiple of kv_heads ({out.kv_heads})")
    return out


def _mlp(where: str, m: dict | None):
    if m is None:
        return None
    kind = read_field(m, "kind", str)
    if kind == "dense":
        out = DomoraxMLP("dense", ff=read_field(m, "ff", int))
        _positive(where, ff=out.ff)
        return out
    if kind != "moe":
        raise ConfigError(f"config key '{where}.kind': unknown feed-forward '{kind}'")
    router, shared = read_object(m, "router"), read_object(m, "shared", None)
    out = DomoraxMLP("moe", ff=read_field(read_object(m, "expert"), "ff", int), experts=read_field(router, "experts", int),
                     top=read_field(router, "top", int), shared_ff=read_field(shared, "ff", int) if shared else 0)
    _positive(where, ff=out.ff, experts=out.experts, top=out.top)
    if out.top > out.experts:
        raise ConfigError(f"config key '{where}.router.top' ({out.top}) exceeds the {out.experts} experts")
    return out


@dataclasses.dataclass
class DomoraxConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    residual_mult: float = 1.0
    norm_eps: float = 1e-6
    norm_groups: int = 1
    layers: list = dataclasses.field(default_factory=list)
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_dict(cls, data: dict) -> "DomoraxConfig":
        norm = read_object(data, "norm")
        raw = data.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw):
            if not isinstance(entry, dict):
                raise ConfigError(f"config key 'layers[{i}]': expected an object")
            kind = read_field(entry, "type", str)
            layers.append(DomoraxLayer(kind, _mixer(f"layers[{i}].mixer", kind, read_object(entry, "mixer")),
                                       _mlp(f"layers[{i}].mlp", read_object(entry, "mlp", None))))
        cfg = cls(architecture=architecture_name(data), vocab=read_field(data, "vocab", int),
                  width=read_field(data, "width", int), residual_mult=read_field(data, "residual_mult", float, 1.0),
                  norm_eps=read_field(norm, "eps", float), norm_groups=read_field(norm, "groups", int, 1), layers=layers,
                  torch_dtype=read_field(data, "torch_dtype", str, "bfloat16"))
        if cfg.vocab <= 0 or cfg.width <= 0:
            raise ConfigError("config keys 'vocab' and 'width' must be positive")
        if cfg.norm_groups <= 0 or cfg.width % cfg.norm_groups:
            raise ConfigError(f"config key 'norm.groups' ({cfg.norm_groups}) must divide 'width' ({cfg.width})")
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "residual_mult": self.residual_mult,
                "torch_dtype": self.torch_dtype, "vocab": self.vocab, "width": self.width}
