"""Nenotar's typed configuration, read from its own config.json keys.

A decoder whose layers are listed one by one: each has a mixer ("latent_attention": softmax attention over one cached
latent a token; "mingru": a gated element-wise recurrence) and an optional dense feed-forward, both reading the same
input; every layer also takes a per-layer token input from a second table.  config.json gives every size and every
constant that differs between models of the design:

  architecture "Nenotar"; vocab; width; embedding.scale; norm.eps; token_side.dim (optional); layers[]: type, mixer
  (latent_attention: heads, dim, rot_dim, vdim, kv_rank, scale, rot {base, dims, scaling {factor, original, fast, slow}};
  mingru: width), mlp (null | {kind "dense", ff}).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .reader import ConfigError, KeyReader

ARCHITECTURE = "Nenotar"
LAYER_TYPES = ("latent_attention", "mingru")


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[RotaryScaling] = None


@dataclass(frozen=True)
class MinGRUConfig:
    width: int


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any                      # LatentAttentionConfig | MinGRUConfig
    ff: Optional[int] = None        # the dense feed-forward's inner width; None: the layer has none


@dataclass(frozen=True)
class NenotarConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[LayerConfig, ...]
    token_side_dim: Optional[int] = None

    architecture = ARCHITECTURE

    def __post_init__(self):
        object.__setattr__(self, "layers", tuple(self.layers))
        check(self)

    # -- reading ----------------------------------------------------------
    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "NenotarConfig":
        r = KeyReader(values)
        name = r.raw("architecture")
        if name != ARCHITECTURE:
            raise r.unsupported("architecture", f"{name!r}; expected {ARCHITECTURE!r}")
        emb = r.child("embedding")
        scale = emb.real("scale")
        emb.finish((), ARCHITECTURE)
        norm = r.child("norm")
        eps = norm.real("eps", lo=0.0)
        norm.finish((), ARCHITECTURE)
        side = r.child("token_side", required=False)
        side_dim = None
        if side is not None:
            side_dim = side.integer("dim")
            side.finish((), ARCHITECTURE)
        raw_layers = r.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise r.unsupported("layers", "a list of at least one layer is expected")
        layers = tuple(_read_layer(entry, i) for i, entry in enumerate(raw_layers))
        cfg = cls(vocab=r.integer("vocab"), width=r.integer("width"), embedding_scale=scale, norm_eps=eps, layers=layers,
                  token_side_dim=side_dim)
        r.finish((), ARCHITECTURE)
        return cfg

    @property
    def vocab_size(self) -> int:
        """The vocabulary under the name the command line asks every configuration for."""
        return self.vocab

    def to_json(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "latent_attention":
                rot: Dict[str, Any] = {"base": m.rot_base, "dims": m.rot_dims}
                if m.rot_scaling is not None:
                    s = m.rot_scaling
                    rot["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "rot": rot}
            else:
                mixer = {"width": m.width}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
               "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.token_side_dim is not None:
            out["token_side"] = {"dim": self.token_side_dim}
        return out


def _read_layer(entry, i: int) -> LayerConfig:
    r = KeyReader(entry, where=f"layers[{i}]")
    kind = r.choice("type", LAYER_TYPES)
    m = r.child("mixer")
    if kind == "latent_attention":
        rot = m.child("rot")
        sc = rot.child("scaling", required=False)
        scaling = None
        if sc is not None:
            scaling = RotaryScaling(factor=sc.real("factor", positive=True), original=sc.real("original", positive=True),
                                    fast=sc.real("fast", positive=True), slow=sc.real("slow", positive=True))
            sc.finish((), ARCHITECTURE)
        mixer = LatentAttentionConfig(heads=m.integer("heads"), dim=m.integer("dim"), rot_dim=m.integer("rot_dim", lo=0), vdim=m.integer("vdim"),
                                      kv_rank=m.integer("kv_rank"), scale=m.real("scale", positive=True),
                                      rot_base=rot.real("base", positive=True), rot_dims=rot.integer("dims", lo=0), rot_scaling=scaling)
        rot.finish((), ARCHITECTURE)
    else:
        mixer = MinGRUConfig(width=m.integer("width"))
    m.finish((), ARCHITECTURE)
    mlp = r.child("mlp", required=False)
    ff = None
    if mlp is not None:
        mlp.choice("kind", ("dense",))
        ff = mlp.integer("ff")
        mlp.finish((), ARCHITECTURE)
    r.finish((), ARCHITECTURE)
    return LayerConfig(kind, mixer, ff)


def check(c: NenotarConfig) -> None:
    """The rules a configuration keeps wherever it came from."""
    def bad(key, why):
        return ConfigError(f"config: unsupported value for {key} ({why})")
    if c.vocab < 1 or c.width < 1:
        raise bad("width", "vocab and width are at least 1")
    if not c.layers:
        raise bad("layers", "at least one layer")
    if c.token_side_dim is not None and c.token_side_dim < 1:
        raise bad("token_side.dim", "at least 1")
    for i, layer in enumerate(c.layers):
        if layer.type not in LAYER_TYPES:
            raise bad(f"layers[{i}].type", f"{layer.type!r}; this engine computes {list(LAYER_TYPES)}")
        m = layer.mixer
        if layer.type == "latent_attention":
            if not isinstance(m, LatentAttentionConfig):
                raise bad(f"layers[{i}].mixer", "not the sizes of latent attention")
            if m.rot_dims % 2 or m.rot_dims > m.rot_dim:
                raise bad(f"layers[{i}].mixer.rot.dims", "the rotated dims are even and at most rot_dim")
            if m.rot_base <= 1.0 and m.rot_dims:
                raise bad(f"layers[{i}].mixer.rot.base", "above 1")
        elif not isinstance(m, MinGRUConfig):
            raise bad(f"layers[{i}].mixer", "not the sizes of a minGRU")
        if layer.ff is not None and layer.ff < 1:
            raise bad(f"layers[{i}].mlp.ff", "at least 1")
