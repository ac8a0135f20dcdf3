"""Bonerax's typed configuration, read from its own config.json keys.

A decoder whose layers are listed one by one.  A layer norms each sublayer's result (layer norm with a weight) on its way
into the residual; its mixer is "gla" (gated linear attention), "channel_delta" (a gated delta rule with a decay a key
channel) or "parallel" (windowed softmax attention and such a delta rule side by side, their weighted sum); its
feed-forward is a dense SwiGLU, routed SwiGLU experts, or absent.  A layer with `weights_of: j` runs layer j's tensors
with a cache of its own.  config.json gives every size and every constant that differs between models of the design:

  architecture "Bonerax"; vocab; width; norm.eps; logit_scale; logit_softcap; layers[]: type, weights_of (optional), mixer
  (gla: heads, dim, vdim, tau; channel_delta: heads, kv_heads, dim, vdim, conv; parallel: left {heads, kv_heads, dim, vdim,
  scale, mask {size}, rot {base, dims, scaling {factor, original, fast, slow}}}, right (as channel_delta), left_scale,
  right_scale), mlp (null | {kind "dense", ff} | {kind "moe", expert {ff}, router {experts, top}}).

Inner widths of the low-rank projections (the decays' and gates') are not in config.json: the tensors' shapes give them.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .nenotar import RotaryScaling
from .reader import ConfigError, KeyReader

ARCHITECTURE = "Bonerax"
#: keys a model folder's config.json may carry that say nothing about the arithmetic (how the folder was made, what it is
#: called, how its file stores numbers: the loader reads the stored type from the file itself)
WITHOUT_EFFECT = ("name", "seed", "comment", "description", "dtype", "torch_dtype")
LAYER_TYPES = ("gla", "channel_delta", "parallel")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class GLAConfig:
    heads: int
    dim: int
    vdim: int
    tau: float


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[RotaryScaling] = None


@dataclass(frozen=True)
class ParallelConfig:
    left: WindowAttentionConfig
    right: DeltaConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class MLPConfig:
    kind: str                       # "dense" | "moe"
    ff: int                         # inner width (of one expert for "moe")
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any                      # GLAConfig | DeltaConfig | ParallelConfig
    mlp: Optional[MLPConfig] = None
    weights_of: Optional[int] = None


@dataclass(frozen=True)
class BoneraxConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    logit_softcap: Optional[float]
    layers: Tuple[LayerConfig, ...]
    #: inner widths of the low-rank projections by layer, read from the tensors' shapes when a model folder is opened
    #: ({layer: {"decay": r, "gate": r}}); a configuration made in code states them here
    ranks: Optional[Mapping[int, Mapping[str, int]]] = None

    architecture = ARCHITECTURE

    def __post_init__(self):
        object.__setattr__(self, "layers", tuple(self.layers))
        check(self)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "BoneraxConfig":
        r = KeyReader(values)
        name = r.raw("architecture")
        if name != ARCHITECTURE:
            raise r.unsupported("architecture", f"{name!r}; expected {ARCHITECTURE!r}")
        norm = r.child("norm")
        eps = norm.real("eps", lo=0.0)
        norm.finish((), ARCHITECTURE)
        raw_layers = r.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise r.unsupported("layers", "a list of at least one layer is expected")
        layers = tuple(_read_layer(entry, i) for i, entry in enumerate(raw_layers))
        cap = r.real("logit_softcap", default=None, positive=True)
        ranks = r.raw("ranks", None)
        cfg = cls(vocab=r.integer("vocab"), width=r.integer("width"), norm_eps=eps, logit_scale=r.real("logit_scale", default=1.0),
                  logit_softcap=cap, layers=layers,
                  ranks=None if ranks is None else {int(k): {str(a): int(b) for a, b in v.items()} for k, v in ranks.items()})
        r.finish(WITHOUT_EFFECT, ARCHITECTURE)
        return cfg

    @property
    def vocab_size(self) -> int:
        """The vocabulary under the name the command line asks every configuration for."""
        return self.vocab

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "BoneraxConfig":
        """The configuration with the sizes that only the tensors' shapes give (the low-rank projections' inner widths),
        read from {tensor name: shape}; a tensor that is not there leaves its size open, and the weights check names it."""
        from dataclasses import replace
        ranks: Dict[int, Dict[str, int]] = {}
        for i, layer in enumerate(self.layers):
            if layer.weights_of is not None:
                continue
            p = f"l{i}.mix." + ("right." if layer.type == "parallel" else "")
            found = {}
            for key, tensor in (("decay", "a1"), ("gate", "g1")):
                shape = shapes.get(p + tensor)
                if shape is not None and len(shape) == 2:
                    found[key] = int(shape[0])
            ranks[i] = found
        return replace(self, ranks=ranks)

    def rank(self, i: int, key: str) -> int:
        """The inner width `key` ("decay" | "gate") of layer i's low-rank projection."""
        try:
            return int(self.ranks[self.owner(i)][key])
        except (KeyError, TypeError):
            raise ConfigError(f"config: the inner width of layers[{i}]'s {key} projection is not known: config.json does not hold it "
                              f"(the tensors' shapes do; a configuration made without a model folder states `ranks`)") from None

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs."""
        j = self.layers[i].weights_of
        return i if j is None else j

    def to_json(self) -> dict:
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "logit_scale": self.logit_scale, "layers": [_layer_json(layer) for layer in self.layers]}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.ranks is not None:
            out["ranks"] = {str(k): dict(v) for k, v in self.ranks.items()}
        return out


def _read_delta(m: KeyReader) -> DeltaConfig:
    return DeltaConfig(heads=m.integer("heads"), kv_heads=m.integer("kv_heads"), dim=m.integer("dim"), vdim=m.integer("vdim"),
                       conv=m.integer("conv"))


def _read_window_attention(m: KeyReader) -> WindowAttentionConfig:
    mask = m.child("mask")
    window = mask.integer("size")
    mask.finish((), ARCHITECTURE)
    rot = m.child("rot")
    sc = rot.child("scaling", required=False)
    scaling = None
    if sc is not None:
        scaling = RotaryScaling(factor=sc.real("factor", positive=True), original=sc.real("original", positive=True),
                                fast=sc.real("fast", positive=True), slow=sc.real("slow", positive=True))
        sc.finish((), ARCHITECTURE)
    cfg = WindowAttentionConfig(heads=m.integer("heads"), kv_heads=m.integer("kv_heads"), dim=m.integer("dim"), vdim=m.integer("vdim"),
                                scale=m.real("scale", positive=True), window=window, rot_base=rot.real("base", positive=True),
                                rot_dims=rot.integer("dims", lo=0), rot_scaling=scaling)
    rot.finish((), ARCHITECTURE)
    return cfg


def _read_layer(entry, i: int) -> LayerConfig:
    r = KeyReader(entry, where=f"layers[{i}]")
    kind = r.choice("type", LAYER_TYPES)
    m = r.child("mixer")
    if kind == "gla":
        mixer = GLAConfig(heads=m.integer("heads"), dim=m.integer("dim"), vdim=m.integer("vdim"), tau=m.real("tau", positive=True))
    elif kind == "channel_delta":
        mixer = _read_delta(m)
    else:
        left, right = m.child("left"), m.child("right")
        mixer = ParallelConfig(left=_read_window_attention(left), right=_read_delta(right), left_scale=m.real("left_scale"),
                               right_scale=m.real("right_scale"))
        left.finish((), ARCHITECTURE)
        right.finish((), ARCHITECTURE)
    m.finish((), ARCHITECTURE)
    mlp = r.child("mlp", required=False)
    ff = None
    if mlp is not None:
        if mlp.choice("kind", MLP_KINDS) == "dense":
            ff = MLPConfig("dense", mlp.integer("ff"))
        else:
            expert, router = mlp.child("expert"), mlp.child("router")
            ff = MLPConfig("moe", expert.integer("ff"), experts=router.integer("experts"), top=router.integer("top"))
            expert.finish((), ARCHITECTURE)
            router.finish((), ARCHITECTURE)
        mlp.finish((), ARCHITECTURE)
    weights_of = r.integer("weights_of", lo=0, default=None)
    r.finish(("name", "comment"), ARCHITECTURE)
    return LayerConfig(kind, mixer, ff, weights_of)


def _delta_json(m: DeltaConfig) -> dict:
    return {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}


def _layer_json(layer: LayerConfig) -> dict:
    m = layer.mixer
    if layer.type == "gla":
        mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau}
    elif layer.type == "channel_delta":
        mixer = _delta_json(m)
    else:
        a = m.left
        rot: Dict[str, Any] = {"base": a.rot_base, "dims": a.rot_dims}
        if a.rot_scaling is not None:
            s = a.rot_scaling
            rot["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
        mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                          "mask": {"size": a.window}, "rot": rot},
                 "right": _delta_json(m.right), "left_scale": m.left_scale, "right_scale": m.right_scale}
    if layer.mlp is None:
        mlp = None
    elif layer.mlp.kind == "dense":
        mlp = {"kind": "dense", "ff": layer.mlp.ff}
    else:
        mlp = {"kind": "moe", "expert": {"ff": layer.mlp.ff}, "router": {"experts": layer.mlp.experts, "top": layer.mlp.top}}
    out = {"type": layer.type, "mixer": mixer, "mlp": mlp}
    if layer.weights_of is not None:
        out["weights_of"] = layer.weights_of
    return out


def check(c: BoneraxConfig) -> None:
    """The rules a configuration keeps wherever it came from."""
    def bad(key, why):
        return ConfigError(f"config: unsupported value for {key} ({why})")
    if c.vocab < 1 or c.width < 1:
        raise bad("width", "vocab and width are at least 1")
    if not c.layers:
        raise bad("layers", "at least one layer")

    def check_delta(m, where):
        if not isinstance(m, DeltaConfig):
            raise bad(where, "not the sizes of a delta rule")
        if m.heads % m.kv_heads:
            raise bad(f"{where}.kv_heads", "the head count must be divisible by it")
        if m.dim > 256:
            raise bad(f"{where}.dim", "at most 256")

    for i, layer in enumerate(c.layers):
        where = f"layers[{i}]"
        if layer.type not in LAYER_TYPES:
            raise bad(f"{where}.type", f"{layer.type!r}; this engine computes {list(LAYER_TYPES)}")
        m = layer.mixer
        if layer.type == "gla":
            if not isinstance(m, GLAConfig):
                raise bad(f"{where}.mixer", "not the sizes of gated linear attention")
            if m.dim > 256:
                raise bad(f"{where}.mixer.dim", "at most 256")
        elif layer.type == "channel_delta":
            check_delta(m, f"{where}.mixer")
        else:
            if not isinstance(m, ParallelConfig) or not isinstance(m.left, WindowAttentionConfig):
                raise bad(f"{where}.mixer", "not the sizes of a parallel mixer")
            check_delta(m.right, f"{where}.mixer.right")
            a = m.left
            if a.heads % a.kv_heads:
                raise bad(f"{where}.mixer.left.kv_heads", "the head count must be divisible by it")
            if a.rot_dims % 2 or a.rot_dims > a.dim:
                raise bad(f"{where}.mixer.left.rot.dims", "the rotated dims are even and at most dim")
            if a.rot_base <= 1.0 and a.rot_dims:
                raise bad(f"{where}.mixer.left.rot.base", "above 1")
        if layer.mlp is not None:
            if layer.mlp.kind not in MLP_KINDS or layer.mlp.ff < 1:
                raise bad(f"{where}.mlp", "a dense or routed feed-forward with an inner width of at least 1")
            if layer.mlp.kind == "moe" and not 0 < layer.mlp.top <= layer.mlp.experts:
                raise bad(f"{where}.mlp.router.top", "between 1 and the expert count")
        if layer.weights_of is not None:
            j = layer.weights_of
            if not 0 <= j < len(c.layers) or j == i or c.layers[j].weights_of is not None:
                raise bad(f"{where}.weights_of", "names another layer that has tensors of its own")
            if (c.layers[j].type, c.layers[j].mixer, c.layers[j].mlp) != (layer.type, layer.mixer, layer.mlp):
                raise bad(f"{where}.weights_of", f"the layer's sizes are not layer {j}'s")
