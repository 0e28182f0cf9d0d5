"""Salipel's typed configuration, read from its own config.json keys.

A decoder whose layers are listed one by one.  A layer has one RMS norm; its mixer and its feed-forward both read the
normed rows and their sum, times a constant, joins the residual.  The mixer is "attention" (softmax attention inside chunks
of the sequence, a distance penalty a head, unit-RMS values, a sink in the softmax), "attention_2" (two soft-capped causal
score maps a head over one set of values, the second taken off lambda times, the difference normed and gated) or
"parallel" (attention over a sliding window that keeps the sequence's first tokens, its values being its projected keys,
beside a matrix memory with exponential gates, their weighted sum); the feed-forward is a dense gated unit with the tanh
form of gelu, routed experts of squared-relu units (softmax scores, a correction on the choice only), or absent.
config.json gives every size and every constant that differs between models of the design:

  architecture "Salipel"; vocab; width; norm.eps; residual_mult; layers[]: type, mixer
  (attention: heads, kv_heads, dim, vdim, scale, mask {size};
   attention_2: heads, kv_heads, dim, vdim, scale, softcap (optional), diff, rot {base, dims, scaling (optional)};
   parallel: left {heads, kv_heads, dim, vdim, scale, mask {size, keep_first}, rot {base, dims, scaling {factor, low, high,
   original} (optional)}}, right {heads, dim, vdim, gate_cap}, left_scale, right_scale),
  mlp (null | {kind "dense", ff} | {kind "moe", expert {ff}, router {experts, top, scale}}).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .givozen import WavelengthScaling
from .reader import ConfigError, KeyReader

ARCHITECTURE = "Salipel"
#: keys a model folder's config.json may carry that say nothing about the arithmetic
WITHOUT_EFFECT = ("name", "seed", "comment", "description", "dtype", "torch_dtype")
LAYER_TYPES = ("attention", "attention_2", "parallel")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: Optional[WavelengthScaling] = None


@dataclass(frozen=True)
class ChunkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int


@dataclass(frozen=True)
class DifferenceAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]        # None: the scores are not capped
    diff: float
    rot: Rotation


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int
    rot: Rotation


@dataclass(frozen=True)
class MemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class ParallelConfig:
    left: WindowAttentionConfig
    right: MemoryConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class MLPConfig:
    kind: str                       # "dense" | "moe"
    ff: int                         # inner width (of one expert for "moe")
    experts: int = 0
    top: int = 0
    scale: float = 1.0              # moe: the factor on the normalized weights


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any                      # ChunkAttentionConfig | DifferenceAttentionConfig | ParallelConfig
    mlp: Optional[MLPConfig] = None


@dataclass(frozen=True)
class SalipelConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[LayerConfig, ...]

    architecture = ARCHITECTURE

    def __post_init__(self):
        object.__setattr__(self, "layers", tuple(self.layers))
        check(self)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "SalipelConfig":
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
        cfg = cls(vocab=r.integer("vocab"), width=r.integer("width"), norm_eps=eps, residual_mult=r.real("residual_mult"), layers=layers)
        r.finish(WITHOUT_EFFECT, ARCHITECTURE)
        return cfg

    @property
    def vocab_size(self) -> int:
        """The vocabulary under the name the command line asks every configuration for."""
        return self.vocab

    def to_json(self) -> dict:
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "layers": [_layer_json(layer) for layer in self.layers]}


def _read_rotation(m: KeyReader) -> Rotation:
    rot = m.child("rot")
    sc = rot.child("scaling", required=False)
    scaling = None
    if sc is not None:
        scaling = WavelengthScaling(factor=sc.real("factor", positive=True), low=sc.real("low", positive=True),
                                    high=sc.real("high", positive=True), original=sc.real("original", positive=True))
        sc.finish((), ARCHITECTURE)
    out = Rotation(base=rot.real("base", positive=True), dims=rot.integer("dims", lo=0), scaling=scaling)
    rot.finish((), ARCHITECTURE)
    return out


def _heads(m: KeyReader) -> Dict[str, Any]:
    return dict(heads=m.integer("heads"), kv_heads=m.integer("kv_heads"), dim=m.integer("dim"), vdim=m.integer("vdim"),
                scale=m.real("scale", positive=True))


def _read_mixer(kind: str, m: KeyReader):
    if kind == "attention":
        mask = m.child("mask")
        out = ChunkAttentionConfig(chunk=mask.integer("size"), **_heads(m))
        mask.finish((), ARCHITECTURE)
        return out
    if kind == "attention_2":
        return DifferenceAttentionConfig(softcap=m.real("softcap", positive=True, default=None), diff=m.real("diff"), rot=_read_rotation(m), **_heads(m))
    left, right = m.child("left"), m.child("right")
    mask = left.child("mask")
    a = WindowAttentionConfig(window=mask.integer("size"), keep_first=mask.integer("keep_first", lo=0, default=0), rot=_read_rotation(left),
                              **_heads(left))
    mask.finish((), ARCHITECTURE)
    left.finish((), ARCHITECTURE)
    b = MemoryConfig(heads=right.integer("heads"), dim=right.integer("dim"), vdim=right.integer("vdim"),
                     gate_cap=right.real("gate_cap", positive=True))
    right.finish((), ARCHITECTURE)
    return ParallelConfig(a, b, left_scale=m.real("left_scale"), right_scale=m.real("right_scale"))


def _read_layer(entry, i: int) -> LayerConfig:
    r = KeyReader(entry, where=f"layers[{i}]")
    kind = r.choice("type", LAYER_TYPES)
    m = r.child("mixer")
    mixer = _read_mixer(kind, m)
    m.finish((), ARCHITECTURE)
    mlp = r.child("mlp", required=False)
    ff = None
    if mlp is not None:
        if mlp.choice("kind", MLP_KINDS) == "dense":
            ff = MLPConfig("dense", mlp.integer("ff"))
        else:
            expert, router = mlp.child("expert"), mlp.child("router")
            ff = MLPConfig("moe", expert.integer("ff"), experts=router.integer("experts"), top=router.integer("top"),
                           scale=router.real("scale", default=1.0))
            expert.finish((), ARCHITECTURE)
            router.finish((), ARCHITECTURE)
        mlp.finish((), ARCHITECTURE)
    r.finish(("name", "comment"), ARCHITECTURE)
    return LayerConfig(kind, mixer, ff)


def _rot_json(rot: Rotation) -> dict:
    out: Dict[str, Any] = {"base": rot.base, "dims": rot.dims}
    if rot.scaling is not None:
        s = rot.scaling
        out["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
    return out


def _layer_json(layer: LayerConfig) -> dict:
    a = layer.mixer
    if layer.type == "parallel":
        l, r = a.left, a.right
        mixer = {"left": {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                          "mask": {"size": l.window, "keep_first": l.keep_first}, "rot": _rot_json(l.rot)},
                 "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "gate_cap": r.gate_cap},
                 "left_scale": a.left_scale, "right_scale": a.right_scale}
    else:
        mixer = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
        if layer.type == "attention":
            mixer["mask"] = {"size": a.chunk}
        else:
            mixer.update({"diff": a.diff, "rot": _rot_json(a.rot)})
            if a.softcap is not None:
                mixer["softcap"] = a.softcap
    if layer.mlp is None:
        mlp = None
    elif layer.mlp.kind == "dense":
        mlp = {"kind": "dense", "ff": layer.mlp.ff}
    else:
        mlp = {"kind": "moe", "expert": {"ff": layer.mlp.ff},
               "router": {"experts": layer.mlp.experts, "top": layer.mlp.top, "scale": layer.mlp.scale}}
    return {"type": layer.type, "mixer": mixer, "mlp": mlp}


def check(c: SalipelConfig) -> None:
    """The rules a configuration keeps wherever it came from."""
    def bad(key, why):
        return ConfigError(f"config: unsupported value for {key} ({why})")

    def heads(where, a):
        if a.heads % a.kv_heads:
            raise bad(f"{where}.kv_heads", "the head count must be divisible by it")

    def rotation(where, rot, dim):
        if rot.dims % 2 or rot.dims > dim:
            raise bad(f"{where}.rot.dims", "the rotated dims are even and at most dim")
        if rot.base <= 1.0 and rot.dims:
            raise bad(f"{where}.rot.base", "above 1")
        if rot.scaling is not None and not rot.scaling.high > rot.scaling.low:
            raise bad(f"{where}.rot.scaling.high", "above low")

    if c.vocab < 1 or c.width < 1:
        raise bad("width", "vocab and width are at least 1")
    if not c.layers:
        raise bad("layers", "at least one layer")
    for i, layer in enumerate(c.layers):
        where = f"layers[{i}]"
        if layer.type not in LAYER_TYPES:
            raise bad(f"{where}.type", f"{layer.type!r}; this engine computes {list(LAYER_TYPES)}")
        a = layer.mixer
        want = {"attention": ChunkAttentionConfig, "attention_2": DifferenceAttentionConfig, "parallel": ParallelConfig}[layer.type]
        if not isinstance(a, want):
            raise bad(f"{where}.mixer", f"not the sizes of a mixer of type {layer.type!r}")
        if layer.type == "attention":
            heads(f"{where}.mixer", a)
            if a.chunk < 1:
                raise bad(f"{where}.mixer.mask.size", "at least 1")
        elif layer.type == "attention_2":
            heads(f"{where}.mixer", a)
            rotation(f"{where}.mixer", a.rot, a.dim)
            if not a.diff < 1.0:
                raise bad(f"{where}.mixer.diff", "below 1")
        else:
            heads(f"{where}.mixer.left", a.left)
            rotation(f"{where}.mixer.left", a.left.rot, a.left.dim)
            if a.left.vdim != a.left.dim:
                raise bad(f"{where}.mixer.left.vdim", "the values are the projected keys, so as wide as dim")
            if a.left.window < 1:
                raise bad(f"{where}.mixer.left.mask.size", "at least 1")
        if layer.mlp is not None:
            if layer.mlp.kind not in MLP_KINDS or layer.mlp.ff < 1:
                raise bad(f"{where}.mlp", "a dense or routed feed-forward with an inner width of at least 1")
            if layer.mlp.kind == "moe" and not 0 < layer.mlp.top <= layer.mlp.experts:
                raise bad(f"{where}.mlp.router.top", "between 1 and the expert count")
