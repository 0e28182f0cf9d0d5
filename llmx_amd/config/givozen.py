"""Givozen's typed configuration, read from its own config.json keys.

A decoder whose layers are listed one by one.  A layer has a norm before and after each sublayer; its mixer is causal
grouped-query softmax attention (biased q, k, v; a partial rotation in halves with frequencies rescaled by wavelength; a
temperature and a sigmoid gate a head); its feed-forward is dense with a polynomial of unit-RMS powers between its two
products, routed experts of a clamped gated unit (sigmoid scores that multiply the expert's input) with an optional gated
shared expert, or absent.  A run of layers may repeat (`loop`), each pass with caches of its own.  config.json gives every
size and every constant that differs between models of the design:

  architecture "Givozen"; vocab; width; norm.eps; loop {start, stop, times} (optional); layers[]: type "attention", mixer
  {heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling {factor, low, high, original} (optional)}}, mlp (null |
  {kind "dense", ff} | {kind "moe", expert {ff, limit}, router {experts, top}, shared {ff, limit} (optional)}).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .reader import ConfigError, KeyReader

ARCHITECTURE = "Givozen"
#: keys a model folder's config.json may carry that say nothing about the arithmetic
WITHOUT_EFFECT = ("name", "seed", "comment", "description", "dtype", "torch_dtype")
LAYER_TYPES = ("attention",)
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class WavelengthScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[WavelengthScaling] = None


@dataclass(frozen=True)
class SharedExpertConfig:
    ff: int
    limit: float


@dataclass(frozen=True)
class MLPConfig:
    kind: str                       # "dense" | "moe"
    ff: int                         # inner width (of one expert for "moe")
    limit: float = 0.0              # moe: the gated unit's clamp
    experts: int = 0
    top: int = 0
    shared: Optional[SharedExpertConfig] = None


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: AttentionConfig
    mlp: Optional[MLPConfig] = None


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class GivozenConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[LayerConfig, ...]
    loop: Optional[LoopConfig] = None

    architecture = ARCHITECTURE

    def __post_init__(self):
        object.__setattr__(self, "layers", tuple(self.layers))
        check(self)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "GivozenConfig":
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
        lp = r.child("loop", required=False)
        loop = None
        if lp is not None:
            loop = LoopConfig(start=lp.integer("start", lo=0), stop=lp.integer("stop", lo=0), times=lp.integer("times", lo=1))
            lp.finish((), ARCHITECTURE)
        cfg = cls(vocab=r.integer("vocab"), width=r.integer("width"), norm_eps=eps, layers=layers, loop=loop)
        r.finish(WITHOUT_EFFECT, ARCHITECTURE)
        return cfg

    @property
    def vocab_size(self) -> int:
        """The vocabulary under the name the command line asks every configuration for."""
        return self.vocab

    def to_json(self) -> dict:
        out: Dict[str, Any] = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                               "layers": [_layer_json(layer) for layer in self.layers]}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out

    def passes(self):
        """The layers in the order they run: (layer, pass number or None outside the loop, whether it opens its pass)."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None, False) for i in range(n)]
        lp = self.loop
        order = [(i, None, False) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t, i == lp.start) for i in range(lp.start, lp.stop)]
        return order + [(i, None, False) for i in range(lp.stop, n)]


def _read_attention(m: KeyReader) -> AttentionConfig:
    rot = m.child("rot")
    sc = rot.child("scaling", required=False)
    scaling = None
    if sc is not None:
        scaling = WavelengthScaling(factor=sc.real("factor", positive=True), low=sc.real("low", positive=True),
                                    high=sc.real("high", positive=True), original=sc.real("original", positive=True))
        sc.finish((), ARCHITECTURE)
    cfg = AttentionConfig(heads=m.integer("heads"), kv_heads=m.integer("kv_heads"), dim=m.integer("dim"), vdim=m.integer("vdim"),
                          scale=m.real("scale", positive=True), rot_base=rot.real("base", positive=True),
                          rot_dims=rot.integer("dims", lo=0), rot_scaling=scaling)
    rot.finish((), ARCHITECTURE)
    return cfg


def _read_layer(entry, i: int) -> LayerConfig:
    r = KeyReader(entry, where=f"layers[{i}]")
    kind = r.choice("type", LAYER_TYPES)
    m = r.child("mixer")
    mixer = _read_attention(m)
    m.finish((), ARCHITECTURE)
    mlp = r.child("mlp", required=False)
    ff = None
    if mlp is not None:
        if mlp.choice("kind", MLP_KINDS) == "dense":
            ff = MLPConfig("dense", mlp.integer("ff"))
        else:
            expert, router = mlp.child("expert"), mlp.child("router")
            sh = mlp.child("shared", required=False)
            shared = None
            if sh is not None:
                shared = SharedExpertConfig(ff=sh.integer("ff"), limit=sh.real("limit", positive=True))
                sh.finish((), ARCHITECTURE)
            ff = MLPConfig("moe", expert.integer("ff"), limit=expert.real("limit", positive=True), experts=router.integer("experts"),
                           top=router.integer("top"), shared=shared)
            expert.finish((), ARCHITECTURE)
            router.finish((), ARCHITECTURE)
        mlp.finish((), ARCHITECTURE)
    r.finish(("name", "comment"), ARCHITECTURE)
    return LayerConfig(kind, mixer, ff)


def _layer_json(layer: LayerConfig) -> dict:
    a = layer.mixer
    rot: Dict[str, Any] = {"base": a.rot_base, "dims": a.rot_dims}
    if a.rot_scaling is not None:
        s = a.rot_scaling
        rot["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
    mixer = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale, "rot": rot}
    if layer.mlp is None:
        mlp = None
    elif layer.mlp.kind == "dense":
        mlp = {"kind": "dense", "ff": layer.mlp.ff}
    else:
        mlp = {"kind": "moe", "expert": {"ff": layer.mlp.ff, "limit": layer.mlp.limit},
               "router": {"experts": layer.mlp.experts, "top": layer.mlp.top}}
        if layer.mlp.shared is not None:
            mlp["shared"] = {"ff": layer.mlp.shared.ff, "limit": layer.mlp.shared.limit}
    return {"type": layer.type, "mixer": mixer, "mlp": mlp}


def check(c: GivozenConfig) -> None:
    """The rules a configuration keeps wherever it came from."""
    def bad(key, why):
        return ConfigError(f"config: unsupported value for {key} ({why})")
    if c.vocab < 1 or c.width < 1:
        raise bad("width", "vocab and width are at least 1")
    if not c.layers:
        raise bad("layers", "at least one layer")
    for i, layer in enumerate(c.layers):
        where = f"layers[{i}]"
        if layer.type not in LAYER_TYPES:
            raise bad(f"{where}.type", f"{layer.type!r}; this engine computes {list(LAYER_TYPES)}")
        a = layer.mixer
        if not isinstance(a, AttentionConfig):
            raise bad(f"{where}.mixer", "not the sizes of an attention")
        if a.heads % a.kv_heads:
            raise bad(f"{where}.mixer.kv_heads", "the head count must be divisible by it")
        if a.rot_dims % 2 or a.rot_dims > a.dim:
            raise bad(f"{where}.mixer.rot.dims", "the rotated dims are even and at most dim")
        if a.rot_base <= 1.0 and a.rot_dims:
            raise bad(f"{where}.mixer.rot.base", "above 1")
        if a.rot_scaling is not None and not a.rot_scaling.high > a.rot_scaling.low:
            raise bad(f"{where}.mixer.rot.scaling.high", "above low")
        if layer.mlp is not None:
            if layer.mlp.kind not in MLP_KINDS or layer.mlp.ff < 1:
                raise bad(f"{where}.mlp", "a dense or routed feed-forward with an inner width of at least 1")
            if layer.mlp.kind == "moe":
                if not 0 < layer.mlp.top <= layer.mlp.experts:
                    raise bad(f"{where}.mlp.router.top", "between 1 and the expert count")
                if not layer.mlp.limit > 0.0:
                    raise bad(f"{where}.mlp.expert.limit", "positive")
    if c.loop is not None:
        lp = c.loop
        if not 0 <= lp.start < lp.stop <= len(c.layers) or lp.times < 1:
            raise bad("loop", "0 <= start < stop <= the number of layers, and at least one pass")
