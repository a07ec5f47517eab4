"""Typed configuration of Sagedra (config.json with ``"architecture": "Sagedra"``).

A list of layers, each with a mixer of its own kind and sizes and an optional feed-forward; a span of the layers
may run several times in a row; the residual may be several streams (hyper-connections):

    {"architecture": "Sagedra", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "streams": S (optional), "loop": {"start": a, "stop": b, "times": n} (optional), "logit_softcap": c (optional),
     "layers": [{"type": "attention" | "parallel", "mixer": {...}, "mlp": {"kind": "dense", "ff": F} | null}, ...]}

mixer of ``attention`` (two score maps a head): heads, kv_heads, dim, vdim, scale, diff, optional conv (taps) and
q_temp {coef, every}.  mixer of ``parallel``: {left: {heads, kv_heads, dim, vdim, scale, optional rot {base, dims,
optional scaling {factor, low, high, original}}, optional mask {size}}, right: {heads, kv_heads, dim, vdim, conv}}.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, field_from, require

ARCHITECTURE = "Sagedra"
MIXER_KINDS = ("attention", "parallel")


def _object(raw: Dict[str, Any], key: str, where: str, needed: bool = False) -> Optional[Dict[str, Any]]:
    v = raw.get(key)
    if v is None:
        require(not needed, f"{where}: '{key}' must be an object")
        return None
    require(isinstance(v, dict), f"{where}: '{key}' must be an object")
    return v


@dataclass(frozen=True)
class DifferentialAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: int = 0                         # taps of the convolution on q, k, v; 0: none
    temp_coef: float = 0.0
    temp_every: int = 0                   # 0: no query temperature

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        temp = _object(raw, "q_temp", where)
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), g("dim"),
                field_from(raw, "vdim", int, g("dim"), where=where), field_from(raw, "scale", float, where=where),
                field_from(raw, "diff", float, where=where), field_from(raw, "conv", int, 0, where=where),
                field_from(temp, "coef", float, where=where + " q_temp") if temp is not None else 0.0,
                field_from(temp, "every", int, where=where + " q_temp") if temp is not None else 0)
        require(min(c.heads, c.kv_heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.conv >= 0, f"{where}: conv must not be negative")
        require(temp is None or c.temp_every > 0, f"{where} q_temp: every must be positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale, "diff": self.diff}
        if self.conv:
            d["conv"] = self.conv
        if self.temp_every:
            d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        return d


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float = 10000.0
    rot_dims: int = 0                                            # 0: no rotation
    rot_scaling: Optional[Tuple[float, float, float, float]] = None   # (factor, low, high, original)
    window: Optional[int] = None                                 # None: every earlier token is seen

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        rot, mask = _object(raw, "rot", where), _object(raw, "mask", where)
        rot_dims = field_from(rot, "dims", int, 0, where=where + " rot") if rot is not None else 0
        scaling = _object(rot, "scaling", where + " rot") if rot is not None else None
        s = lambda k: field_from(scaling, k, float, where=where + " rot scaling")
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), g("dim"),
                field_from(raw, "vdim", int, g("dim"), where=where), field_from(raw, "scale", float, where=where),
                field_from(rot, "base", float, where=where + " rot") if rot_dims else 10000.0, rot_dims,
                (s("factor"), s("low"), s("high"), s("original")) if (scaling is not None and rot_dims) else None,
                field_from(mask, "size", int, None, where=where + " mask") if mask is not None else None)
        require(min(c.heads, c.kv_heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.rot_dims >= 0 and c.rot_dims % 2 == 0 and c.rot_dims <= c.dim,
                f"{where}: rot.dims ({c.rot_dims}) must be even and at most dim ({c.dim})")
        require(c.rot_dims == 0 or c.rot_base > 1.0, f"{where}: rot.base must exceed 1")
        if c.rot_scaling is not None:
            factor, low, high, original = c.rot_scaling
            require(factor > 0 and high > low and original > 0,
                    f"{where} rot scaling: factor and original must be positive and high must exceed low")
        require(c.window is None or c.window > 0, f"{where}: mask.size must be positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                d["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), self.rot_scaling))
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class GatedDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), g("dim"),
                field_from(raw, "vdim", int, g("dim"), where=where), field_from(raw, "conv", int, 1, where=where))
        require(min(c.heads, c.kv_heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.conv >= 1, f"{where}: conv must be at least 1")
        return c

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class ParallelConfig:
    left: WindowAttentionConfig
    right: GatedDeltaConfig

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        return cls(WindowAttentionConfig.from_dict(_object(raw, "left", where, True), where + " left"),
                   GatedDeltaConfig.from_dict(_object(raw, "right", where, True), where + " right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


_MIXER_CONFIGS = {"attention": DifferentialAttentionConfig, "parallel": ParallelConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    ff: Optional[int]                     # width of the gated feed-forward; None: the layer has none

    @classmethod
    def from_dict(cls, raw: Any, i: int):
        where = f"config.json layers[{i}]"
        require(isinstance(raw, dict), f"{where}: must be an object")
        kind = field_from(raw, "type", str, where=where)
        if kind not in _MIXER_CONFIGS:
            raise ConfigError(f"{where}: type '{kind}' is not supported (supported: {', '.join(MIXER_KINDS)})")
        mixer = _MIXER_CONFIGS[kind].from_dict(_object(raw, "mixer", where, True), where + " mixer")
        mlp, ff = _object(raw, "mlp", where), None
        if mlp is not None:
            mlp_kind = field_from(mlp, "kind", str, "dense", where=where + " mlp")
            if mlp_kind != "dense":
                raise ConfigError(f"{where} mlp: kind '{mlp_kind}' is not supported (supported: dense)")
            ff = field_from(mlp, "ff", int, where=where + " mlp")
            require(ff > 0, f"{where} mlp: ff must be positive")
        return cls(kind, mixer, ff)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": {"kind": "dense", "ff": self.ff} if self.ff is not None else None}


@dataclass(frozen=True)
class SagedraConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    eps: float = 1e-5
    embedding_scale: float = 1.0
    streams: Optional[int] = None                     # None: one residual, plain pre-norm layers
    loop: Optional[Tuple[int, int, int]] = None       # (start, stop, times): layers start..stop-1 run `times` times
    logit_softcap: Optional[float] = None
    layers: Tuple[LayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "SagedraConfig":
        vocab, width = field_from(raw, "vocab", int), field_from(raw, "width", int)
        require(vocab > 0 and width > 0, "config.json: vocab and width must be positive")
        norm = _object(raw, "norm", "config.json", True)
        eps = field_from(norm, "eps", float, where="config.json norm")
        require(eps >= 0, "config.json norm: eps must not be negative")
        emb = _object(raw, "embedding", "config.json")
        scale = field_from(emb, "scale", float, 1.0, where="config.json embedding") if emb is not None else 1.0
        streams = field_from(raw, "streams", int, None)
        require(streams is None or streams >= 1, "config.json: streams must be at least 1")
        layers = raw.get("layers")
        require(isinstance(layers, list) and len(layers) > 0, "config.json: 'layers' must be a non-empty list")
        loop_raw, loop = _object(raw, "loop", "config.json"), None
        if loop_raw is not None:
            l = lambda k: field_from(loop_raw, k, int, where="config.json loop")
            loop = (l("start"), l("stop"), l("times"))
            require(0 <= loop[0] <= loop[1] <= len(layers), f"config.json loop: start {loop[0]} and stop {loop[1]} "
                    f"must lie in 0..{len(layers)}, in this order")
            require(loop[2] >= 1, "config.json loop: times must be at least 1")
        cap = field_from(raw, "logit_softcap", float, None)
        require(cap is None or cap > 0, "config.json: logit_softcap must be positive")
        return cls(ARCHITECTURE, vocab, width, eps, scale, streams, loop, cap,
                   tuple(LayerConfig.from_dict(l, i) for i, l in enumerate(layers)))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "norm": {"eps": self.eps}, "embedding": {"scale": self.embedding_scale},
                             "layers": [l.to_dict() for l in self.layers]}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d

    def layer_runs(self) -> Tuple[int, ...]:
        """The layers in the order they run: the looped span repeated in place."""
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        start, stop, times = self.loop
        return tuple(range(start)) + tuple(range(start, stop)) * times + tuple(range(stop, n))

    @property
    def vocabulary_size(self) -> int:
        return self.vocab
