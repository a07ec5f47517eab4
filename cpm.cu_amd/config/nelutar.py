"""Typed configuration of Nelutar (config.json with ``"architecture": "Nelutar"``).

A list of parallel layers (one norm; mixer and feed-forward read its output; each result times a learned vector),
each with a mixer of its own kind and sizes and an optional feed-forward; a layer may borrow another layer's
weights; the embedding may add a hashed bigram table:

    {"architecture": "Nelutar", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"bigram": {"buckets": B, "mul_prev": a, "mul_cur": b}} (optional),
     "layers": [{"type": "parallel" | "parallel_2" | "retention", "mixer": {...}, "mlp": {...} | null,
                 "weights_of": j (optional)}, ...]}

mixer of ``parallel``: {left: attention, right: {heads, kv_heads, dim, vdim, conv}} (a gated delta rule whose decay
is a number a key channel).  mixer of ``parallel_2``: {left: attention, right: {heads, dim, vdim, decay: [...]},
left_scale, right_scale}.  mixer of ``retention``: {heads, dim, vdim, decay: [...], optional rot {base, dims}}.
attention: {heads, kv_heads, dim, vdim, scale, optional rot {base, dims}, mask {size}, conv (taps), softcap}.
mlp: {"kind": "dense", "ff": F} or {"kind": "moe", "expert": {ff, limit}, "router": {experts, top, scale, optional
groups {count, keep}}, optional "shared": {ff, limit}}.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, field_from, require

ARCHITECTURE = "Nelutar"
MIXER_KINDS = ("parallel", "parallel_2", "retention")


def _object(raw: Dict[str, Any], key: str, where: str, needed: bool = False) -> Optional[Dict[str, Any]]:
    v = raw.get(key)
    if v is None:
        require(not needed, f"{where}: '{key}' must be an object")
        return None
    require(isinstance(v, dict), f"{where}: '{key}' must be an object")
    return v


def _rotation(raw: Dict[str, Any], dim: int, where: str) -> Tuple[float, int]:
    """(base, dims) of an optional 'rot' object; dims 0: no rotation."""
    rot = _object(raw, "rot", where)
    dims = field_from(rot, "dims", int, 0, where=where + " rot") if rot is not None else 0
    base = field_from(rot, "base", float, where=where + " rot") if dims else 10000.0
    require(dims >= 0 and dims % 2 == 0 and dims <= dim, f"{where}: rot.dims ({dims}) must be even and at most dim ({dim})")
    require(dims == 0 or base > 1.0, f"{where}: rot.base must exceed 1")
    return base, dims


def _decays(raw: Dict[str, Any], heads: int, where: str) -> Tuple[float, ...]:
    d = raw.get("decay")
    require(isinstance(d, list) and len(d) == heads and all(isinstance(x, (int, float)) and not isinstance(x, bool) for x in d),
            f"{where}: 'decay' must list one number for each of the {heads} heads")
    require(all(0.0 <= float(x) <= 1.0 for x in d), f"{where}: decays must lie in 0..1")
    return tuple(float(x) for x in d)


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float = 10000.0
    rot_dims: int = 0                     # 0: no rotation
    window: Optional[int] = None          # None: every earlier token is seen
    conv: int = 0                         # taps of the convolution on q, k, v; 0: none
    softcap: Optional[float] = None

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        mask = _object(raw, "mask", where)
        dim = g("dim")
        base, dims = _rotation(raw, dim, where)
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), dim,
                field_from(raw, "vdim", int, dim, where=where), field_from(raw, "scale", float, where=where), base, dims,
                field_from(mask, "size", int, None, where=where + " mask") if mask is not None else None,
                field_from(raw, "conv", int, 0, where=where), field_from(raw, "softcap", float, None, where=where))
        require(min(c.heads, c.kv_heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.window is None or c.window > 0, f"{where}: mask.size must be positive")
        require(c.conv >= 0, f"{where}: conv must not be negative")
        require(c.softcap is None or c.softcap > 0, f"{where}: softcap must be positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.conv:
            d["conv"] = self.conv
        if self.softcap is not None:
            d["softcap"] = self.softcap
        return d


@dataclass(frozen=True)
class ChannelDeltaConfig:
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
class DecayAttentionConfig:
    """Linear attention with a fixed decay a head (retention; the second mixer of ``parallel_2``)."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_base: float = 10000.0
    rot_dims: int = 0

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        heads, dim = g("heads"), g("dim")
        require(heads > 0 and dim > 0, f"{where}: sizes must be positive")
        base, dims = _rotation(raw, dim, where)
        c = cls(heads, dim, field_from(raw, "vdim", int, dim, where=where), _decays(raw, heads, where), base, dims)
        require(c.vdim > 0, f"{where}: sizes must be positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return d


@dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: ChannelDeltaConfig

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        return cls(AttentionConfig.from_dict(_object(raw, "left", where, True), where + " left"),
                   ChannelDeltaConfig.from_dict(_object(raw, "right", where, True), where + " right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class Parallel2Config:
    left: AttentionConfig
    right: DecayAttentionConfig
    left_scale: float = 1.0
    right_scale: float = 1.0

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        return cls(AttentionConfig.from_dict(_object(raw, "left", where, True), where + " left"),
                   DecayAttentionConfig.from_dict(_object(raw, "right", where, True), where + " right"),
                   field_from(raw, "left_scale", float, 1.0, where=where), field_from(raw, "right_scale", float, 1.0, where=where))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                             # "dense" or "moe"
    ff: int                               # width of the dense layer, or of one expert
    limit: Optional[float] = None         # experts: where their gate and up halves are cut off
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    groups: Optional[Tuple[int, int]] = None      # (count, keep)
    shared_ff: Optional[int] = None
    shared_limit: Optional[float] = None

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        require(isinstance(raw, dict), f"{where}: must be an object or null")
        kind = field_from(raw, "kind", str, "dense", where=where)
        if kind == "dense":
            c = cls(kind, field_from(raw, "ff", int, where=where))
            require(c.ff > 0, f"{where}: ff must be positive")
            return c
        if kind != "moe":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (supported: dense, moe)")
        expert, router = _object(raw, "expert", where, True), _object(raw, "router", where, True)
        shared, groups = _object(raw, "shared", where), _object(router, "groups", where + " router")
        c = cls(kind, field_from(expert, "ff", int, where=where + " expert"),
                field_from(expert, "limit", float, where=where + " expert"),
                field_from(router, "experts", int, where=where + " router"),
                field_from(router, "top", int, where=where + " router"),
                field_from(router, "scale", float, 1.0, where=where + " router"),
                (field_from(groups, "count", int, where=where + " router groups"),
                 field_from(groups, "keep", int, where=where + " router groups")) if groups is not None else None,
                field_from(shared, "ff", int, where=where + " shared") if shared is not None else None,
                field_from(shared, "limit", float, where=where + " shared") if shared is not None else None)
        require(c.ff > 0 and c.experts > 0, f"{where}: sizes must be positive")
        require(c.limit > 0 and (c.shared_limit is None or c.shared_limit > 0), f"{where}: limits must be positive")
        require(0 < c.top <= c.experts, f"{where} router: top ({c.top}) must lie in 1..experts ({c.experts})")
        if c.groups is not None:
            count, keep = c.groups
            require(count > 0 and c.experts % count == 0,
                    f"{where} router: experts ({c.experts}) must split into groups.count ({count}) equal groups")
            require(0 < keep <= count, f"{where} router: groups.keep ({keep}) must lie in 1..count ({count})")
            require(c.top <= keep * (c.experts // count),
                    f"{where} router: top ({c.top}) exceeds the experts of the {keep} groups that may be chosen from")
        require(c.shared_ff is None or c.shared_ff > 0, f"{where} shared: ff must be positive")
        return c

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top, "scale": self.router_scale}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        d: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit}, "router": router}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


_MIXER_CONFIGS = {"parallel": ParallelConfig, "parallel_2": Parallel2Config, "retention": DecayAttentionConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    mlp: Optional[FeedForwardConfig]      # None: the layer has no feed-forward
    weights_of: Optional[int] = None      # the layer whose tensors this one uses; None: its own

    @classmethod
    def from_dict(cls, raw: Any, i: int):
        where = f"config.json layers[{i}]"
        require(isinstance(raw, dict), f"{where}: must be an object")
        kind = field_from(raw, "type", str, where=where)
        if kind not in _MIXER_CONFIGS:
            raise ConfigError(f"{where}: type '{kind}' is not supported (supported: {', '.join(MIXER_KINDS)})")
        mixer = _MIXER_CONFIGS[kind].from_dict(_object(raw, "mixer", where, True), where + " mixer")
        mlp = raw.get("mlp")
        return cls(kind, mixer, FeedForwardConfig.from_dict(mlp, where + " mlp") if mlp is not None else None,
                   field_from(raw, "weights_of", int, None, where=where))

    def to_dict(self):
        d = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class NelutarConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    eps: float = 1e-5
    bigram: Optional[Tuple[int, int, int]] = None     # (buckets, mul_prev, mul_cur)
    layers: Tuple[LayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "NelutarConfig":
        vocab, width = field_from(raw, "vocab", int), field_from(raw, "width", int)
        require(vocab > 0 and width > 0, "config.json: vocab and width must be positive")
        norm = _object(raw, "norm", "config.json", True)
        eps = field_from(norm, "eps", float, where="config.json norm")
        require(eps >= 0, "config.json norm: eps must not be negative")
        emb = _object(raw, "embedding", "config.json")
        big_raw, bigram = (_object(emb, "bigram", "config.json embedding") if emb is not None else None), None
        if big_raw is not None:
            b = lambda k: field_from(big_raw, k, int, where="config.json embedding bigram")
            bigram = (b("buckets"), b("mul_prev"), b("mul_cur"))
            require(bigram[0] > 0 and bigram[1] >= 0 and bigram[2] >= 0,
                    "config.json embedding bigram: buckets must be positive, the multipliers not negative")
        layers = raw.get("layers")
        require(isinstance(layers, list) and len(layers) > 0, "config.json: 'layers' must be a non-empty list")
        # a layer that uses another's weights equals it in everything else: what its entry leaves out is the other's
        filled = []
        for i, l in enumerate(layers):
            j = l.get("weights_of") if isinstance(l, dict) else None
            if isinstance(j, int) and not isinstance(j, bool) and 0 <= j < len(layers) and j != i and isinstance(layers[j], dict):
                l = {**{k: v for k, v in layers[j].items() if k != "weights_of"}, **l}
            filled.append(l)
        parsed = tuple(LayerConfig.from_dict(l, i) for i, l in enumerate(filled))
        for i, l in enumerate(parsed):
            if l.weights_of is None:
                continue
            j = l.weights_of
            require(0 <= j < len(parsed) and j != i and parsed[j].weights_of is None,
                    f"config.json layers[{i}]: weights_of ({j}) must name another layer that has weights of its own")
            require(l.type == parsed[j].type and (l.mlp is None) == (parsed[j].mlp is None) and
                    (l.mlp is None or l.mlp.kind == parsed[j].mlp.kind),
                    f"config.json layers[{i}]: a layer that uses layer {j}'s weights must equal it in type and kind of mlp")
        return cls(ARCHITECTURE, vocab, width, eps, bigram, parsed)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "norm": {"eps": self.eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.bigram is not None:
            d["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        return d

    def layer_weights(self) -> Tuple[int, ...]:
        """For every layer, the layer whose tensors it uses (itself, unless it says otherwise)."""
        return tuple(i if l.weights_of is None else l.weights_of for i, l in enumerate(self.layers))

    def shares_block(self, i: int) -> bool:
        """Whether layer i is its weights' owner run once more: it borrows, and equals the owner in every size and
        constant (what a borrowing layer is meant to be; one that differs, in a window or a decay, say, is built as a
        layer of its own that reads the owner's tensors)."""
        l = self.layers[i]
        if l.weights_of is None:
            return False
        o = self.layers[l.weights_of]
        return (l.type, l.mixer, l.mlp) == (o.type, o.mixer, o.mlp)

    @property
    def vocabulary_size(self) -> int:
        return self.vocab
