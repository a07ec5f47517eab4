"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode.  Every tensor is drawn from a generator keyed by
(seed, tensor name), so a tensor's values depend on nothing but those two and
its shape: matrices and tables N(0, std), norm weights 1 + N(0, norm_std).
Values are stored in bfloat16 (the checkpoint's dtype), or as each spec says.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Callable, Dict, Optional

import torch

from ..config.base import ModelConfig
from ..parts.base import WeightSpec
from ..registry import get_architecture

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "int32": torch.int32}


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


# init rule name (WeightSpec.init) -> function(spec, generator, device, dtype, std, norm_std) -> tensor of
# spec.shape in dtype.  A part with another kind of tensor (decay rates, convolution taps) registers its own
# rule under a new name and names it in its WeightSpecs; this file needs no change for it.
INIT_RULES: Dict[str, Callable] = {}


def register_init_rule(name: str, fn: Optional[Callable] = None):
    def deco(f):
        if name in INIT_RULES and INIT_RULES[name] is not f:
            raise ValueError(f"init rule '{name}' is already registered")
        INIT_RULES[name] = f
        return f
    return deco if fn is None else deco(fn)


@register_init_rule("norm")
def _init_norm(spec, g, device, dtype, std, norm_std):
    """1 + N(0, norm_std)."""
    t = torch.ones(spec.shape, dtype=torch.float32, device=device)
    if norm_std > 0:
        t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * norm_std
    return t.to(dtype)


@register_init_rule("norm_offset")
def _init_norm_offset(spec, g, device, dtype, std, norm_std):
    """N(0, norm_std): the weight of a norm that multiplies by 1 + w."""
    t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
    if norm_std > 0:
        t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * norm_std
    return t.to(dtype)


@register_init_rule("poly_coefficients")
def _init_poly_coefficients(spec, g, device, dtype, std, norm_std):
    """The numbers of a polynomial activation: each of order 1, none near zero, signs mixed."""
    t = 0.4 + torch.rand(spec.shape, generator=g, dtype=torch.float32, device=device)
    sign = torch.where(torch.rand(spec.shape, generator=g, dtype=torch.float32, device=device) < 0.3, -1.0, 1.0)
    return (t * sign).to(dtype)


@register_init_rule("small")
def _init_small(spec, g, device, dtype, std, norm_std):
    """N(0, 0.5): biases of a convolution or of a step size."""
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * 0.5).to(dtype)


@register_init_rule("slight")
def _init_slight(spec, g, device, dtype, std, norm_std):
    """N(0, 0.05): a correction added to softmax scores, which must shift a choice now and then, not make it."""
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * 0.05).to(dtype)


@register_init_rule("conv_taps")
def _init_conv_taps(spec, g, device, dtype, std, norm_std):
    """N(0, 1/sqrt(taps)): the taps of a short convolution per channel."""
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * spec.shape[-1] ** -0.5).to(dtype)


@register_init_rule("log_decay")
def _init_log_decay(spec, g, device, dtype, std, norm_std):
    """ln of decay rates spread over (0.05, 4): slow heads that remember far back and fast ones."""
    u = torch.rand(spec.shape, generator=g, dtype=torch.float32, device=device)
    return torch.log(0.05 + 3.95 * u).to(dtype)


@register_init_rule("stream_read")
def _init_stream_read(spec, g, device, dtype, std, norm_std):
    """1/S + N(0, 0.2): the numbers with which a sub-layer reads a residual of S streams (near their mean)."""
    t = torch.full(spec.shape, 1.0 / spec.shape[-1], dtype=torch.float32, device=device)
    return (t + torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * 0.2).to(dtype)


@register_init_rule("stream_mix")
def _init_stream_mix(spec, g, device, dtype, std, norm_std):
    """identity + N(0, 0.15): the matrix that carries a residual of several streams past a sub-layer."""
    t = torch.eye(spec.shape[-1], dtype=torch.float32, device=device).expand(spec.shape).clone()
    return (t + torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * 0.15).to(dtype)


@register_init_rule("matrix")
def _init_matrix(spec, g, device, dtype, std, norm_std):
    """N(0, std)."""
    if len(spec.shape) == 2 and spec.shape[0] * spec.shape[1] > (1 << 28):
        # large tables row-block by row-block, to bound the float32 temporary
        out = torch.empty(spec.shape, dtype=dtype, device=device)
        step = max((1 << 28) // spec.shape[1], 1)
        for r in range(0, spec.shape[0], step):
            rows = min(step, spec.shape[0] - r)
            out[r:r + rows] = (torch.randn((rows, spec.shape[1]), generator=g, dtype=torch.float32, device=device)
                               * std).to(dtype)
        return out
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std).to(dtype)


register_init_rule("table", _init_matrix)


def draw(spec: WeightSpec, seed: int, std: float = 0.02, norm_std: float = 0.0, device="cpu") -> torch.Tensor:
    g = _generator(seed, spec.name, device)
    rule = INIT_RULES.get(spec.init)
    if rule is None:
        raise ValueError(f"tensor '{spec.name}': unknown init rule '{spec.init}' (registered: {sorted(INIT_RULES)})")
    t = rule(spec, g, device, _STORAGE[spec.storage], std, norm_std)
    if tuple(t.shape) != tuple(spec.shape) or t.dtype != _STORAGE[spec.storage]:
        raise ValueError(f"tensor '{spec.name}': init rule '{spec.init}' gave {tuple(t.shape)} {t.dtype}, "
                         f"{tuple(spec.shape)} {_STORAGE[spec.storage]} expected")
    return t


def random_tensors(config: ModelConfig, seed: int, std: float = 0.02, norm_std: float = 0.0, device="cpu"
                   ) -> Dict[str, torch.Tensor]:
    """All tensors the architecture's model asks for, drawn from (seed, name)."""
    model = get_architecture(config.architecture).build_model(config)
    return {s.name: draw(s, seed, std, norm_std, device) for s in model.all_weight_specs()}


def write_model_dir(config: ModelConfig, out_dir: str, seed: int, std: float = 0.02, norm_std: float = 0.0) -> str:
    """Write config.json and model.safetensors for ``config`` into out_dir."""
    from safetensors.torch import save_file
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    tensors = random_tensors(config, seed, std, norm_std)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    return out_dir
