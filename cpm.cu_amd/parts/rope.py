"""Rotary position encoding, plain and LongRoPE.

Rotate-half rotation by theta = position * inv_freq[c] (src/model/rotary.cuh:7-34); with ``pairs='interleaved'`` the
plain encoding pairs neighbouring features (2c, 2c + 1) instead of (c, c + head_dim/2), with the same angles.
The reference loads inv_freq once, computed for the engine's whole token budget
(cpmcu/llm.py:181-191): the choice between LongRoPE's short and long factors is
static per engine, long iff the engine holds sequences longer than
original_max_position_embeddings.  inv_freq[c] = 1 / (factor[c] * theta^(2c/hd)).
cos and sin carry the magnitude m = sqrt(1 + ln(max_position/original_max) /
ln(original_max)) when the position range was stretched (the reference drops it,
cpmcu/llm.py:190-192; ``attention_scaling=False`` does the same).
"""
from __future__ import annotations

import math
from typing import Mapping, Optional, Sequence, Tuple

import torch

from .base import POSITION_ENCODINGS, PositionEncoding, Runtime


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, pairs: str = "halves"):
        if pairs not in ("halves", "interleaved"):
            raise ValueError(f"rope: pairs '{pairs}' (halves or interleaved)")
        self.pairs = pairs
        self.head_dim = head_dim
        self.theta = float(theta)
        self.inv_freq: Optional[torch.Tensor] = None
        self.magnitude = 1.0

    def factors(self, max_seq_len: int) -> Optional[Sequence[float]]:
        return None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        c = torch.arange(0, self.head_dim, 2, dtype=torch.float64)
        base = self.theta ** (c / self.head_dim)
        f = self.factors(rt.max_seq_len)
        if f is not None:
            base = base * torch.tensor(list(f), dtype=torch.float64)
        self.inv_freq = (1.0 / base).to(torch.float32).to(rt.device)

    def rotary_params(self) -> Tuple[torch.Tensor, float]:
        return self.inv_freq, self.magnitude


@POSITION_ENCODINGS.register("longrope")
class LongRotaryEncoding(RotaryEncoding):
    def __init__(self, head_dim: int, theta: float, short_factor: Sequence[float], long_factor: Sequence[float],
                 original_max_position: int, max_position: int, attention_scaling: bool = True):
        super().__init__(head_dim, theta)
        if len(short_factor) != head_dim // 2 or len(long_factor) != head_dim // 2:
            raise ValueError(f"longrope: factor lists need head_dim/2 = {head_dim // 2} entries")
        self.short_factor = tuple(short_factor)
        self.long_factor = tuple(long_factor)
        self.original_max_position = original_max_position
        self.max_position = max_position
        ratio = max_position / original_max_position
        if attention_scaling and ratio > 1.0:
            self.magnitude = math.sqrt(1.0 + math.log(ratio) / math.log(original_max_position))

    def factors(self, max_seq_len: int):
        return self.long_factor if max_seq_len > self.original_max_position else self.short_factor


@POSITION_ENCODINGS.register("yarn")
class YarnRotaryEncoding(RotaryEncoding):
    """Rotation of ``head_dim`` features (a head may hold more; those pass unchanged) with YaRN's blend of
    stretched and plain frequencies.  With f_i = theta^(-2i/head_dim):
        d(t)   = head_dim * ln(original / (2 pi t)) / (2 ln theta)        (the feature that turns t times)
        lo, hi = max(floor(d(fast)), 0), min(ceil(d(slow)), head_dim - 1)
        ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
        freq_i = f_i / factor * ramp_i + f_i * (1 - ramp_i)
    and cos and sin carry the magnitude 0.1 ln(factor) + 1."""

    def __init__(self, head_dim: int, theta: float, factor: float, original: int, fast: float, slow: float):
        super().__init__(head_dim, theta)
        self.factor, self.original, self.fast, self.slow = float(factor), float(original), float(fast), float(slow)
        self.magnitude = 0.1 * math.log(self.factor) + 1.0

    def _turns_to_feature(self, turns: float) -> float:
        return self.head_dim * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        i = torch.arange(0, self.head_dim // 2, dtype=torch.float64)
        f = self.theta ** (-2.0 * i / self.head_dim)
        lo = max(math.floor(self._turns_to_feature(self.fast)), 0)
        hi = min(math.ceil(self._turns_to_feature(self.slow)), self.head_dim - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        self.inv_freq = (f / self.factor * ramp + f * (1.0 - ramp)).to(torch.float32).to(rt.device)


@POSITION_ENCODINGS.register("llama3")
class Llama3RotaryEncoding(RotaryEncoding):
    """Rotation of ``head_dim`` features whose slow frequencies are stretched (the frequency scaling of Llama 3.1).
    With f_i = theta^(-2i/head_dim) and wavelength l_i = 2 pi / f_i: f_i stays where l_i < original / high, becomes
    f_i / factor where l_i > original / low, and in between is (1 - t) f_i / factor + t f_i with
    t = (original / l_i - low) / (high - low).  The magnitude stays 1."""

    def __init__(self, head_dim: int, theta: float, factor: float, low: float, high: float, original: float):
        super().__init__(head_dim, theta)
        self.factor, self.low, self.high, self.original = float(factor), float(low), float(high), float(original)
        if self.factor <= 0 or self.high <= self.low or self.original <= 0:
            raise ValueError(f"llama3 rotation: factor {factor}, low {low}, high {high}, original {original}")

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        i = torch.arange(0, self.head_dim // 2, dtype=torch.float64)
        f = self.theta ** (-2.0 * i / self.head_dim)
        wave = 2.0 * math.pi / f
        t = ((self.original / wave - self.low) / (self.high - self.low)).clamp(0.0, 1.0)
        blend = (1.0 - t) * f / self.factor + t * f
        out = torch.where(wave < self.original / self.high, f, torch.where(wave > self.original / self.low, f / self.factor, blend))
        self.inv_freq = out.to(torch.float32).to(rt.device)
