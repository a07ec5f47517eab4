"""Differential attention: every head has two score maps over the same values and puts out their difference.

q has heads * 2 * dim rows and k has kv_heads * 2 * dim rows, laid out head by head as [map 1 | map 2]; v has
kv_heads * vdim rows.  q, k, v (with their biases) may pass a short causal convolution per channel over time (taps
weights a channel, the last one the current token's, zeros before the sequence's start, no activation); the last
taps - 1 projected rows of a sequence are fixed-size state in its cache slot.  Positions enter through the query
alone: q is multiplied by 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1).  Each map is a causal softmax
attention, score = q.k * scale, query head h on key/value head h // (heads / kv_heads); with a1 and a2 the maps'
outputs of a head and lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number a layer, from four checkpoint
vectors of dim numbers):

    o = a1 - lambda * a2;   o <- o / sqrt(mean(o^2) + eps) * (1 - diff)   per head, then the output projection.

The attention itself is the library's general kernel over 2 * heads query heads and 2 * kv_heads key heads of
which every two neighbours share a value head, so the cache holds the values once.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec, StreamSpec
from .base import MIXERS, BiasedBranch, Mixer, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


def _pad16(n: int) -> int:
    return -(-n // 16) * 16


@MIXERS.register("differential_attention")
class DifferentialAttention(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, scale: float, diff: float, norm_eps: float, conv_taps: int = 0, temp_coef: float = 0.0,
                 temp_every: int = 0):
        """``names``: checkpoint tensors for 'q', 'k', 'v', 'out', 'lq1', 'lk1', 'lq2', 'lk2', optionally 'q_bias',
        'k_bias', 'v_bias', 'out_bias', and with ``conv_taps`` > 0 'q_conv', 'k_conv', 'v_conv'.  ``temp_every`` 0:
        no query temperature."""
        if num_heads % num_kv_heads:
            raise ValueError(f"differential attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if key_dim > 1024 or value_dim > 1024:
            raise ValueError(f"differential attention: key size {key_dim} / value size {value_dim} exceed the kernel's 1024")
        if conv_taps < 0 or temp_every < 0:
            raise ValueError(f"differential attention: {conv_taps} convolution taps, a temperature step of {temp_every}")
        self.names = dict(names)
        self.hidden_size, self.nh, self.nkv, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, key_dim, value_dim
        self.scale, self.diff, self.eps = float(scale), float(diff), float(norm_eps)
        self.taps, self.temp_coef, self.temp_every = int(conv_taps), float(temp_coef), int(temp_every)
        self.widths = (num_heads * 2 * key_dim, num_kv_heads * 2 * key_dim, num_kv_heads * value_dim)
        self.channels = sum(self.widths)
        n = self.names
        biases = [n.get("q_bias"), n.get("k_bias"), n.get("v_bias")]
        self.qkv = Linear(list(zip((n["q"], n["k"], n["v"]), self.widths)), hidden_size,
                          bias_names=biases if any(biases) else None)
        self.o = Linear([(n["out"], hidden_size)], num_heads * value_dim,
                        bias_names=[n["out_bias"]] if n.get("out_bias") else None)

    def parts(self) -> List[Part]:
        return [self.qkv, self.o]

    def weight_specs(self) -> List[WeightSpec]:
        n = self.names
        specs = [WeightSpec(n[k], (self.dk,), "small") for k in ("lq1", "lk1", "lq2", "lk2")]
        if self.taps:
            specs += [WeightSpec(n[k], (w, self.taps), "conv_taps") for k, w in zip(("q_conv", "k_conv", "v_conv"), self.widths)]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        f = lambda k: tensors[self.names[k]].to(torch.float32)
        lam = torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum()) + self.diff
        self.lam = float(lam.item())
        if self.taps:
            self.conv_w = torch.cat([f("q_conv"), f("k_conv"), f("v_conv")], 0).contiguous()
        else:
            # without a convolution the same kernel adds the biases: one tap of weight 1
            self.conv_w = torch.ones((self.channels, 1), dtype=torch.float32, device=rt.device)

    def cache_needs(self) -> CacheNeeds:
        state = ()
        if self.taps > 1:
            state = (("conv", StateSpec((self.taps - 1, self.channels), torch.float32)),)
        return CacheNeeds(streams=(("k", StreamSpec(2 * self.nkv * _pad16(self.dk))),
                                   ("v", StreamSpec(self.nkv * _pad16(self.dv)))), state=state)

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        ops.reserve_attention_general(ws, rt.dtype, 2 * self.nh, 2 * self.nkv, self.dv, _pad16(self.dv), rt.max_seq_len,
                                      max_step_tokens)

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True):
        if not writes_cache:
            raise ValueError("differential attention: a run that reads another run's cache has no convolution state "
                             "of its own")
        n, H, G, dk, dv = h.shape[0], self.nh, self.nkv, self.dk, self.dv
        with ctx.timed("attn_qkv_rope"):
            qkv = self.qkv.forward(h, ctx, "dattn.qkv")
            mixed = ctx.ws.get("dattn.conv", (n, self.channels), torch.float32)
            ops.conv_silu(qkv, self.conv_w, None, cache.state.get("conv"), mixed, ctx.cu_q, ctx.seq_slot, max(ctx.q_lens),
                          update_state=True, in_bias=self.qkv.bias, activation=False)
            q = ctx.ws.get("dattn.q", (n, 2 * H * dk), self.rt.dtype)
            ops.diff_qkv_store(mixed, q, H, G, dk, dv, self.temp_coef, self.temp_every, ctx.positions, ctx.tok_slot,
                               cache.streams["k"], cache.streams["v"], cache.page_table, cache.page_size)
        # the two maps' outputs stay float: where they nearly cancel, their difference would carry bf16's rounding
        # of each, enlarged by the division that follows
        maps = ctx.ws.get("dattn.maps", (n, 2 * H * dv), torch.float32)
        with ctx.timed("attn_core"):
            ops.attention_any(q, maps, 2 * H, 2 * G, dk, dv, self.scale, cache.streams["k"], cache.streams["v"],
                              cache.page_table, cache.page_size, ctx, v_share=2)
        out = ctx.ws.get("dattn.out", (n, H * dv), self.rt.dtype)
        with ctx.timed("attn_combine"):
            ops.diff_combine(maps, out, H, G, dv, self.lam, self.eps, 1.0 - self.diff)
        with ctx.timed("attn_o"):
            branch = self.o.forward(out, ctx, "dattn.o", out_dtype=torch.float32, partials=True)
        return BiasedBranch(branch, self.o.bias, ctx, "dattn.o") if self.o.bias is not None else branch
