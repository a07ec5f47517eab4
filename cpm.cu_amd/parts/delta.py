"""Gated delta rule mixer: a linear recurrence whose state is a matrix a head, which decays, corrects what it holds
under the current key and then writes the new value.

One input projection gives [q: kv_heads*dim | k: kv_heads*dim | v: heads*vdim | gate: heads*vdim | a: heads |
b: heads] per token.  q, k and v pass a causal convolution per channel (``conv_taps`` taps, the last one the current
token's, zeros before the sequence's start, no bias) and SiLU.  Per head h, with its q and k from head
h // (heads / kv_heads):

    q <- q / sqrt(sum q^2 + 1e-6) / sqrt(dim),   k <- k / sqrt(sum k^2 + 1e-6)
    beta = sigmoid(b),   g = exp(-exp(A_log[h]) * softplus(a + dt_bias[h]))
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          S: [dim, vdim], zero at the start

so the read-out sees the current token's write.  Each head's o is divided by its root mean square, multiplied by a
weight of vdim numbers shared by the heads and by silu(gate), then projected out.

Everything after the convolution runs in float; S and the convolution's last ``conv_taps - 1`` inputs live as float
fixed-size state in the sequence's cache slot, so a step of any number of tokens continues where the last one ended.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec
from .base import MIXERS, Mixer, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


@MIXERS.register("gated_delta")
class GatedDeltaMixer(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, heads: int, kv_heads: int, key_dim: int,
                 value_dim: int, conv_taps: int, eps: float):
        """``names``: checkpoint tensors for 'q', 'k', 'v', 'gate', 'decay' (a), 'beta' (b), 'q_conv', 'k_conv',
        'v_conv', 'A_log', 'dt_bias', 'norm', 'out'."""
        if heads % kv_heads:
            raise ValueError(f"gated_delta: {heads} heads are not a multiple of {kv_heads} key heads")
        if key_dim > 256:
            raise ValueError(f"gated_delta: a key size of {key_dim} is not supported (at most 256)")
        if conv_taps < 1:
            raise ValueError(f"gated_delta: {conv_taps} convolution taps")
        self.names = dict(names)
        self.hidden_size, self.heads, self.kv_heads, self.dk, self.dv = hidden_size, heads, kv_heads, key_dim, value_dim
        self.taps, self.eps = int(conv_taps), float(eps)
        n = self.names
        self.widths = (kv_heads * key_dim, kv_heads * key_dim, heads * value_dim)
        self.channels = sum(self.widths)
        self.in_proj = Linear([(n["q"], self.widths[0]), (n["k"], self.widths[1]), (n["v"], self.widths[2]),
                               (n["gate"], heads * value_dim), (n["decay"], heads), (n["beta"], heads)], hidden_size)
        self.out_proj = Linear([(n["out"], hidden_size)], heads * value_dim)
        self.g_off = self.channels
        self.a_off = self.channels + heads * value_dim
        self.b_off = self.a_off + heads

    def parts(self) -> List[Part]:
        return [self.in_proj, self.out_proj]

    def weight_specs(self) -> List[WeightSpec]:
        n = self.names
        return [WeightSpec(n[k], (w, self.taps), "conv_taps") for k, w in zip(("q_conv", "k_conv", "v_conv"), self.widths)] + [
            WeightSpec(n["A_log"], (self.heads,), "log_decay"), WeightSpec(n["dt_bias"], (self.heads,), "small"),
            WeightSpec(n["norm"], (self.dv,), "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        f = lambda k: tensors[self.names[k]].to(torch.float32).contiguous()
        self.conv_w = torch.cat([f("q_conv"), f("k_conv"), f("v_conv")], 0).contiguous()
        self.A_log, self.dt_bias = f("A_log"), f("dt_bias")
        self.norm_w = f("norm").repeat(self.heads).contiguous()       # shared by the heads
        self.rt = rt

    def cache_needs(self) -> CacheNeeds:
        state = [("delta", StateSpec((self.heads, self.dv, self.dk), torch.float32))]
        if self.taps > 1:
            state.append(("conv", StateSpec((self.taps - 1, self.channels), torch.float32)))
        return CacheNeeds(state=tuple(state))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        n, hv = h.shape[0], self.heads * self.dv
        with ctx.timed("delta_in"):
            u = self.in_proj.forward(h, ctx, "delta.in")
        qkv = ctx.ws.get("delta.qkv", (n, self.channels), torch.float32)
        y = ctx.ws.get("delta.y", (n, hv), torch.float32)
        with ctx.timed("delta_conv"):
            ops.conv_silu(u[:, :self.channels], self.conv_w, None, cache.state.get("conv"), qkv, ctx.cu_q, ctx.seq_slot,
                          max(ctx.q_lens), update_state=writes_cache)
        with ctx.timed("delta_scan"):
            ops.delta_scan(qkv, u, self.a_off, self.b_off, self.dt_bias, self.A_log, cache.state["delta"], y, ctx.cu_q,
                           ctx.seq_slot, self.heads, self.kv_heads, self.dk, self.dv, self.dk ** -0.5,
                           write_state=writes_cache)
        gated = ctx.ws.get("delta.gated", (n, hv), self.rt.dtype)
        with ctx.timed("delta_norm"):
            ops.rms_norm_groups(y, self.norm_w, self.eps, gated, groups=self.heads, gate=u[:, self.g_off:self.g_off + hv],
                                gate_after="silu")
        with ctx.timed("delta_out"):
            return self.out_proj.forward(gated, ctx, "delta.out", out_dtype=torch.float32, partials=True)
