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

Two things may be low-rank products instead of rows of the input projection (``names`` then holds a pair of tensors
for them): the decay, which is then a number a head *and key channel*, a = W_up (W_down h) of heads*dim numbers with a
dt_bias as long, g acting on the rows of S (S <- diag(g) S); and the output gate, W_up (W_down h) of heads*vdim
numbers.  ``gate_activation`` chooses silu or sigmoid for the gate.

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
                 value_dim: int, conv_taps: int, eps: float, gate_activation: str = "silu", decay_rank: int = 0,
                 gate_rank: int = 0):
        """``names``: checkpoint tensors for 'q', 'k', 'v', 'beta' (b), 'q_conv', 'k_conv', 'v_conv', 'A_log',
        'dt_bias', 'norm', 'out', and 'gate', 'decay' (a) as rows of the input projection or, with ``gate_rank`` /
        ``decay_rank`` > 0, 'gate_down', 'gate_up' / 'decay_down', 'decay_up' as products of that rank (the decay
        then a number a head and key channel)."""
        if heads % kv_heads:
            raise ValueError(f"gated_delta: {heads} heads are not a multiple of {kv_heads} key heads")
        if key_dim > 256:
            raise ValueError(f"gated_delta: a key size of {key_dim} is not supported (at most 256)")
        if conv_taps < 1:
            raise ValueError(f"gated_delta: {conv_taps} convolution taps")
        if gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"gated_delta: gate nonlinearity '{gate_activation}' (silu or sigmoid)")
        if decay_rank < 0 or gate_rank < 0:
            raise ValueError("gated_delta: a rank must not be negative")
        self.names = dict(names)
        self.hidden_size, self.heads, self.kv_heads, self.dk, self.dv = hidden_size, heads, kv_heads, key_dim, value_dim
        self.taps, self.eps = int(conv_taps), float(eps)
        self.gate_activation = gate_activation
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        n = self.names
        self.widths = (kv_heads * key_dim, kv_heads * key_dim, heads * value_dim)
        self.channels = sum(self.widths)
        hv = heads * value_dim
        # the input projection's rows: q, k, v, then what is not low-rank of (gate, decay), then beta, then the
        # low-rank products' first halves
        stacked = [(n["q"], self.widths[0]), (n["k"], self.widths[1]), (n["v"], self.widths[2])]
        off = self.channels
        self.g_off = self.a_off = None
        if not self.gate_rank:
            stacked.append((n["gate"], hv))
            self.g_off, off = off, off + hv
        if not self.decay_rank:
            stacked.append((n["decay"], heads))
            self.a_off, off = off, off + heads
        stacked.append((n["beta"], heads))
        self.b_off, off = off, off + heads
        self.low_off, self.low = off, self.decay_rank + self.gate_rank
        if self.decay_rank:
            stacked.append((n["decay_down"], self.decay_rank))
        if self.gate_rank:
            stacked.append((n["gate_down"], self.gate_rank))
        self.in_proj = Linear(stacked, hidden_size)
        self.out_proj = Linear([(n["out"], hidden_size)], hv)
        # columns of the low-rank products' second halves, side by side: [decay: heads*dim | gate: heads*vdim]
        self.up_decay = heads * key_dim if self.decay_rank else 0
        self.up_width = self.up_decay + (hv if self.gate_rank else 0)

    def parts(self) -> List[Part]:
        return [self.in_proj, self.out_proj]

    def weight_specs(self) -> List[WeightSpec]:
        n = self.names
        specs = [WeightSpec(n[k], (w, self.taps), "conv_taps") for k, w in zip(("q_conv", "k_conv", "v_conv"), self.widths)] + [
            WeightSpec(n["A_log"], (self.heads,), "log_decay"),
            WeightSpec(n["dt_bias"], (self.heads * self.dk if self.decay_rank else self.heads,), "small"),
            WeightSpec(n["norm"], (self.dv,), "norm")]
        if self.decay_rank:
            specs.append(WeightSpec(n["decay_up"], (self.heads * self.dk, self.decay_rank)))
        if self.gate_rank:
            specs.append(WeightSpec(n["gate_up"], (self.heads * self.dv, self.gate_rank)))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        f = lambda k: tensors[self.names[k]].to(torch.float32).contiguous()
        self.conv_w = torch.cat([f("q_conv"), f("k_conv"), f("v_conv")], 0).contiguous()
        self.A_log, self.dt_bias = f("A_log"), f("dt_bias")
        self.norm_w = f("norm").repeat(self.heads).contiguous()       # shared by the heads
        self.rt = rt
        self.up_w = None
        if self.low:
            # both second halves as one product: the weights stand corner to corner, zeros elsewhere
            w = torch.zeros((self.up_width, self.low), dtype=torch.float32, device=self.conv_w.device)
            if self.decay_rank:
                w[:self.up_decay, :self.decay_rank] = f("decay_up")
            if self.gate_rank:
                w[self.up_decay:, self.decay_rank:] = f("gate_up")
            self.up_w = w.to(rt.dtype).contiguous()

    def cache_needs(self) -> CacheNeeds:
        state = [("delta", StateSpec((self.heads, self.dv, self.dk), torch.float32))]
        if self.taps > 1:
            state.append(("conv", StateSpec((self.taps - 1, self.channels), torch.float32)))
        return CacheNeeds(state=tuple(state))

    def _low_rank(self, u: torch.Tensor, ctx: StepContext):
        """(decay rows float32 [n, heads*dim] or None, gate rows [n, heads*vdim] or None) of the low-rank products."""
        n = u.shape[0]
        low = ctx.ws.get("delta.low", (n, self.low), self.rt.dtype)
        low.copy_(u[:, self.low_off:self.low_off + self.low])
        few = n <= ops.SKINNY_MAX_ROWS or self.rt.dtype == torch.float32
        up = ctx.ws.get("delta.up", (n, self.up_width), torch.float32 if few else self.rt.dtype)
        ops.linear(low, self.up_w, up)
        decay = gate = None
        if self.decay_rank:
            decay = up[:, :self.up_decay]
            if decay.dtype != torch.float32:
                wide = ctx.ws.get("delta.decay", (n, self.up_decay), torch.float32)
                wide.copy_(decay)
                decay = wide
        if self.gate_rank:
            gate = up[:, self.up_decay:]
        return decay, gate

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        n, hv = h.shape[0], self.heads * self.dv
        with ctx.timed("delta_in"):
            u = self.in_proj.forward(h, ctx, "delta.in")
            decay = gate = None
            if self.low:
                decay, gate = self._low_rank(u, ctx)
            if gate is None:
                gate = u[:, self.g_off:self.g_off + hv]
        qkv = ctx.ws.get("delta.qkv", (n, self.channels), torch.float32)
        y = ctx.ws.get("delta.y", (n, hv), torch.float32)
        with ctx.timed("delta_conv"):
            ops.conv_silu(u[:, :self.channels], self.conv_w, None, cache.state.get("conv"), qkv, ctx.cu_q, ctx.seq_slot,
                          max(ctx.q_lens), update_state=writes_cache)
        with ctx.timed("delta_scan"):
            ops.delta_scan(qkv, u, self.a_off or 0, self.b_off, self.dt_bias, self.A_log, cache.state["delta"], y, ctx.cu_q,
                           ctx.seq_slot, self.heads, self.kv_heads, self.dk, self.dv, self.dk ** -0.5,
                           write_state=writes_cache, rule="channel" if self.decay_rank else "delta",
                           channel_decay=decay)
        gated = ctx.ws.get("delta.gated", (n, hv), self.rt.dtype)
        with ctx.timed("delta_norm"):
            ops.rms_norm_groups(y, self.norm_w, self.eps, gated, groups=self.heads, gate=gate,
                                gate_after="silu" if self.gate_activation == "silu" else True)
        with ctx.timed("delta_out"):
            return self.out_proj.forward(gated, ctx, "delta.out", out_dtype=torch.float32, partials=True)
