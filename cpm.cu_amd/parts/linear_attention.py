"""Linear attention with a fixed decay a head: a recurrence whose state is a matrix a head and which has neither a
softmax nor a denominator,

    S <- d_h S + k v^T;   o = S^T q          S: [dim, vdim], zero at the start; d_h a constant of the configuration

One input projection gives [q: heads*dim | k: heads*dim | v: heads*vdim | gate: heads*vdim] per token.  What stands
between the projection and the recurrence, and between the recurrence and the output projection, are parameters:

    ``activation``       None, or 'silu' on q, k and v;
    ``position``         a rotation of the first features of q and k heads (of the pairs that ``position.pairs``
                         says), or None;
    ``key_scale``        k is multiplied by it after the rotation;
    ``norm``             'heads': each head's o is divided by its own root mean square; 'all': the heads side by side are
                         divided by one root mean square; with 'norm' in ``names`` the result is multiplied by that
                         tensor (heads*vdim numbers);
    ``gate_activation``  the normed heads are multiplied by silu(gate) or sigmoid(gate).

Everything behind the projection runs in float; S lives as float fixed-size state in the sequence's cache slot, so a
step of any number of tokens continues where the last one ended.
"""
from __future__ import annotations

from typing import List, Mapping, Optional, Sequence

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec
from .base import MIXERS, Mixer, Part, PositionEncoding, Runtime, StepContext, WeightSpec
from .linear import Linear


@MIXERS.register("decay_linear_attention")
class DecayLinearAttention(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, heads: int, key_dim: int, value_dim: int,
                 decay: Sequence[float], eps: float, activation: Optional[str] = None,
                 position: Optional[PositionEncoding] = None, key_scale: float = 1.0,
                 norm: str = "heads", gate_activation: str = "silu"):
        """``names``: checkpoint tensors for 'q', 'k', 'v', 'gate', 'out' and optionally 'norm'."""
        if len(decay) != heads:
            raise ValueError(f"decay_linear_attention: {len(decay)} decays for {heads} heads")
        if any(not 0.0 <= float(d) <= 1.0 for d in decay):
            raise ValueError(f"decay_linear_attention: decays must lie in 0..1, got {list(decay)}")
        if key_dim > 256:
            raise ValueError(f"decay_linear_attention: a key size of {key_dim} is not supported (at most 256)")
        if activation not in (None, "silu"):
            raise ValueError(f"decay_linear_attention: activation '{activation}' (none or silu)")
        if norm not in ("heads", "all"):
            raise ValueError(f"decay_linear_attention: norm over '{norm}' (heads or all)")
        if gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"decay_linear_attention: gate nonlinearity '{gate_activation}' (silu or sigmoid)")
        self.names = dict(names)
        self.hidden_size, self.heads, self.dk, self.dv = hidden_size, heads, key_dim, value_dim
        self.decay = [float(d) for d in decay]
        self.eps, self.activation, self.position = float(eps), activation, position
        self.interleaved = position is not None and position.pairs == "interleaved"
        self.key_scale = float(key_scale)
        self.norm_groups = heads if norm == "heads" else 1
        self.gate_activation = gate_activation
        n, hk, hv = self.names, heads * key_dim, heads * value_dim
        self.in_proj = Linear([(n["q"], hk), (n["k"], hk), (n["v"], hv), (n["gate"], hv)], hidden_size)
        self.out_proj = Linear([(n["out"], hidden_size)], hv)
        self.g_off = 2 * hk + hv

    def parts(self) -> List[Part]:
        return [self.in_proj, self.out_proj] + ([self.position] if self.position is not None else [])

    def weight_specs(self) -> List[WeightSpec]:
        if self.names.get("norm"):
            return [WeightSpec(self.names["norm"], (self.heads * self.dv,), "norm")]
        return []

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        self.decays = torch.tensor(self.decay, dtype=torch.float32, device=rt.device)
        self.norm_w = (tensors[self.names["norm"]].to(torch.float32).contiguous() if self.names.get("norm") else None)

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state=(("memory", StateSpec((self.heads, self.dv, self.dk), torch.float32)),))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        n, hk, hv = h.shape[0], self.heads * self.dk, self.heads * self.dv
        inv_freq = None
        if self.position is not None:
            rot = self.position.rotary_params()
            if rot is None or rot[1] != 1.0:
                raise ValueError("decay_linear_attention: the position encoding must be a plain rotation")
            inv_freq = rot[0]
        with ctx.timed("linattn_in"):
            u = self.in_proj.forward(h, ctx, "linattn.in")
        qkv = ctx.ws.get("linattn.qkv", (n, 2 * hk + hv), torch.float32)
        y = ctx.ws.get("linattn.y", (n, hv), torch.float32)
        with ctx.timed("linattn_prepare"):
            ops.linear_attention_prepare(u, 0, hk, 2 * hk, qkv, self.heads, self.dk, self.dv, self.activation == "silu",
                                         ctx.positions, inv_freq, self.interleaved, self.key_scale)
        with ctx.timed("linattn_scan"):
            ops.delta_scan(qkv, None, 0, 0, None, self.decays, cache.state["memory"], y, ctx.cu_q, ctx.seq_slot,
                           self.heads, self.heads, self.dk, self.dv, 1.0, write_state=writes_cache, rule="decay")
        gated = ctx.ws.get("linattn.gated", (n, hv), self.rt.dtype)
        with ctx.timed("linattn_norm"):
            ops.rms_norm_groups(y, self.norm_w, self.eps, gated, groups=self.norm_groups,
                                gate=u[:, self.g_off:self.g_off + hv],
                                gate_after="silu" if self.gate_activation == "silu" else True)
        with ctx.timed("linattn_out"):
            return self.out_proj.forward(gated, ctx, "linattn.out", out_dtype=torch.float32, partials=True)
