"""Gated feed-forward: down( act(x Wg^T) * (x Wu^T) ), act = SiLU (or the tanh form of GELU, or a clamped swish).

gate and up are one stacked product, gate rows first (src/model/ffn.cuh:31-59,
77-84); silu(g) * u in float (src/model/activation.cuh:6-18).
"""
from __future__ import annotations

from typing import List, Mapping, Optional, Tuple

import torch

from .. import ops
from .base import FEED_FORWARDS, DeferredBranch, FeedForward, Part, Runtime, StepContext, WeightSpec
from .linear import Linear


@FEED_FORWARDS.register("gated")
@FEED_FORWARDS.register("gated_silu")
class GatedFFN(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, names: Optional[Mapping[str, str]] = None,
                 activation="silu"):
        """``names``: the checkpoint tensors for 'gate', 'up', 'down' behind the prefix (default: the MiniCPM
        checkpoint's gate_proj.weight, up_proj.weight, down_proj.weight).  ``activation``: the gate's
        nonlinearity, 'silu' or 'gelu_tanh' (0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))), or
        ('clamped_swish', limit): g <- min(g, limit), up <- clamp(up, -limit, limit), and the pair's product is
        g sigmoid(1.702 g) (up + 1)."""
        try:
            self.activation = ops.gate_activation(activation)
        except ops.KernelError as e:
            raise ValueError(f"feed-forward: {e}") from None
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        names = names or {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        self.gate_up = Linear([(prefix + names["gate"], intermediate_size),
                               (prefix + names["up"], intermediate_size)], hidden_size)
        self.down = Linear([(prefix + names["down"], hidden_size)], intermediate_size)

    def parts(self) -> List[Part]:
        return [self.gate_up, self.down]

    def takes_row_scale(self, n: int, ctx: StepContext) -> bool:
        return self.gate_up.gated_takes_row_scale(n)

    can_defer_last = True

    def forward(self, h: torch.Tensor, ctx: StepContext, row_scale=None, defer_last: bool = False):
        with ctx.timed("ffn_gate_up"):
            act = self.gate_up.forward_gated(h, ctx, "ffn.gate_up", row_scale=row_scale, activation=self.activation)
        if defer_last and self.down.defers(act):
            return DeferredBranch(self.down, act, ctx, "ffn.down")
        with ctx.timed("ffn_down"):
            return self.down.forward(act, ctx, "ffn.down", out_dtype=torch.float32, partials=True)


@FEED_FORWARDS.register("poly_norm")
class PolyNormFFN(FeedForward):
    """down( act(up x) ) with the PolyNorm activation act(z) = a N(z) + b N(z^2) + c N(z^3) + e: powers element by
    element, N divides a token's vector by its root mean square sqrt(mean(v^2) + eps); the four numbers are a
    checkpoint tensor.  The statistics and the polynomial are computed in float."""

    def __init__(self, up_name: str, down_name: str, act_name: str, hidden_size: int, intermediate_size: int, eps: float):
        self.hidden_size, self.intermediate_size, self.eps = hidden_size, intermediate_size, float(eps)
        self.act_name = act_name
        self.up = Linear([(up_name, intermediate_size)], hidden_size)
        self.down = Linear([(down_name, hidden_size)], intermediate_size)

    def parts(self) -> List[Part]:
        return [self.up, self.down]

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.act_name, (4,), "poly_coefficients")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.coef = tensors[self.act_name].to(torch.float32).contiguous()
        self.rt = rt

    def forward(self, h: torch.Tensor, ctx: StepContext):
        with ctx.timed("ffn_up"):
            # few rows: float out of the decode product (one slice: its many output rows fill the chip without a
            # split of K); many rows: the library's product in the engine's element type
            few = h.shape[0] <= ops.SKINNY_MAX_ROWS
            z = self.up.forward(h, ctx, "ffn.up", out_dtype=torch.float32 if few else None)
        act = ctx.ws.get("ffn.act", (h.shape[0], self.intermediate_size), self.rt.dtype)
        with ctx.timed("ffn_act"):
            ops.poly_norm(z, self.coef, self.eps, act)
        with ctx.timed("ffn_down"):
            return self.down.forward(act, ctx, "ffn.down", out_dtype=torch.float32, partials=True)


@FEED_FORWARDS.register("routed_experts")
class RoutedExpertsFFN(FeedForward):
    """A mixture of small gated feed-forwards (no biases), of which every token uses ``top``.

    Router: logits z = W_router h in float, scores s = softmax(z) over all experts (``score`` 'sigmoid': sigmoid of
    every logit alone).  The choice goes by s + a correction a expert (a checkpoint tensor; the weights use s without
    it).  With ``groups`` = (count, keep) the experts form ``count`` equal groups of neighbours, a group's score is
    its largest choice score (``group_score`` 'top2_sum': the sum of its two largest), and only experts of the
    ``keep`` best groups can be chosen.  The chosen experts' outputs are added with weights s / (sum of the chosen s +
    1e-20) * ``weight_scale``.  A shared expert (``shared_size``) runs for every token and is added, times
    sigmoid(w . h), one number a token, if ``names`` holds 'shared_scale'.  ``activation`` / ``shared_activation``:
    the experts' and the shared expert's nonlinearity as GatedFFN takes it.

    ``names``: 'router', 'correction' (or absent), 'expert' (a format with {e} for the expert's number and {part}
    for gate / up / down), and for the shared expert 'shared_gate', 'shared_up', 'shared_down', 'shared_scale'."""

    def __init__(self, names: Mapping[str, str], hidden_size: int, expert_size: int, experts: int, top: int,
                 groups: Optional[Tuple[int, int]] = None, shared_size: Optional[int] = None, score: str = "softmax",
                 group_score: str = "max", weight_scale: float = 1.0, activation="silu", shared_activation=None):
        if experts > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"routed_experts: {experts} experts (up to {ops.MOE_MAX_EXPERTS} are taken)")
        if not 0 < top <= experts:
            raise ValueError(f"routed_experts: {top} of {experts} experts a token")
        if groups is not None:
            count, keep = groups
            if count <= 0 or experts % count or not 0 < keep <= count or top > keep * (experts // count):
                raise ValueError(f"routed_experts: {experts} experts in {count} groups, {keep} kept, {top} chosen")
        if score not in ops.MOE_SCORES or group_score not in ops.MOE_GROUP_SCORES:
            raise ValueError(f"routed_experts: score '{score}' ({sorted(ops.MOE_SCORES)}) or group score "
                             f"'{group_score}' ({sorted(ops.MOE_GROUP_SCORES)})")
        try:
            self.activation = ops.gate_activation(activation)
        except ops.KernelError as e:
            raise ValueError(f"routed_experts: {e}") from None
        self.score, self.group_score, self.weight_scale = score, group_score, float(weight_scale)
        self.names = dict(names)
        self.hidden_size, self.expert_size, self.experts, self.top = hidden_size, expert_size, experts, top
        self.groups = tuple(groups) if groups is not None else (1, 1)
        self.shared = None
        if shared_size is not None:
            self.shared = GatedFFN("", hidden_size, shared_size, names={"gate": self.names["shared_gate"],
                                                                        "up": self.names["shared_up"],
                                                                        "down": self.names["shared_down"]},
                                   activation=shared_activation if shared_activation is not None else activation)
        self.shared_gated = self.shared is not None and bool(self.names.get("shared_scale"))

    def _expert(self, e: int, part: str) -> str:
        return self.names["expert"].format(e=e, part=part)

    def parts(self) -> List[Part]:
        return [self.shared] if self.shared is not None else []

    def weight_specs(self) -> List[WeightSpec]:
        H, F = self.hidden_size, self.expert_size
        specs = [WeightSpec(self.names["router"], (self.experts, H))]
        if self.names.get("correction"):
            specs.append(WeightSpec(self.names["correction"], (self.experts,), "slight"))
        for e in range(self.experts):
            specs += [WeightSpec(self._expert(e, "gate"), (F, H)), WeightSpec(self._expert(e, "up"), (F, H)),
                      WeightSpec(self._expert(e, "down"), (H, F))]
        if self.shared_gated:
            specs.append(WeightSpec(self.names["shared_scale"], (1, H)))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()
        self.router = f32(self.names["router"])
        self.correction = f32(self.names["correction"]) if self.names.get("correction") else None
        self.shared_scale = f32(self.names["shared_scale"]).reshape(-1) if self.shared_gated else None
        # an expert's gate rows, then its up rows: [E, 2F, H]; down: [E, H, F]
        self.gate_up = torch.stack([torch.cat([tensors[self._expert(e, "gate")], tensors[self._expert(e, "up")]], 0)
                                    for e in range(self.experts)]).to(rt.dtype).contiguous()
        self.down = torch.stack([tensors[self._expert(e, "down")] for e in range(self.experts)]).to(rt.dtype).contiguous()

    def forward(self, h: torch.Tensor, ctx: StepContext):
        n = h.shape[0]
        idx = ctx.ws.get("moe.idx", (n, self.top), torch.int32)
        wts = ctx.ws.get("moe.weights", (n, self.top), torch.float32)
        sg = ctx.ws.get("moe.shared_gate", (n,), torch.float32) if self.shared_gated else None
        logits = ctx.ws.get("moe.logits", (n, self.experts + 1), torch.float32)
        with ctx.timed("moe_route"):
            ops.moe_route(h, self.router, self.correction, self.shared_scale, self.groups[0], self.groups[1], self.top,
                          idx, wts, sg, logits, score=self.score, group_score=self.group_score,
                          weight_scale=self.weight_scale)
        shared = self.shared.forward(h, ctx) if self.shared is not None else None
        act = ctx.ws.get("moe.act", (n, self.top, self.expert_size), self.rt.dtype)
        out = ctx.ws.get("moe.out", (n, self.hidden_size), torch.float32)
        tiles = ops.moe_tiles(n, self.top, self.experts)
        with ctx.timed("moe_experts"):
            # few tokens read an expert's matrices once for every token that chose it; from about one and a half
            # (token, expert) pairs an expert on, most experts are chosen more than once and grouping pays
            grouped = n > ops.SKINNY_MAX_ROWS or 2 * n * self.top >= 3 * self.experts
            if grouped and ops.moe_experts_mfma_ok(h, self.expert_size, tiles):
                # many tokens: experts are shared by many of them; pairs grouped by expert, on the matrix cores
                y = ctx.ws.get("moe.pair_out", (n, self.top, self.hidden_size), torch.bfloat16)
                rows = ctx.ws.get("moe.tile_rows", (tiles * ops.MOE_TILE,), torch.int32)
                tile_expert = ctx.ws.get("moe.tile_expert", (tiles,), torch.int32)
                n_tiles = ctx.ws.get("moe.n_tiles", (1,), torch.int32)
                ops.moe_experts_mfma(h, self.gate_up, self.down, idx, wts, out, act, y, rows, tile_expert, n_tiles,
                                     shared, sg, activation=self.activation)
            else:
                # few tokens: an expert's weights stream once for every token that chose it
                ops.moe_gated(h, self.gate_up, idx, act, activation=self.activation)
                ops.moe_down(act, self.down, idx, wts, out, shared, sg)
        return out
