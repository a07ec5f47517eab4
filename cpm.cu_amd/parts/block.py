"""Arrangement of a layer's parts around the residual stream.

Pre-norm with scaled residual branches: x += s * Mixer(norm1(x)); x += s *
FeedForward(norm2(x)).  As in the reference each branch is added by the norm
that follows it (src/model/minicpm4/minicpm4_layer.cuh:42-62), so a block
leaves its feed-forward branch pending for the next block's first norm (or the
model's final norm).
"""
from __future__ import annotations

from typing import List, Optional

from ..cache.paged import CacheView
import torch

from .. import ops
from .base import (BLOCKS, BiasedBranch, Block, DeferredBranch, FeedForward, Mixer, Norm, NormedBranch, Part,
                   ResidualStream, Runtime, StepContext, StreamsBranch, WeightSpec, branch_for, branch_tensor,
                   forward_declares)
from .linear import Linear


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ff_norm: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None, residual_scale: float = 1.0):
        if (feed_forward is None) != (ff_norm is None):
            raise ValueError("pre_norm: a feed-forward comes with its norm, or neither is given")
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ff_norm = ff_norm
        self.feed_forward = feed_forward
        self.residual_scale = float(residual_scale)
        # a part whose forward can leave its last product to the norm after it is asked to; the class that
        # defines ``forward`` says so itself, so a subclass with a forward of its own is asked only if it
        # declares the same
        self._mixer_defers = forward_declares(mixer, "can_defer_last")
        self._ff_defers = feed_forward is not None and forward_declares(feed_forward, "can_defer_last")

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer] + ([self.ff_norm, self.feed_forward] if self.feed_forward is not None else [])

    @staticmethod
    def _normed(norm: Norm, deferred: bool, x, branch, branch_scale, ctx):
        """The normed rows and None, or (if the consumer finishes the norm itself) the rows without the norm's
        row factor and that factor's ingredients."""
        branch = branch_for(norm, branch)
        # a norm that takes a branch's last product over runs it in the same kernel: the label says so
        label = "norm+" + branch.tag.split(".")[-1] if isinstance(branch, DeferredBranch) else "norm"
        with ctx.timed(label):
            if deferred:
                hs = norm.forward_unscaled(x, branch, branch_scale, ctx, tag="block.h")
                if hs is not None:
                    return hs
            return norm.forward(x, branch, branch_scale, ctx, tag="block.h"), None

    def _mix(self, stream, ctx, cache, writes_cache):
        n = stream.x.shape[0]
        h, rs = self._normed(self.mixer_norm, self.mixer.takes_row_scale(n, ctx, cache, writes_cache),
                             stream.x, stream.take_pending(), stream.pending_scale, ctx)
        kw = {"defer_last": True} if self._mixer_defers else {}
        if rs is not None:
            kw["row_scale"] = rs
        return self.mixer.forward(h, ctx, cache, writes_cache, **kw)

    def _feed(self, stream, a, ctx):
        n = stream.x.shape[0]
        h, rs = self._normed(self.ff_norm, self.feed_forward.takes_row_scale(n, ctx),
                             stream.x, a, self.residual_scale, ctx)
        kw = {"defer_last": True} if self._ff_defers else {}
        if rs is not None:
            kw["row_scale"] = rs
        return self.feed_forward.forward(h, ctx, **kw)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        # the reference's timer labels distinguish prefill from decode and attention from feed-forward
        # (src/model/minicpm4/minicpm4_layer.cuh:46-83); the parts inside time their own kernels by class
        with ctx.timed("attn"):
            a = self._mix(stream, ctx, cache, writes_cache)
        if self.feed_forward is None:           # a layer without a feed-forward leaves its mixer's branch pending
            stream.pending = a
        else:
            with ctx.timed("ffn"):
                stream.pending = self._feed(stream, a, ctx)
        stream.pending_scale = self.residual_scale


@BLOCKS.register("sandwich_norm")
class SandwichNormBlock(Block):
    """A norm before and after every sub-layer: x += post1(Mixer(norm1(x))); x += post2(FeedForward(norm2(x))).
    A layer may have no feed-forward.  The branch with its post-norm is left pending (NormedBranch) for the
    norm that follows, which adds it into the residual while it norms the sum."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_post_norm: Norm, ff_norm: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None, ff_post_norm: Optional[Norm] = None):
        if (feed_forward is None) != (ff_norm is None) or (feed_forward is None) != (ff_post_norm is None):
            raise ValueError("sandwich_norm: a feed-forward comes with both of its norms, or none of the three is given")
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ff_norm, self.feed_forward, self.ff_post_norm = ff_norm, feed_forward, ff_post_norm

    def parts(self) -> List[Part]:
        out = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        if self.feed_forward is not None:
            out += [self.ff_norm, self.feed_forward, self.ff_post_norm]
        return out

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        with ctx.timed("attn"):
            with ctx.timed("norm"):
                h = self.mixer_norm.forward(stream.x, branch_for(self.mixer_norm, stream.take_pending()),
                                            stream.pending_scale, ctx, tag="block.h")
            a = NormedBranch(self.mixer.forward(h, ctx, cache, writes_cache), self.mixer_post_norm, ctx, "block.post")
        if self.feed_forward is None:
            stream.pending = a
        else:
            with ctx.timed("ffn"):
                with ctx.timed("norm"):
                    h = self.ff_norm.forward(stream.x, branch_for(self.ff_norm, a), 1.0, ctx, tag="block.h")
                stream.pending = NormedBranch(self.feed_forward.forward(h, ctx), self.ff_post_norm, ctx, "block.post")
        stream.pending_scale = 1.0


@BLOCKS.register("parallel_gated")
class ParallelGatedBlock(Block):
    """One norm a layer, both sub-layers read its output, and each sub-layer's result passes a gate that is a
    projection of the same rows: with h = norm(x),

        x += sigmoid(G1 h + g1) * Mixer(h) + sigmoid(G2 h + g2) * FeedForward(h)

    element by element.  A layer may have no feed-forward (the second term and its gate are then absent).  The
    two gates are one stacked product; the sum is left pending (float) for the norm that follows.
    ``gate_names``: checkpoint tensors (weight, bias) of the mixer's gate and, with a feed-forward, of its gate."""

    def __init__(self, norm: Norm, mixer: Mixer, feed_forward: Optional[FeedForward], hidden_size: int,
                 gate_names: List[tuple]):
        if len(gate_names) != (2 if feed_forward is not None else 1):
            raise ValueError("parallel_gated: one gate (weight, bias) for every sub-layer")
        self.norm, self.mixer, self.feed_forward, self.hidden_size = norm, mixer, feed_forward, hidden_size
        self.gates = Linear([(w, hidden_size) for w, _ in gate_names], hidden_size, bias_names=[b for _, b in gate_names])

    def parts(self) -> List[Part]:
        return [self.norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else []) + [self.gates]

    @staticmethod
    def _with_bias(branch):
        if isinstance(branch, BiasedBranch):
            return branch.branch, branch.bias
        return branch_tensor(branch), None

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        with ctx.timed("norm"):
            h = self.norm.forward(stream.x, branch_for(self.norm, stream.take_pending()), stream.pending_scale, ctx,
                                  tag="block.h")
        with ctx.timed("attn"):
            a, a_bias = self._with_bias(self.mixer.forward(h, ctx, cache, writes_cache))
        f = f_bias = None
        if self.feed_forward is not None:
            with ctx.timed("ffn"):
                f, f_bias = self._with_bias(self.feed_forward.forward(h, ctx))
        with ctx.timed("gates"):
            few = h.shape[0] <= ops.SKINNY_MAX_ROWS
            g = self.gates.forward(h, ctx, "block.gates", out_dtype=torch.float32 if few else None)
            out = ctx.ws.get("block.gated", (h.shape[0], self.hidden_size), torch.float32)
            ops.gated_branches(g, self.gates.bias, a, a_bias, f, f_bias, out)
        stream.pending = out
        stream.pending_scale = 1.0


@BLOCKS.register("parallel_scaled")
class ParallelScaledBlock(Block):
    """One norm a layer, both sub-layers read its output, and each sub-layer's result is multiplied element by
    element by a learned vector (a layer scale) before the two join the residual: with h = norm(x),

        x += s1 * Mixer(h) + s2 * FeedForward(h)

    A layer may have no feed-forward (the second term and its vector are then absent).  The sum is left pending
    (float) for the norm that follows.  ``scale_names``: checkpoint tensors of s1 and, with a feed-forward, s2."""

    def __init__(self, norm: Norm, mixer: Mixer, feed_forward: Optional[FeedForward], hidden_size: int,
                 scale_names: List[str]):
        if len(scale_names) != (2 if feed_forward is not None else 1):
            raise ValueError("parallel_scaled: one scale vector for every sub-layer")
        self.norm, self.mixer, self.feed_forward, self.hidden_size = norm, mixer, feed_forward, hidden_size
        self.scale_names = list(scale_names)

    def parts(self) -> List[Part]:
        return [self.norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(name, (self.hidden_size,), "norm") for name in self.scale_names]

    def bind(self, tensors, rt: Runtime):
        self.scales = [tensors[name].to(torch.float32).contiguous() for name in self.scale_names]

    @staticmethod
    def _with_bias(branch):
        if isinstance(branch, BiasedBranch):
            return branch.branch, branch.bias
        return branch_tensor(branch), None

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        with ctx.timed("norm"):
            h = self.norm.forward(stream.x, branch_for(self.norm, stream.take_pending()), stream.pending_scale, ctx,
                                  tag="block.h")
        with ctx.timed("attn"):
            a, a_bias = self._with_bias(self.mixer.forward(h, ctx, cache, writes_cache))
        f = f_bias = None
        if self.feed_forward is not None:
            with ctx.timed("ffn"):
                f, f_bias = self._with_bias(self.feed_forward.forward(h, ctx))
        with ctx.timed("layer_scale"):
            out = ctx.ws.get("block.scaled", (h.shape[0], self.hidden_size), torch.float32)
            ops.scaled_branches(a, a_bias, self.scales[0], 1.0, f, f_bias, self.scales[1] if f is not None else None, 1.0,
                                out)
        stream.pending = out
        stream.pending_scale = 1.0


@BLOCKS.register("hyper_connections")
class HyperConnectionBlock(Block):
    """Pre-norm sub-layers over a residual of S streams (hyper-connections).  Sub-layer q (1: mixer, 2:
    feed-forward, which a layer may lack) has numbers in[S], out[S] and mix[S, S] of its own:

        u = sum_s in[s] x_s;   y = sub(norm(u));   x_t <- sum_s mix[s, t] x_s + out[t] * y    (all t at once)

    The result is left pending as a StreamsBranch and added by the norm that follows, which reads the streams with
    the next sub-layer's ``in`` in the same pass (Norm.forward_streams).
    ``names``: for each sub-layer the checkpoint tensors (in, out, mix)."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, streams: int, names: List[tuple], ff_norm: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None):
        if (feed_forward is None) != (ff_norm is None):
            raise ValueError("hyper_connections: a feed-forward comes with its norm, or neither is given")
        if len(names) != (2 if feed_forward is not None else 1):
            raise ValueError("hyper_connections: tensors (in, out, mix) for every sub-layer")
        if streams < 1:
            raise ValueError(f"hyper_connections: {streams} streams")
        self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward = mixer_norm, mixer, ff_norm, feed_forward
        self.streams, self.names = int(streams), [tuple(t) for t in names]

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer] + ([self.ff_norm, self.feed_forward] if self.feed_forward is not None else [])

    def weight_specs(self) -> List[WeightSpec]:
        S, specs = self.streams, []
        for read, out, mix in self.names:
            specs += [WeightSpec(read, (S,), "stream_read"), WeightSpec(out, (S,), "norm"), WeightSpec(mix, (S, S), "stream_mix")]
        return specs

    def bind(self, tensors, rt: Runtime):
        f = lambda name: tensors[name].to(torch.float32).contiguous()
        self.numbers = [(f(read), f(out), f(mix)) for read, out, mix in self.names]

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        x = stream.x
        if x.dim() != 3 or x.shape[0] != self.streams:
            raise ValueError(f"hyper_connections: the residual has shape {tuple(x.shape)}, {self.streams} streams expected")
        read, out, mix = self.numbers[0]
        with ctx.timed("attn"):
            with ctx.timed("norm"):
                h = self.mixer_norm.forward_streams(x, stream.take_pending(), read, ctx, tag="block.h")
            pending = StreamsBranch(self.mixer.forward(h, ctx, cache, writes_cache), mix, out)
        if self.feed_forward is not None:
            read, out, mix = self.numbers[1]
            with ctx.timed("ffn"):
                with ctx.timed("norm"):
                    h = self.ff_norm.forward_streams(x, pending, read, ctx, tag="block.h")
                pending = StreamsBranch(self.feed_forward.forward(h, ctx), mix, out)
        stream.pending = pending
        stream.pending_scale = 1.0
