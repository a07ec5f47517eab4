"""Two mixers side by side: both read the same rows, and the layer's result is the mean of their outputs, each
first divided by its root mean square over the model width and multiplied by a weight of its own:

    y = (left(h) / rms(left(h)) * w_left + right(h) / rms(right(h)) * w_right) / 2

or, with ``scales`` = (a, b) instead of the two norm weights, their plain weighted sum y = a left(h) + b right(h).

The pair owns one cache entry; what the two mixers need of it (per-token streams, fixed-size state, a window) is put
together under the prefixes ``left.`` and ``right.``, and each mixer sees its own part under its own names.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView
from .base import MIXERS, BiasedBranch, Mixer, Part, Runtime, StepContext, WeightSpec, branch_tensor


@MIXERS.register("parallel")
class ParallelMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_norm_name: Optional[str] = None, right_norm_name: Optional[str] = None,
                 hidden_size: int = 0, eps: float = 0.0, scales: Optional[tuple] = None):
        if (scales is None) == (left_norm_name is None) or (left_norm_name is None) != (right_norm_name is None):
            raise ValueError("parallel: either the two norm weights' names or the two numbers of a weighted sum")
        self.left, self.right = left, right
        self.norm_names = (left_norm_name, right_norm_name) if scales is None else ()
        self.scales = (float(scales[0]), float(scales[1])) if scales is not None else None
        self.hidden_size, self.eps = hidden_size, float(eps)
        a, b = left.cache_needs(), right.cache_needs()
        if a.streams and b.streams and (a.window, a.keep_first) != (b.window, b.keep_first):
            raise ValueError("parallel: the two mixers keep different spans of tokens in one cache entry")
        self._needs = CacheNeeds(
            streams=tuple(("left." + k, v) for k, v in a.streams) + tuple(("right." + k, v) for k, v in b.streams),
            state=tuple(("left." + k, v) for k, v in a.state) + tuple(("right." + k, v) for k, v in b.state),
            window=a.window if a.streams else b.window, keep_first=a.keep_first if a.streams else b.keep_first)
        self._views: Dict[int, tuple] = {}

    def parts(self) -> List[Part]:
        return [self.left, self.right]

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(name, (self.hidden_size,), "norm") for name in self.norm_names]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        if self.scales is None:
            self.w_left, self.w_right = (tensors[name].to(torch.float32).contiguous() for name in self.norm_names)
        self.rt = rt

    def cache_needs(self) -> CacheNeeds:
        return self._needs

    def _split(self, cache: CacheView):
        """The entry as each of the two mixers sees it."""
        views = self._views.get(id(cache))
        if views is None or views[0] is not cache:
            def side(prefix):
                pick = lambda d: {k[len(prefix):]: v for k, v in d.items() if k.startswith(prefix)}
                return CacheView(pick(cache.streams), pick(cache.state), cache.page_table, cache.page_size, cache.window,
                                 cache.keep_first)
            views = (cache, side("left."), side("right."))
            self._views[id(cache)] = views
        return views[1], views[2]

    @staticmethod
    def _pieces(branch):
        if isinstance(branch, BiasedBranch):
            return branch.branch, branch.bias
        return branch_tensor(branch), None

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        lv, rv = self._split(cache)
        a, a_bias = self._pieces(self.left.forward(h, ctx, lv, writes_cache))
        b, b_bias = self._pieces(self.right.forward(h, ctx, rv, writes_cache))
        out = ctx.ws.get("parallel.out", (h.shape[0], self.hidden_size), torch.float32)
        with ctx.timed("parallel_join"):
            if self.scales is None:
                ops.pair_norm_mean(a, a_bias, b, b_bias, self.w_left, self.w_right, self.eps, out)
            else:
                ops.scaled_branches(a, a_bias, None, self.scales[0], b, b_bias, None, self.scales[1], out)
        return out
