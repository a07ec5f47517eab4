"""Token embedding (times its scale) and the output head.

x[t] = E[id_t] * scale_emb (src/model/embedding.cuh:7-20, 49-52), optionally plus a row of a second table chosen
by a hash of the previous token and the current one (a bigram embedding); logits =
(y * head_scale) . W^T with the head reading the unscaled table when the
embeddings are tied (src/model/linear.cuh:86-105, cpmcu/llm.py:136-137).
"""
from __future__ import annotations

from typing import List, Mapping, Optional, Tuple

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec
from .base import Part, Runtime, StepContext, WeightSpec


class TokenEmbedding(Part):
    """``bigram`` = (tensor name, buckets, mul_prev, mul_cur): a table of buckets + 1 rows is added,
    x[t] += B[(id_(t-1) * mul_prev + id_t * mul_cur) mod buckets], and a sequence's first token reads the last row.
    The previous token is part of a sequence's state: the embedding then asks for a cache entry of its own that
    holds one integer a slot (``cache_needs``), so that a step of any number of tokens goes on where the last ended."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 bigram: Optional[Tuple[str, int, int, int]] = None):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.table: Optional[torch.Tensor] = None
        self.bigram = None
        if bigram is not None:
            bname, buckets, mul_prev, mul_cur = bigram
            if buckets <= 0 or mul_prev < 0 or mul_cur < 0:
                raise ValueError(f"embedding: a bigram table of {buckets} buckets with multipliers {mul_prev}, {mul_cur}")
            if (vocab_size - 1) * (mul_prev + mul_cur) >= 2 ** 62:
                raise ValueError("embedding: the bigram hash exceeds 64 bits")
            self.bigram = (str(bname), int(buckets), int(mul_prev), int(mul_cur))
        self.bigram_table: Optional[torch.Tensor] = None

    def weight_specs(self) -> List[WeightSpec]:
        specs = [WeightSpec(self.name, (self.vocab_size, self.hidden_size), "table")]
        if self.bigram is not None:
            specs.append(WeightSpec(self.bigram[0], (self.bigram[1] + 1, self.hidden_size), "table"))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.table = tensors[self.name].to(rt.dtype).contiguous()
        if self.bigram is not None:
            self.bigram_table = tensors[self.bigram[0]].to(rt.dtype).contiguous()

    def cache_needs(self) -> Optional[CacheNeeds]:
        """What the embedding keeps per sequence (None: nothing)."""
        if self.bigram is None:
            return None
        return CacheNeeds(state=(("previous_token", StateSpec((), torch.int32)),))

    def forward(self, ctx: StepContext, cache: Optional[CacheView] = None) -> torch.Tensor:
        x = ctx.ws.get("residual", (ctx.n_tokens, self.hidden_size), torch.float32)
        ops.embed(self.table, ctx.token_ids, x, self.scale)
        if self.bigram is not None:
            _, buckets, mul_prev, mul_cur = self.bigram
            ops.bigram_add(self.bigram_table, ctx.token_ids, ctx.positions, ctx.tok_slot, cache.state["previous_token"],
                           ctx.cu_q, ctx.seq_slot, x, buckets, mul_prev, mul_cur)
        return x


class LMHead(Part):
    def __init__(self, name: str, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 tied_to: Optional[TokenEmbedding] = None, softcap: Optional[float] = None):
        """``softcap`` c: the logits leave as c * tanh(logits / c)."""
        if softcap is not None and not softcap > 0:
            raise ValueError(f"head: a logit cap of {softcap}")
        self.softcap = float(softcap) if softcap is not None else None
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self) -> List[WeightSpec]:
        return [] if self.tied_to is not None else [WeightSpec(self.name, (self.vocab_size, self.hidden_size), "table")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        if self.tied_to is None:
            self.weight = tensors[self.name].to(rt.dtype).contiguous()
        self.rt = rt
        self.tiled = None

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        # the table in the decode product's layout (made here and not at bind: a tied table is bound by its owner)
        if self.tiled is None and rt.dtype == torch.bfloat16 and rt.tiled_weights:
            self.tiled = ops.TiledWeight(self.tied_to.table if self.tied_to is not None else self.weight)
        # logits are float32: every product of the head goes through the re-laid copy, whatever the number of rows,
        # so a head of its own lets the checkpoint's layout go (a tied head's table stays: the embedding reads it)
        if self.tiled is not None and self.tied_to is None and self.hidden_size % 8 == 0:
            self.weight = None

    def forward(self, y: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        w = self.tied_to.table if self.tied_to is not None else self.weight
        if self.tiled is None and self.rt.dtype == torch.bfloat16 and self.rt.tiled_weights:
            self.tiled = ops.TiledWeight(w)
        logits = ctx.ws.get("logits", (y.shape[0], self.vocab_size), torch.float32)
        ops.linear(y, w, logits, self.scale, w_tiled=self.tiled)
        if self.softcap is not None:
            ops.softcap(logits, self.softcap)
        return logits
