"""Latent attention: keys and values of all heads come from one small latent vector per token.

Per token, a down projection gives kv_rank + rot_dim numbers: the first kv_rank, RMS-normed with a weight, are
the latent c; the last rot_dim are one rotated key part shared by all heads.  Head h's key is
[W_uk[h] c | rotated part], its value W_uv[h] c; its query is [q_plain (key_dim) | q_rot (rot_dim)] and the
score (q_plain . W_uk[h] c + q_rot . k_rot) * scale.  Only c and the rotated key part are cached.

The cache is read without expanding it: q_plain . (W_uk[h] c) = (W_uk[h]^T q_plain) . c, so the query is taken
into the latent space once per token and head, attention runs with one cached "head" of kv_rank + rot_dim
key features and kv_rank value features shared by all query heads, and W_uv[h] is applied to the attention's
output instead of to every cached token.  (The cache holds c twice, in the key and in the value layout of the
matrix cores' operands.)  Causal mask, ordinary softmax in float; an output gate sigmoid(W_g x)[h] a head,
read from the mixer's input; output projection on the concatenated heads.

A layer may read the latent cache that another layer wrote (``shares_cache``): it has no down projection and
brings its own W_uk, W_uv, queries and everything else.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StreamSpec
from .base import MIXERS, Mixer, Part, PositionEncoding, Runtime, StepContext, WeightSpec
from .linear import Linear


def _pad16(n: int) -> int:
    return -(-n // 16) * 16


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    def __init__(self, names: Mapping[str, str], hidden_size: int, num_heads: int, key_dim: int, rot_dim: int,
                 value_dim: int, kv_rank: int, position: Optional[PositionEncoding], scale: float, eps: float,
                 shares_cache: bool = False):
        """``names``: checkpoint tensors for 'q', 'down' and 'down_norm' (unless shares_cache), 'up_k', 'up_v',
        'gate', 'out'.  ``position`` rotates the rot_dim part of queries and of the shared key part."""
        if rot_dim % 2:
            raise ValueError(f"latent_attention: {rot_dim} rotated features (an even number is needed)")
        if kv_rank + rot_dim > 1024:
            raise ValueError(f"latent_attention: {kv_rank} + {rot_dim} cached key features exceed the attention "
                             f"kernel's 1024")
        self.names = dict(names)
        self.hidden_size, self.nh, self.dim, self.rot, self.vdim, self.rank = (hidden_size, num_heads, key_dim, rot_dim,
                                                                              value_dim, kv_rank)
        self.position, self.scale, self.eps, self.shares_cache = position, float(scale), float(eps), bool(shares_cache)
        self.qw = key_dim + rot_dim                      # a head's query as projected
        self.dk = kv_rank + rot_dim                      # a head's query and the cached key as attended
        stacked = [(self.names["q"], num_heads * self.qw)]
        if not shares_cache:
            stacked.append((self.names["down"], kv_rank + rot_dim))
        stacked.append((self.names["gate"], num_heads))
        self.proj = Linear(stacked, hidden_size)         # everything that reads the mixer's input, one product
        self.o = Linear([(self.names["out"], hidden_size)], num_heads * value_dim)

    def parts(self) -> List[Part]:
        return [self.proj, self.o] + ([self.position] if self.position is not None else [])

    def weight_specs(self) -> List[WeightSpec]:
        specs = [WeightSpec(self.names["up_k"], (self.nh * self.dim, self.rank)),
                 WeightSpec(self.names["up_v"], (self.nh * self.vdim, self.rank))]
        if not self.shares_cache:
            specs.append(WeightSpec(self.names["down_norm"], (self.rank,), "norm"))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        # W_uk[h]^T as the weight of a product over heads: [H, kv_rank, key_dim]; W_uv[h]: [H, value_dim, kv_rank]
        uk = tensors[self.names["up_k"]].to(rt.dtype).view(self.nh, self.dim, self.rank)
        self.uk_t = uk.transpose(1, 2).contiguous()
        self.uv = tensors[self.names["up_v"]].to(rt.dtype).view(self.nh, self.vdim, self.rank).contiguous()
        if not self.shares_cache:
            self.down_norm = tensors[self.names["down_norm"]].to(torch.float32).contiguous()

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(streams=(("k", StreamSpec(_pad16(self.dk))), ("v", StreamSpec(_pad16(self.rank)))))

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        ops.reserve_attention_general(ws, rt.dtype, self.nh, 1, self.rank, _pad16(self.rank), rt.max_seq_len, max_step_tokens)

    def _rotation(self):
        rot = self.position.rotary_params() if self.position is not None else None
        if self.rot and rot is None:
            raise ValueError("latent_attention: the position encoding must be a rotation (rotary_params)")
        inv_freq, mag = rot if rot is not None else (None, 1.0)
        if self.rot and self.position.pairs != "halves":
            raise ValueError(f"latent_attention: the rotation pairs feature i with i + rot/2, not '{self.position.pairs}'")
        if self.rot and inv_freq.shape[0] * 2 != self.rot:
            raise ValueError(f"latent_attention: the rotation covers {inv_freq.shape[0] * 2} features, the rotated "
                             f"part has {self.rot}")
        return inv_freq, mag

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: CacheView, writes_cache: bool = True):
        if writes_cache == self.shares_cache:
            raise ValueError("latent_attention: a layer with a down projection writes its cache entry, a layer "
                             "without one reads another layer's")
        n, H, R = h.shape[0], self.nh, self.rank
        inv_freq, mag = self._rotation()
        with ctx.timed("attn_qkv_rope"):
            proj = self.proj.forward(h, ctx, "lat.proj")
            # the query in the latent space: [W_uk[h]^T q_plain | rotated q_rot] per head
            q = ctx.ws.get("lat.q", (n, H * self.dk), self.rt.dtype)
            ops.gemm_heads(proj, 0, self.qw, self.uk_t, q, 0, self.dk)
            # rotated query parts, the normed latent and the rotated shared key part, to their places: one launch
            ops.latent_store(proj, q, H, self.dim, self.rot, R, self.down_norm if writes_cache else None, self.eps,
                             ctx.positions, ctx.tok_slot, inv_freq, mag, cache.streams["k"], cache.streams["v"],
                             cache.page_table, cache.page_size, write_cache=writes_cache)
            off = H * self.qw + ((R + self.rot) if writes_cache else 0)
        o_lat = ctx.ws.get("lat.o_lat", (n, H * R), self.rt.dtype)
        with ctx.timed("attn_core"):
            ops.attention_any(q, o_lat, H, 1, self.dk, R, self.scale, cache.streams["k"], cache.streams["v"],
                              cache.page_table, cache.page_size, ctx)
        out = ctx.ws.get("lat.out", (n, H * self.vdim), self.rt.dtype)
        with ctx.timed("attn_up_v"):
            ops.gemm_heads(o_lat, 0, R, self.uv, out, 0, self.vdim, gate=proj[:, off:off + H])
        with ctx.timed("attn_o"):
            return self.o.forward(out, ctx, "attn.o", out_dtype=torch.float32, partials=True)
