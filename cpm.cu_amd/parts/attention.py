"""Attention mixers: dense causal GQA attention, and InfLLM-v2 block-sparse
attention on top of it.

Dense (src/model/attn.cuh:58-284): q, k, v from one stacked product, position
encoding on q and k, k and v into the cache (the cache holds encoded keys),
attention of every query over its sequence's cached keys up to itself, output
projection.  scores = (q.k) * head_dim^-1/2; query head h reads kv head
h // (heads / kv_heads).

InfLLM-v2 (src/model/minicpm4/minicpm4_attn.cuh:107-202): past ``dense_len``
tokens a query attends only to chosen blocks of keys: blocks scored through
compressed keys (means of kernel_size keys every kernel_stride), the top-k of
them, plus initial blocks and a trailing window.  The reference selects per
call; here the selection of the query at position p uses only what lies before
p, so it does not depend on how the tokens were cut into steps:
compressed key j is visible iff kernel_stride*j + kernel_size <= p.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StateSpec, StreamSpec
from .base import MIXERS, BiasedBranch, DeferredBranch, Mixer, Part, PositionEncoding, Runtime, StepContext
from .linear import Linear


@MIXERS.register("gqa_attention")
class GQAAttention(Mixer):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim <= 0 or head_dim % 16 or head_dim > 256:
            # the cache lays keys and values out in pieces of 16 features (the matrix cores' operands), and the
            # plain attention kernel holds a head in 256 features; said here so that no engine is built that
            # would fail at its first step
            raise ValueError(f"attention: head_dim {head_dim} is not supported: the cache and attention kernels take "
                             f"head sizes in steps of 16 up to 256")
        self.hidden_size = hidden_size
        self.nh, self.nkv, self.hd = num_heads, num_kv_heads, head_dim
        if position is not None and position.pairs != "halves":
            raise ValueError(f"gqa_attention: the fused rotation pairs feature i with i + head_dim/2; an encoding of "
                             f"'{position.pairs}' pairs belongs to the mixer kind 'attention'")
        self.position = position
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.qkv = Linear([(prefix + "q_proj.weight", num_heads * head_dim),
                           (prefix + "k_proj.weight", num_kv_heads * head_dim),
                           (prefix + "v_proj.weight", num_kv_heads * head_dim)], hidden_size)
        self.o = Linear([(prefix + "o_proj.weight", hidden_size)], num_heads * head_dim)

    def parts(self) -> List[Part]:
        return [self.qkv, self.o] + ([self.position] if self.position is not None else [])

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        self._qkv_fused = None               # the q/k/v weight re-laid for the fused decode kernel, made at first use

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        # the q/k/v weight in the fused decode kernel's order, if any step of this engine can run that kernel
        plain_rotation = self._kernel_rotates()
        if (self._qkv_fused is None and plain_rotation and rt.dtype == torch.bfloat16 and self.qkv.tiled is not None
                and self.hd % 16 == 0 and self.hidden_size % 8 == 0 and rt.page_size % 32 == 0):
            self._qkv_fused = ops.qkv_rope_weight(self.qkv.weight, self.nh, self.nkv, self.hd)
        # split-KV shares of steps of few tokens: their number grows with the context
        if rt.dtype == torch.bfloat16:
            most = max((n * ops.attention_splits(n, self.nkv, self.nh // self.nkv, rt.max_seq_len)
                        for n in range(1, min(max_step_tokens, ops.compute_units()) + 1)), default=0)
            if most > 1:
                ws.get("attn.part_o", (most, self.nh, self.hd), torch.float32)
                ws.get("attn.part_ml", (most, self.nh, 2), torch.float32)

    def cache_needs(self) -> CacheNeeds:
        w = self.nkv * self.hd
        return CacheNeeds(streams=(("k", StreamSpec(w)), ("v", StreamSpec(w))))

    def _kernel_rotates(self) -> bool:
        """Whether the projection kernels do all that the position encoding asks of q and k: a rotate-half
        rotation, or nothing (no encoding, or one that only biases the scores)."""
        return (self.position is None or self.position.rotary_params() is not None
                or not self.position.rewrites_vectors())

    # -- steps of forward, so that a subclass can put its own between them --
    def _fused_projection(self, n: int, dtype, cache: Optional[CacheView], writes_cache: bool) -> bool:
        """Decode steps: projection, rotation and cache write in one kernel (one kernel of the chain less)."""
        plain_rotation = self._kernel_rotates()
        return (writes_cache and cache is not None and plain_rotation and n <= ops.QKV_ROPE_MAX_ROWS
                and dtype == torch.bfloat16 and self.qkv.tiled is not None and self.hd % 16 == 0
                and self.hidden_size % 8 == 0 and cache.page_size % 32 == 0)

    def takes_row_scale(self, n: int, ctx: StepContext, cache, writes_cache: bool) -> bool:
        return self._fused_projection(n, self.rt.dtype, cache, writes_cache)

    def project_and_store(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool, row_scale=None,
                          compress=None) -> torch.Tensor:
        """q [n, heads * head_dim], position-encoded; k and v go into the cache.  ``compress`` (a pool of
        compressed keys, kernel_size, kernel_stride) is only given where _fused_projection() holds: that kernel
        then also writes the compressed keys that the step's tokens complete."""
        n = h.shape[0]
        nh, nkv, hd = self.nh, self.nkv, self.hd
        plain_rotation = self._kernel_rotates()
        if self._fused_projection(n, h.dtype, cache, writes_cache):
            if self._qkv_fused is None:           # a part used outside an engine (reserve_workspace makes it)
                self._qkv_fused = ops.qkv_rope_weight(self.qkv.weight, nh, nkv, hd)
            rot = self.position.rotary_params() if self.position is not None else None
            inv_freq, mag = (rot if rot is not None else (None, 1.0))
            q = ctx.ws.get("attn.q", (n, nh * hd), self.rt.dtype)
            ops.qkv_rope(h, self._qkv_fused, q, nh, nkv, hd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                         cache.streams["k"], cache.streams["v"], cache.page_table, cache.page_size,
                         row_scale=row_scale, compress=compress)
            return q
        if row_scale is not None or compress is not None:
            raise ValueError("attention: a row scale or compressed keys need the fused projection (takes_row_scale)")
        qkv = self.qkv.forward(h, ctx, "attn.qkv", rows=None if writes_cache else nh * hd, partials=plain_rotation)
        rot = self.position.rotary_params() if self.position is not None else None
        inv_freq, mag = (rot if rot is not None else (None, 1.0))
        if self.position is not None and rot is None and self.position.rewrites_vectors():
            q3 = qkv[:, :nh * hd].unflatten(1, (nh, hd))
            k3 = qkv[:, nh * hd:(nh + nkv) * hd].unflatten(1, (nkv, hd)) if writes_cache else None
            self.position.apply(q3, k3, ctx)
        q = ctx.ws.get("attn.q", (n, nh * hd), self.rt.dtype)
        ops.rope_store(qkv, q, nh, nkv, hd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                       cache.streams["k"] if writes_cache else None, cache.streams["v"] if writes_cache else None,
                       cache.page_table if writes_cache else None, cache.page_size, writes_cache)
        return q

    can_defer_last = True

    def attend_and_project(self, q, ctx: StepContext, cache: CacheView, sel=None, defer_last: bool = False):
        """Attention of q over the cache (all keys up to each query, or the blocks listed in ``sel``), then the
        output projection."""
        sel_blocks, sel_count, bs, window_blocks = sel if sel is not None else (None, None, 0, 0)
        out = ctx.ws.get("attn.out", tuple(q.shape), q.dtype)
        slopes = self.position.score_bias() if self.position is not None else None
        with ctx.timed("attn_core"):
            ops.attention(q, out, self.nh, self.nkv, self.hd, self.scale, cache.streams["k"], cache.streams["v"],
                          cache.page_table, cache.page_size, ctx, sel_blocks, sel_count, bs, window_blocks,
                          head_slopes=slopes)
        if defer_last and self.o.defers(out):
            return DeferredBranch(self.o, out, ctx, "attn.o")
        with ctx.timed("attn_o"):
            return self.o.forward(out, ctx, "attn.o", out_dtype=torch.float32, partials=True)

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True, row_scale=None,
                defer_last: bool = False):
        with ctx.timed("attn_qkv_rope"):
            q = self.project_and_store(h, ctx, cache, writes_cache, row_scale)
        return self.attend_and_project(q, ctx, cache, defer_last=defer_last)


@MIXERS.register("infllm_v2_attention")
class InfLLMv2Attention(GQAAttention):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], kernel_size: int, kernel_stride: int, block_size: int,
                 init_blocks: int, topk: int, window_size: int, dense_len: int, scale: Optional[float] = None):
        super().__init__(prefix, hidden_size, num_heads, num_kv_heads, head_dim, position, scale)
        if block_size % kernel_stride or kernel_size < kernel_stride:
            raise ValueError("infllm_v2: block_size must be a multiple of kernel_stride <= kernel_size")
        if window_size % block_size or window_size < block_size:
            raise ValueError("infllm_v2: window_size must be a positive multiple of block_size")
        self.ks, self.st, self.bs = kernel_size, kernel_stride, block_size
        self.init_blocks, self.topk, self.dense_len = init_blocks, topk, dense_len
        self.window_blocks = window_size // block_size

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        super().bind(tensors, rt)
        if rt.page_size % self.st:
            raise ValueError(f"infllm_v2: kernel_stride {self.st} must divide the cache page of {rt.page_size} tokens "
                             f"(a compressed key's row lies in the page of its first key)")

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        super().reserve_workspace(ws, rt, max_step_tokens, max_slots)
        # the selection's scores grow with the context: sized here for the longest sequence, for steps of few
        # tokens (many small workgroups through scratch) and of many
        few = max(256 // self.nkv, 1)
        need = max(ops.sparse_select_scratch(rt.dtype, n, self.nh, self.nkv, self.hd, rt.max_seq_len - 1, self.ks,
                                             self.st, self.bs)
                   for n in {1, min(few, max_step_tokens), min(few + 1, max_step_tokens), max_step_tokens})
        if need:
            ws.get("attn.sel_scores", (need,), torch.float32)
        # the block lists of the largest step (a rehearsal pass at short positions never selects)
        ws.get("attn.sel_blocks", (max_step_tokens, self.nkv, self.topk + self.window_blocks), torch.int32)
        ws.get("attn.sel_count", (max_step_tokens, self.nkv), torch.int32)

    def cache_needs(self) -> CacheNeeds:
        w = self.nkv * self.hd
        return CacheNeeds(streams=(("k", StreamSpec(w)), ("v", StreamSpec(w)), ("ck", StreamSpec(w, every=self.st))))

    can_defer_last = True

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True, row_scale=None,
                defer_last: bool = False):
        # decode steps: the projection kernel completes the compressed keys itself (one kernel of the chain less)
        fused = self._fused_projection(h.shape[0], h.dtype, cache, writes_cache)
        with ctx.timed("attn_qkv_rope"):
            q = self.project_and_store(h, ctx, cache, writes_cache, row_scale,
                                       compress=(cache.streams["ck"], self.ks, self.st) if fused else None)
        if writes_cache and not fused:
            with ctx.timed("attn_compress"):
                ops.compress_keys(cache.streams["k"], cache.streams["ck"], self.nkv, cache.page_table,
                                  cache.page_size, ctx.positions, ctx.tok_slot, self.ks, self.st)
        sel = None
        if ctx.max_pos + 1 > self.dense_len:
            n = q.shape[0]
            max_sel = self.topk + self.window_blocks
            sel_blocks = ctx.ws.get("attn.sel_blocks", (n, self.nkv, max_sel), torch.int32)
            sel_count = ctx.ws.get("attn.sel_count", (n, self.nkv), torch.int32)
            need = ops.sparse_select_scratch(q.dtype, n, self.nh, self.nkv, self.hd, ctx.max_pos, self.ks, self.st, self.bs)
            scratch = ctx.ws.get("attn.sel_scores", (need,), torch.float32) if need else None
            # the reference times its two selection stages apart (minicpm4_attn.cuh:107-202); here they are one call
            with ctx.timed("attn_select"):
                ops.sparse_select(q, cache.streams["ck"], self.nh, self.nkv, self.hd, self.scale, cache.page_table,
                                  cache.page_size, ctx.positions, ctx.tok_slot, self.ks, self.st, self.bs,
                                  self.init_blocks, self.topk, self.window_blocks, self.dense_len, ctx.max_pos,
                                  sel_blocks, sel_count, scratch=scratch)
            sel = (sel_blocks, sel_count, self.bs, self.window_blocks)
        return self.attend_and_project(q, ctx, cache, sel, defer_last=defer_last)


def _pad16(n: int) -> int:
    return -(-n // 16) * 16


@MIXERS.register("attention")
class GeneralAttention(Mixer):
    """Grouped-query attention whose sizes are free: key size and value size of their own, a rotation that may
    cover only the first features of a head (the rest pass unchanged), a score scale from the configuration,
    and an optional mask beyond the causal one: *chunked* (the query at position p sees key j <= p only if
    j // chunk == p // chunk, chunks counted from position 0 of the sequence, not from where a prompt was cut), or
    a *sliding window with kept first tokens* (key j <= p is seen if p - j < mask_window or j < mask_keep_first;
    kept tokens keep their own positions).  Query head h reads kv head h // (heads / kv_heads); softmax in float.
    With a mask the cache keeps a trailing window (and the kept first tokens' pages) and gives older pages back.

    ``names``: checkpoint tensors for 'q', 'k', 'v', 'out', and optionally
      'q_bias', 'k_bias', 'v_bias', 'out_bias'  biases of the projections (added in float by the kernel that reads
                                                 the product);
      'q_norm', 'k_norm'   weights of dk numbers, shared by the heads: q and k heads are divided by their root mean
                           square (``norm_eps`` inside the root) and multiplied by them before the rotation;
      'sink'               one number a head: exp(sink) joins the softmax's denominator as a term that has no key,
                           no value and no scale;
      'gate'               an output gate: the heads side by side are multiplied element by element with
                           sigmoid(W_gate h) before the output projection (its rows ride in the q/k/v product).
      'q_conv', 'k_conv', 'v_conv'   with ``conv_taps`` > 0: a short causal convolution over time on every channel of
                           q, k and v ([channels, taps], the last tap the current token's, zeros before the start,
                           no bias, no activation) directly behind the projection; the last taps - 1 projected rows
                           of a sequence are fixed-size state of its cache slot.
    ``unit_norm_after_rotation``: q and k heads are divided by their root mean square (``norm_eps`` inside the
    root, no weight) after the rotation.
    The rotation pairs the features that ``position.pairs`` says ('halves': i with i + r/2 of the r rotated features;
    'interleaved': 2i with 2i + 1).
    ``score_softcap`` c: a scaled score s enters the softmax as c tanh(s / c).
    Without 'v' the values are the keys as projected (with their bias, before norm and rotation): value_dim
    must equal key_dim."""

    def __init__(self, names: Mapping[str, str], hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, position: Optional[PositionEncoding], scale: float, mask_chunk: Optional[int] = None,
                 mask_window: Optional[int] = None, mask_keep_first: int = 0, norm_eps: float = 0.0,
                 unit_norm_after_rotation: bool = False, score_softcap: Optional[float] = None, conv_taps: int = 0):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if unit_norm_after_rotation and (names.get("q_norm") or names.get("k_norm")):
            raise ValueError("attention: a norm after the rotation has no weights")
        if key_dim > 1024 or value_dim > 1024:
            raise ValueError(f"attention: key size {key_dim} / value size {value_dim} exceed the kernel's 1024")
        if mask_chunk is not None and mask_chunk <= 0:
            raise ValueError(f"attention: a mask chunk of {mask_chunk} tokens")
        if mask_window is not None and mask_window <= 0:
            raise ValueError(f"attention: a mask window of {mask_window} tokens")
        if mask_chunk and mask_window:
            raise ValueError("attention: a chunked mask or a sliding window, not both")
        if mask_keep_first < 0 or (mask_keep_first and not mask_window):
            raise ValueError("attention: kept first tokens come with a sliding window")
        if score_softcap is not None and not score_softcap > 0:
            raise ValueError(f"attention: a score cap of {score_softcap}")
        if conv_taps < 0:
            raise ValueError(f"attention: {conv_taps} convolution taps")
        self.interleaved = position is not None and position.pairs == "interleaved"
        self.softcap = float(score_softcap) if score_softcap is not None else 0.0
        self.taps = int(conv_taps)
        self.names = dict(names)
        self.values_are_keys = "v" not in self.names
        if self.taps and (self.values_are_keys or self.names.get("gate")):
            raise ValueError("attention: the convolution goes with q, k and v of their own and no output gate")
        if self.values_are_keys and value_dim != key_dim:
            raise ValueError(f"attention: values that are the keys have the keys' size ({value_dim}, {key_dim})")
        self.hidden_size, self.nh, self.nkv, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, key_dim, value_dim
        self.position, self.scale, self.chunk = position, float(scale), int(mask_chunk or 0)
        self.window, self.keep_first, self.norm_eps = int(mask_window or 0), int(mask_keep_first), float(norm_eps)
        stacked = [(self.names["q"], num_heads * key_dim), (self.names["k"], num_kv_heads * key_dim)]
        biases = [self.names.get("q_bias"), self.names.get("k_bias")]
        if not self.values_are_keys:
            stacked.append((self.names["v"], num_kv_heads * value_dim))
            biases.append(self.names.get("v_bias"))
        self.norm_after = bool(unit_norm_after_rotation)
        self.gate_off = None
        if self.names.get("gate"):
            self.gate_off = sum(r for _, r in stacked)
            stacked.append((self.names["gate"], num_heads * value_dim))
            biases.append(None)
        self.qkv = Linear(stacked, hidden_size, bias_names=biases if any(biases) else None)
        self.o = Linear([(self.names["out"], hidden_size)], num_heads * value_dim,
                        bias_names=[self.names["out_bias"]] if self.names.get("out_bias") else None)
        # what the plain rotate-and-store kernel does not do
        self._extras = bool(any(biases) or self.names.get("q_norm") or self.names.get("k_norm") or self.values_are_keys
                            or self.norm_after or self.taps)
        self.conv_widths = (num_heads * key_dim, num_kv_heads * key_dim, num_kv_heads * value_dim)

    def parts(self) -> List[Part]:
        return [self.qkv, self.o] + ([self.position] if self.position is not None else [])

    def weight_specs(self):
        from .base import WeightSpec
        specs = [WeightSpec(self.names[k], (self.dk,), "norm") for k in ("q_norm", "k_norm") if self.names.get(k)]
        if self.names.get("sink"):
            specs.append(WeightSpec(self.names["sink"], (self.nh,), "small"))
        if self.taps:
            specs += [WeightSpec(self.names[k], (w, self.taps), "conv_taps")
                      for k, w in zip(("q_conv", "k_conv", "v_conv"), self.conv_widths)]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        f = lambda k: tensors[self.names[k]].to(torch.float32).contiguous() if self.names.get(k) else None
        self.q_norm, self.k_norm, self.sink = f("q_norm"), f("k_norm"), f("sink")
        if self.taps:
            self.conv_w = torch.cat([f("q_conv"), f("k_conv"), f("v_conv")], 0).contiguous()

    def cache_needs(self) -> CacheNeeds:
        state = ()
        if self.taps > 1:
            state = (("conv", StateSpec((self.taps - 1, sum(self.conv_widths)), torch.float32)),)
        return CacheNeeds(streams=(("k", StreamSpec(self.nkv * _pad16(self.dk))),
                                   ("v", StreamSpec(self.nkv * _pad16(self.dv)))), state=state,
                          window=self.chunk or self.window or None, keep_first=self.keep_first)

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        keys = rt.max_seq_len
        if self.chunk:
            keys = min(keys, self.chunk)
        if self.window:
            keys = min(keys, self.window + self.keep_first)
        ops.reserve_attention_general(ws, rt.dtype, self.nh, self.nkv, self.dv, _pad16(self.dv), keys, max_step_tokens)

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True):
        n, nh, nkv, dk, dv = h.shape[0], self.nh, self.nkv, self.dk, self.dv
        rot = self.position.rotary_params() if self.position is not None else None
        if self.position is not None and rot is None:
            raise ValueError("attention: the position encoding must be a rotation (rotary_params)")
        inv_freq, mag = rot if rot is not None else (None, 1.0)
        rd = 0 if inv_freq is None else 2 * inv_freq.shape[0]
        if rd > dk:
            raise ValueError(f"attention: the rotation covers {rd} features, a head has {dk}")
        if self.taps and not writes_cache:
            raise ValueError("attention: a run that reads another run's cache has no convolution state of its own")
        with ctx.timed("attn_qkv_rope"):
            qkv = self.qkv.forward(h, ctx, "attn.qkv", rows=None if (writes_cache or self.gate_off is not None) else nh * dk)
            if self.taps:
                # the projected rows mixed over time, in float; the slot's state moves on to the step's last rows
                mixed = ctx.ws.get("attn.conv", (n, sum(self.conv_widths)), torch.float32)
                ops.conv_silu(qkv, self.conv_w, None, cache.state.get("conv"), mixed, ctx.cu_q, ctx.seq_slot,
                              max(ctx.q_lens), update_state=True, activation=False)
                qkv = mixed
            q = ctx.ws.get("attn.q", (n, nh * dk), self.rt.dtype)
            if self._extras:
                ops.qkv_norm_rotate_store(qkv, q, nh, nkv, dk, dv, rd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                                          cache.streams["k"], cache.streams["v"], cache.page_table, cache.page_size,
                                          write_kv=writes_cache, bias=self.qkv.bias, q_norm=self.q_norm,
                                          k_norm=self.k_norm, eps=self.norm_eps, values_from_keys=self.values_are_keys,
                                          norm_after=self.norm_after, interleaved=self.interleaved)
            else:
                ops.qkv_rotate_store(qkv, q, nh, nkv, dk, dv, rd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                                     cache.streams["k"], cache.streams["v"], cache.page_table, cache.page_size,
                                     write_kv=writes_cache, interleaved=self.interleaved)
        out = ctx.ws.get("attn.out", (n, nh * dv), self.rt.dtype)
        gate = qkv[:, self.gate_off:self.gate_off + nh * dv] if self.gate_off is not None else None
        with ctx.timed("attn_core"):
            # the matrix-core kernel (and the merge of split keys) applies the gate as it writes
            gated_there = ops.attention_any(q, out, nh, nkv, dk, dv, self.scale, cache.streams["k"], cache.streams["v"],
                                            cache.page_table, cache.page_size, ctx, chunk=self.chunk, window=self.window,
                                            keep_first=self.keep_first, sink=self.sink, gate=gate, softcap=self.softcap)
        if gate is not None and not gated_there:
            with ctx.timed("attn_gate"):
                gated = ctx.ws.get("attn.gated", (n, nh * dv), self.rt.dtype)
                ops.sigmoid_gate(out, gate, gated)
                out = gated
        with ctx.timed("attn_o"):
            branch = self.o.forward(out, ctx, "attn.o", out_dtype=torch.float32, partials=True)
        return BiasedBranch(branch, self.o.bias, ctx, "attn.o") if self.o.bias is not None else branch
