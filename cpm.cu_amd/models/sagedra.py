"""Sagedra: which parts, with which numbers.

A decoder of pre-norm layers (layer norm with a weight and no bias) whose residual may be several streams
(hyper-connections: every sub-layer reads a weighted sum of the streams and its result joins all of them through a
mixing matrix).  A layer's mixer is differential attention (two causal softmax maps a head over the same values,
biased projections, a short convolution on q, k and v, a query temperature that grows with the position) or a pair
side by side: grouped-query attention over a sliding window (rotation with stretched slow frequencies, q and k
divided by their root mean square after it, a sigmoid gate on the heads) beside a gated delta rule, whose two
results are RMS-normed over the width and averaged.  The feed-forward, which a layer may lack, is gated with the
tanh form of GELU.  A span of layers may run several times in a row with the same weights; every run has a cache
entry of its own.  The embedding is multiplied by a number from the configuration; the logits may pass a tanh cap.

Checkpoint tensors: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1|norm2``, with streams
``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mlp.gate|up|down`` and ``l<i>.mix.*``: attention q, k, v, o (+ ``.b``),
q|k|v.conv, lq1, lk1, lq2, lk2; parallel left.q|k|v|g|o, right.q|k|v (+ ``.conv``), right.a|b|g|o|A_log|dt_bias|norm,
left.out, right.out.
"""
from __future__ import annotations

from ..config.sagedra import ARCHITECTURE, SagedraConfig
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, TokenEmbedding
from ..registry import Architecture, register_architecture
from .decoder import DecoderModel, Run

_FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _window_attention(cfg: SagedraConfig, m, p: str):
    position = None
    if m.rot_dims:
        if m.rot_scaling is not None:
            factor, low, high, original = m.rot_scaling
            position = POSITION_ENCODINGS.build("llama3", head_dim=m.rot_dims, theta=m.rot_base, factor=factor, low=low,
                                                high=high, original=original)
        else:
            position = POSITION_ENCODINGS.build("rope", head_dim=m.rot_dims, theta=m.rot_base)
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "gate": p + "g", "out": p + "o"}
    return MIXERS.build("attention", names=names, hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads,
                        key_dim=m.dim, value_dim=m.vdim, position=position, scale=m.scale, mask_window=m.window,
                        norm_eps=cfg.eps, unit_norm_after_rotation=True)


def _gated_delta(cfg: SagedraConfig, m, p: str):
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "gate": p + "g", "decay": p + "a", "beta": p + "b",
             "q_conv": p + "q.conv", "k_conv": p + "k.conv", "v_conv": p + "v.conv", "A_log": p + "A_log",
             "dt_bias": p + "dt_bias", "norm": p + "norm", "out": p + "o"}
    return MIXERS.build("gated_delta", names=names, hidden_size=cfg.width, heads=m.heads, kv_heads=m.kv_heads,
                        key_dim=m.dim, value_dim=m.vdim, conv_taps=m.conv, eps=cfg.eps)


def _mixer(cfg: SagedraConfig, i: int):
    layer, p = cfg.layers[i], f"l{i}.mix."
    m = layer.mixer
    if layer.type == "parallel":
        return MIXERS.build("parallel", left=_window_attention(cfg, m.left, p + "left."),
                            right=_gated_delta(cfg, m.right, p + "right."), left_norm_name=p + "left.out",
                            right_norm_name=p + "right.out", hidden_size=cfg.width, eps=cfg.eps)
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "out": p + "o", "q_bias": p + "q.b", "k_bias": p + "k.b",
             "v_bias": p + "v.b", "out_bias": p + "o.b", "lq1": p + "lq1", "lk1": p + "lk1", "lq2": p + "lq2",
             "lk2": p + "lk2"}
    if m.conv:
        names.update({"q_conv": p + "q.conv", "k_conv": p + "k.conv", "v_conv": p + "v.conv"})
    return MIXERS.build("differential_attention", names=names, hidden_size=cfg.width, num_heads=m.heads,
                        num_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim, scale=m.scale, diff=m.diff,
                        norm_eps=cfg.eps, conv_taps=m.conv, temp_coef=m.temp_coef, temp_every=m.temp_every)


def build(cfg: SagedraConfig) -> DecoderModel:
    norm = lambda name: NORMS.build("layer_norm", name=name, hidden_size=cfg.width, eps=cfg.eps)
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        ff = {}
        if layer.ff is not None:
            ff = dict(ff_norm=norm(p + "norm2"),
                      feed_forward=FEED_FORWARDS.build("gated", prefix=p + "mlp.", hidden_size=cfg.width,
                                                       intermediate_size=layer.ff, names=_FF_NAMES,
                                                       activation="gelu_tanh"))
        if cfg.streams is not None:
            hc = [tuple(f"{p}hc{q}.{t}" for t in ("in", "out", "mix")) for q in ((1, 2) if layer.ff is not None else (1,))]
            layers.append(BLOCKS.build("hyper_connections", mixer_norm=norm(p + "norm1"), mixer=_mixer(cfg, i),
                                       streams=cfg.streams, names=hc, **ff))
        else:
            layers.append(BLOCKS.build("pre_norm", mixer_norm=norm(p + "norm1"), mixer=_mixer(cfg, i), **ff))
    # every run of a layer, also a repeated one, has a cache entry of its own
    schedule = [Run(layer, entry, True) for entry, layer in enumerate(cfg.layer_runs())]
    embedding = TokenEmbedding("embed", cfg.vocab, cfg.width, cfg.embedding_scale)
    head = LMHead("head", cfg.vocab, cfg.width, 1.0, softcap=cfg.logit_softcap)
    return DecoderModel(cfg, embedding, layers, norm("final.norm"), head, schedule, streams=cfg.streams)


def _ignore(cfg: SagedraConfig, name: str) -> bool:
    """A layer without a feed-forward has no second norm and no second set of stream numbers: a checkpoint that
    stores them all the same is read without them."""
    for i, layer in enumerate(cfg.layers):
        if layer.ff is None and (name == f"l{i}.norm2" or name.startswith(f"l{i}.hc2.")):
            return True
    return False


register_architecture(Architecture(name=ARCHITECTURE, config_class=SagedraConfig, build=build, ignore_tensor=_ignore))
