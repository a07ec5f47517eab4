"""Nelutar: which parts, with which numbers.

A decoder of parallel layers: one RMS norm a layer, a mixer and an optional feed-forward that both read the normed
rows, and a learned vector on each of the two results before they join the residual, x += ls1 * mixer(h) + ls2 *
ff(h).  The embedding adds a row of a second table chosen by a hash of the previous and the current token.  A layer
may use another layer's tensors (``weights_of``) with a cache entry of its own.  Mixers:

* ``parallel``: grouped-query attention over a sliding window (rotation of neighbouring pairs of the first features)
  beside a gated delta rule whose decay is a number a head and key channel (low-rank decay and gate projections, a
  sigmoid gate); the two results are RMS-normed over the width and averaged.
* ``parallel_2``: the same attention with a short convolution on q, k and v before the rotation, q and k divided by
  their root mean square after it and scores capped by a tanh, beside linear attention with a fixed decay a head
  (SiLU on q, k, v; one norm over all heads; a sigmoid gate); the two results are added with a number each.
* ``retention``: linear attention with a fixed decay a head, rotated q and k (pairs half a rotation apart), k scaled
  by dim^(-1/2), a norm a head without a weight and a SiLU gate.

Feed-forwards: SiLU-gated, or a mixture of experts with a sigmoid router (a correction that enters the choice only,
groups scored by the sum of their two best, weights normalised and scaled), whose experts, and a shared one, use a
clamped swish: g <- min(g, limit), u <- clamp(u, -limit, limit), g sigmoid(1.702 g) (u + 1).

Checkpoint tensors: ``embed``, ``bigram``, ``head``, ``final.norm``, and per layer i with weights of its own
``l<i>.norm1``, ``l<i>.ls1|ls2``, ``l<i>.mlp.gate|up|down`` or ``l<i>.mlp.router|correction|e<j>.gate|up|down|
shared.gate|up|down``, and ``l<i>.mix.*``: retention q, k, v, g, o; pairs left.q|k|v|o (+ ``.conv``), left.out,
right.out (``parallel``), right.q|k|v (+ ``.conv``), right.b|A_log|dt_bias|norm|a1|a2|g1|g2|o (``parallel``),
right.q|k|v|g|o|norm (``parallel_2``).
"""
from __future__ import annotations

from ..config.nelutar import ARCHITECTURE, NelutarConfig
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, TokenEmbedding
from ..registry import Architecture, register_architecture
from .decoder import DecoderModel, Run

_FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _rotation(m, pairs):
    return POSITION_ENCODINGS.build("rope", head_dim=m.rot_dims, theta=m.rot_base, pairs=pairs) if m.rot_dims else None


def _attention(cfg: NelutarConfig, m, p: str, normed: bool):
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "out": p + "o"}
    if m.conv:
        names.update({"q_conv": p + "q.conv", "k_conv": p + "k.conv", "v_conv": p + "v.conv"})
    return MIXERS.build("attention", names=names, hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads,
                        key_dim=m.dim, value_dim=m.vdim, position=_rotation(m, "interleaved"), scale=m.scale,
                        mask_window=m.window, norm_eps=cfg.eps, unit_norm_after_rotation=normed, score_softcap=m.softcap,
                        conv_taps=m.conv)


def _channel_delta(cfg: NelutarConfig, m, p: str, ranks):
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "beta": p + "b", "q_conv": p + "q.conv", "k_conv": p + "k.conv",
             "v_conv": p + "v.conv", "A_log": p + "A_log", "dt_bias": p + "dt_bias", "norm": p + "norm", "out": p + "o",
             "decay_down": p + "a1", "decay_up": p + "a2", "gate_down": p + "g1", "gate_up": p + "g2"}
    return MIXERS.build("gated_delta", names=names, hidden_size=cfg.width, heads=m.heads, kv_heads=m.kv_heads,
                        key_dim=m.dim, value_dim=m.vdim, conv_taps=m.conv, eps=cfg.eps, gate_activation="sigmoid",
                        decay_rank=ranks[0], gate_rank=ranks[1])


def _mixer(cfg: NelutarConfig, i: int, options):
    """The mixer of layer i, reading the tensors of the layer whose weights it uses."""
    layer, w = cfg.layers[i], cfg.layer_weights()[i]
    p = f"l{w}.mix."
    m = layer.mixer
    if layer.type == "parallel":
        ranks = options.get(f"l{w}.ranks", (max(m.right.heads * m.right.dim // 8, 1), max(m.right.heads * m.right.vdim // 8, 1)))
        return MIXERS.build("parallel", left=_attention(cfg, m.left, p + "left.", normed=False),
                            right=_channel_delta(cfg, m.right, p + "right.", ranks), left_norm_name=p + "left.out",
                            right_norm_name=p + "right.out", hidden_size=cfg.width, eps=cfg.eps)
    if layer.type == "parallel_2":
        r, q = m.right, p + "right."
        right = MIXERS.build("decay_linear_attention",
                             names={"q": q + "q", "k": q + "k", "v": q + "v", "gate": q + "g", "out": q + "o", "norm": q + "norm"},
                             hidden_size=cfg.width, heads=r.heads, key_dim=r.dim, value_dim=r.vdim, decay=r.decay,
                             eps=cfg.eps, activation="silu", position=_rotation(r, "interleaved"), norm="all",
                             gate_activation="sigmoid")
        return MIXERS.build("parallel", left=_attention(cfg, m.left, p + "left.", normed=True), right=right,
                            hidden_size=cfg.width, scales=(m.left_scale, m.right_scale))
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "gate": p + "g", "out": p + "o"}
    return MIXERS.build("decay_linear_attention", names=names, hidden_size=cfg.width, heads=m.heads, key_dim=m.dim,
                        value_dim=m.vdim, decay=m.decay, eps=cfg.eps, position=_rotation(m, "halves"),
                        key_scale=m.dim ** -0.5, norm="heads", gate_activation="silu")


def _feed_forward(cfg: NelutarConfig, i: int):
    ff, p = cfg.layers[i].mlp, f"l{cfg.layer_weights()[i]}.mlp."
    if ff is None:
        return None
    if ff.kind == "dense":
        return FEED_FORWARDS.build("gated_silu", prefix=p, hidden_size=cfg.width, intermediate_size=ff.ff, names=_FF_NAMES)
    names = {"router": p + "router", "correction": p + "correction", "expert": p + "e{e}.{part}",
             "shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down"}
    return FEED_FORWARDS.build("routed_experts", names=names, hidden_size=cfg.width, expert_size=ff.ff,
                               experts=ff.experts, top=ff.top, groups=ff.groups, shared_size=ff.shared_ff,
                               score="sigmoid", group_score="top2_sum", weight_scale=ff.router_scale,
                               activation=("clamped_swish", ff.limit),
                               shared_activation=("clamped_swish", ff.shared_limit) if ff.shared_ff is not None else None)


def build(cfg: NelutarConfig, ranks=None) -> DecoderModel:
    """``ranks``: {layer: (rank of the decay's product, rank of the gate's)} of the ``parallel`` layers, read from the
    checkpoint's tensor shapes (no configuration key holds them); a random-weights model takes an eighth of the
    products' widths."""
    options = {f"l{i}.ranks": tuple(r) for i, r in (ranks or {}).items()}
    norm = lambda name: NORMS.build("rms_norm", name=name, hidden_size=cfg.width, eps=cfg.eps)
    owner = cfg.layer_weights()
    blocks, index = [], {}
    for i in range(len(cfg.layers)):
        if cfg.shares_block(i):
            continue                    # the owner's block runs once more
        p = f"l{owner[i]}."
        ff = _feed_forward(cfg, i)
        index[i] = len(blocks)
        blocks.append(BLOCKS.build("parallel_scaled", norm=norm(p + "norm1"), mixer=_mixer(cfg, i, options), feed_forward=ff,
                                   hidden_size=cfg.width, scale_names=[p + "ls1"] + ([p + "ls2"] if ff is not None else [])))
    # every layer of the configuration is a run with a cache entry of its own, whoever's weights it uses
    schedule = [Run(index[owner[i]] if cfg.shares_block(i) else index[i], entry, True) for entry, i in enumerate(range(len(cfg.layers)))]
    bigram = ("bigram",) + tuple(cfg.bigram) if cfg.bigram is not None else None
    embedding = TokenEmbedding("embed", cfg.vocab, cfg.width, 1.0, bigram=bigram)
    head = LMHead("head", cfg.vocab, cfg.width, 1.0)
    return DecoderModel(cfg, embedding, blocks, norm("final.norm"), head, schedule)


def _checkpoint_options(cfg: NelutarConfig, tensors) -> dict:
    """The ranks of the low-rank decay and gate products stand in no configuration key: the checkpoint's shapes give
    them.  ``tensors``: names (with shapes where the loader knows them)."""
    shapes = tensors if isinstance(tensors, dict) else {}
    ranks = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type != "parallel" or layer.weights_of is not None:
            continue
        a, g = shapes.get(f"l{i}.mix.right.a1"), shapes.get(f"l{i}.mix.right.g1")
        if a is not None and g is not None:
            ranks[i] = (int(a[0]), int(g[0]))
    return {"ranks": ranks} if ranks else {}


def _ignore(cfg: NelutarConfig, name: str) -> bool:
    """A layer without a feed-forward has no second scale vector: a checkpoint that stores one all the same is read
    without it."""
    for i, layer in enumerate(cfg.layers):
        if layer.mlp is None and name == f"l{i}.ls2":
            return True
    return False


register_architecture(Architecture(name=ARCHITECTURE, config_class=NelutarConfig, build=build, options={"ranks": None},
                                   checkpoint_options=_checkpoint_options, ignore_tensor=_ignore))
