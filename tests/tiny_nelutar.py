"""Tiny Nelutar configurations for the tests.  They differ from each other in every size, in the order of the layers
and in what they have at all: a bigram table with many buckets, with one bucket, or none; layers that use another
layer's weights (once, twice, never); windows shorter than, equal to and longer than a cache page, of one token, or
no window; rotations of a whole head, part of it or nothing; grouped, single and ungrouped key heads; convolutions of
one to five taps or none; a score cap or none; decays of 0 and 1; routers with and without groups (groups of one
expert, all experts chosen, one expert chosen), with and without a shared expert; layers without a feed-forward."""
import json
import os


def tiny_p():
    """Five layer runs over three sets of weights: the pair with the delta rule (window 20, 8 of 24 features rotate,
    3 query heads a key head; delta rule of 4 heads on 2 key heads, 2 taps) with routed experts in 3 groups of 4;
    retention; the pair with linear attention (window 70, longer than a page; 4 taps; a cap of 5) without a
    feed-forward; then the first and the third once more with their own caches."""
    return {
        "architecture": "Nelutar", "vocab": 211, "width": 96, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 97, "mul_prev": 13, "mul_cur": 5}},
        "layers": [
            {"type": "parallel", "mixer": {
                "left": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.3,
                         "rot": {"base": 5000.0, "dims": 8}, "mask": {"size": 20}},
                "right": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 20, "conv": 2}},
             "mlp": {"kind": "moe", "expert": {"ff": 40, "limit": 1.2},
                     "router": {"experts": 12, "top": 2, "scale": 1.7, "groups": {"count": 3, "keep": 2}},
                     "shared": {"ff": 56, "limit": 2.5}}},
            {"type": "retention", "mixer": {"heads": 3, "dim": 16, "vdim": 24, "decay": [0.9, 0.97, 0.6],
                                            "rot": {"base": 300.0, "dims": 16}},
             "mlp": {"kind": "dense", "ff": 120}},
            {"type": "parallel_2", "mixer": {
                "left": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.5, "conv": 4, "softcap": 5.0,
                         "rot": {"base": 100.0, "dims": 32}, "mask": {"size": 70}},
                "right": {"heads": 2, "dim": 16, "vdim": 32, "decay": [0.8, 0.99]},
                "left_scale": 0.7, "right_scale": 1.3},
             "mlp": None},
            {"type": "parallel", "weights_of": 0, "mixer": {
                "left": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.3,
                         "rot": {"base": 5000.0, "dims": 8}, "mask": {"size": 20}},
                "right": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 20, "conv": 2}},
             "mlp": {"kind": "moe", "expert": {"ff": 40, "limit": 1.2},
                     "router": {"experts": 12, "top": 2, "scale": 1.7, "groups": {"count": 3, "keep": 2}},
                     "shared": {"ff": 56, "limit": 2.5}}},
            {"type": "parallel_2", "weights_of": 2, "mixer": {
                "left": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.5, "conv": 4, "softcap": 5.0,
                         "rot": {"base": 100.0, "dims": 32}, "mask": {"size": 70}},
                "right": {"heads": 2, "dim": 16, "vdim": 32, "decay": [0.8, 0.99]},
                "left_scale": 0.7, "right_scale": 1.3},
             "mlp": None},
        ],
    }


def tiny_q():
    """Sizes that suit no vector access and no matrix-core tile, and nothing optional: no bigram table, no borrowed
    weights, a width of 100, a vocabulary of 77.  Retention that rotates nothing, with experts that are all chosen
    (no groups, no shared expert); the pair with linear attention whose attention has no convolution, no cap, no
    rotation and no window, beside one head of 12 by 7 that never forgets (decay 1); the pair with the delta rule
    (window 33, 6 of 20 features rotate, one tap) whose router has groups of one expert and chooses one."""
    return {
        "architecture": "Nelutar", "vocab": 77, "width": 100, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "retention", "mixer": {"heads": 5, "dim": 20, "vdim": 12, "decay": [0.5, 0.75, 0.9, 0.99, 0.999]},
             "mlp": {"kind": "moe", "expert": {"ff": 28, "limit": 0.8}, "router": {"experts": 5, "top": 5, "scale": 1.0}}},
            {"type": "parallel_2", "mixer": {
                "left": {"heads": 3, "kv_heads": 1, "dim": 24, "vdim": 24, "scale": 0.7},
                "right": {"heads": 1, "dim": 12, "vdim": 7, "decay": [1.0]},
                "left_scale": 1.0, "right_scale": 1.0},
             "mlp": {"kind": "dense", "ff": 44}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 5, "kv_heads": 5, "dim": 20, "vdim": 28, "scale": 0.4,
                         "rot": {"base": 1000.0, "dims": 6}, "mask": {"size": 33}},
                "right": {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 36, "conv": 1}},
             "mlp": {"kind": "moe", "expert": {"ff": 36, "limit": 3.0},
                     "router": {"experts": 8, "top": 1, "scale": 0.5, "groups": {"count": 8, "keep": 1}},
                     "shared": {"ff": 20, "limit": 0.6}}},
        ],
    }


def tiny_r():
    """A bigram table of one bucket (every later token reads row 0, the first token row 1); a window of one token (a
    query sees itself only) with one tap, a hard cap of 0.5 and one rotated pair, beside heads whose decay is 0 (the
    current token alone), a half, 1 and nearly 1; the pair with the delta rule whose window is exactly a page, one key
    head for four heads and 5 taps, 64 experts in 4 groups, twice with the same weights; retention that rotates half
    of a head and has no feed-forward."""
    return {
        "architecture": "Nelutar", "vocab": 130, "width": 64, "norm": {"eps": 1e-5},
        "embedding": {"bigram": {"buckets": 1, "mul_prev": 0, "mul_cur": 1}},
        "layers": [
            {"type": "parallel_2", "mixer": {
                "left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 1.5, "conv": 1, "softcap": 0.5,
                         "rot": {"base": 50.0, "dims": 2}, "mask": {"size": 1}},
                "right": {"heads": 4, "dim": 32, "vdim": 40, "decay": [0.0, 0.5, 1.0, 0.999]},
                "left_scale": 2.0, "right_scale": 0.25},
             "mlp": {"kind": "dense", "ff": 80}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.5,
                         "rot": {"base": 100.0, "dims": 16}, "mask": {"size": 64}},
                "right": {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 40, "conv": 5}},
             "mlp": {"kind": "moe", "expert": {"ff": 16, "limit": 1.0},
                     "router": {"experts": 64, "top": 6, "scale": 2.0, "groups": {"count": 4, "keep": 2}},
                     "shared": {"ff": 24, "limit": 1.0}}},
            {"type": "parallel", "weights_of": 1, "mixer": {
                "left": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.5,
                         "rot": {"base": 100.0, "dims": 16}, "mask": {"size": 64}},
                "right": {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 40, "conv": 5}},
             "mlp": {"kind": "moe", "expert": {"ff": 16, "limit": 1.0},
                     "router": {"experts": 64, "top": 6, "scale": 2.0, "groups": {"count": 4, "keep": 2}},
                     "shared": {"ff": 24, "limit": 1.0}}},
            {"type": "retention", "mixer": {"heads": 2, "dim": 16, "vdim": 16, "decay": [0.95, 0.7],
                                            "rot": {"base": 20.0, "dims": 8}},
             "mlp": None},
        ],
    }


def medium_m():
    """Sizes of a real model's kind, so that the kernels for aligned sizes run (matrix-core attention with heads of
    128, strip and skinny products, the library's product, experts on the matrix cores, 16 state values a lane): width
    1,024, heads of 128 by 128, windows of 256, 8 experts of 512 with a shared one, ranks of 64 (by the writer's
    rule)."""
    left = {"heads": 8, "kv_heads": 2, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "mask": {"size": 256}}
    moe = {"kind": "moe", "expert": {"ff": 512, "limit": 4.0},
           "router": {"experts": 8, "top": 2, "scale": 2.0, "groups": {"count": 4, "keep": 2}}, "shared": {"ff": 512, "limit": 4.0}}
    decays = [0.9, 0.97, 0.99, 0.999]
    return {
        "architecture": "Nelutar", "vocab": 1000, "width": 1024, "norm": {"eps": 1e-6},
        "embedding": {"bigram": {"buckets": 4099, "mul_prev": 1009, "mul_cur": 757}},
        "layers": [
            {"type": "parallel_2", "mixer": {
                "left": dict(left, rot={"base": 10000.0, "dims": 64}, conv=4, softcap=30.0),
                "right": {"heads": 4, "dim": 128, "vdim": 128, "decay": decays}, "left_scale": 0.7, "right_scale": 0.4},
             "mlp": {"kind": "dense", "ff": 2048}},
            {"type": "parallel", "mixer": {"left": dict(left, rot={"base": 500000.0, "dims": 128}),
                                           "right": {"heads": 4, "kv_heads": 2, "dim": 128, "vdim": 128, "conv": 4}},
             "mlp": moe},
            {"type": "retention", "mixer": {"heads": 4, "dim": 128, "vdim": 128, "decay": decays,
                                            "rot": {"base": 100000.0, "dims": 128}}, "mlp": moe},
        ],
    }


def write_model(raw, out_dir, seed, std=0.08, norm_std=0.1, router_gain=1.0):
    """A model folder with random weights through the package's own writer; config.json is the raw dictionary.
    ``router_gain`` multiplies the routers' weights: with the writer's small weights the experts' scores lie close
    together and every other token's choice is a close call; a gain spreads them."""
    import cpmcu_amd
    from cpmcu_amd.weights import write_model_dir
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    cfg = arch.config_class.from_dict(raw)
    write_model_dir(cfg, out_dir, seed, std=std, norm_std=norm_std)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    if router_gain != 1.0:
        from safetensors.torch import load_file, save_file
        path = os.path.join(out_dir, "model.safetensors")
        tensors = load_file(path)
        for name in tensors:
            if name.endswith(".mlp.router"):
                tensors[name] = (tensors[name].float() * router_gain).to(tensors[name].dtype)
        save_file(tensors, path)
    return out_dir
