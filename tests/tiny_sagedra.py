"""Tiny Sagedra configurations for the tests.  They differ from each other in every size, in the order of the
layers and in what they have at all: two, one or no residual streams; a looped span in the middle, at the start, of
one pass, or none; windows shorter and longer than a cache page, or no window; a rotation that covers a whole head,
part of it or nothing, with and without stretched frequencies; grouped, single and ungrouped key heads; convolutions
of two to five taps or none; a query temperature that steps every token, every few tokens or is absent; layers
without a feed-forward; a logit cap or none."""
import json
import os


def tiny_u():
    """Two streams; layers 1..2 run three times.  A pair first (window 20, 16 of 24 features rotate with stretched
    slow frequencies, 3 query heads a key head; delta rule of 4 heads on 2 key heads, 2 taps); differential
    attention with one key head, 4 taps, a temperature step of 7; a pair without a feed-forward whose window (70)
    is longer than a page and whose delta rule has one head of 72 by 8 and 5 taps; differential attention of
    ungrouped heads whose temperature steps every token."""
    return {
        "architecture": "Sagedra", "vocab": 210, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
        "streams": 2, "loop": {"start": 1, "stop": 3, "times": 3}, "logit_softcap": 12.0,
        "layers": [
            {"type": "parallel", "mixer": {
                "left": {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.6,
                         "rot": {"base": 10000.0, "dims": 16,
                                 "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}},
                         "mask": {"size": 20}},
                "right": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 20, "conv": 2}},
             "mlp": {"kind": "dense", "ff": 136}},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24, "scale": 0.3, "diff": 0.3,
                                            "conv": 4, "q_temp": {"coef": 0.5, "every": 7}},
             "mlp": {"kind": "dense", "ff": 120}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.5,
                         "rot": {"base": 500.0, "dims": 32}, "mask": {"size": 70}},
                "right": {"heads": 1, "kv_heads": 1, "dim": 72, "vdim": 8, "conv": 5}},
             "mlp": None},
            {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 40, "vdim": 16, "scale": 0.2, "diff": 0.7,
                                            "conv": 2, "q_temp": {"coef": 0.2, "every": 1}},
             "mlp": {"kind": "dense", "ff": 72}},
        ],
    }


def tiny_v():
    """Sizes that suit no vector access and no matrix-core tile, and nothing optional: one residual (no streams),
    no loop, no logit cap, an embedding scale of 1, a width of 100, a vocabulary of 77.  Differential attention
    without convolution and without temperature (heads of 20 by 12); a pair whose attention sees every earlier
    token and rotates nothing beside a delta rule of 12 by 7 with one tap; a pair with a window of 33 whose
    rotation of 6 of 20 features is not stretched; differential attention with 3 taps and no feed-forward."""
    return {
        "architecture": "Sagedra", "vocab": 77, "width": 100, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "attention", "mixer": {"heads": 5, "kv_heads": 5, "dim": 20, "vdim": 12, "scale": 0.3, "diff": 0.2},
             "mlp": {"kind": "dense", "ff": 52}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 3, "kv_heads": 1, "dim": 24, "vdim": 24, "scale": 0.7},
                "right": {"heads": 2, "kv_heads": 1, "dim": 12, "vdim": 7, "conv": 1}},
             "mlp": {"kind": "dense", "ff": 44}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 5, "kv_heads": 5, "dim": 20, "vdim": 28, "scale": 0.4,
                         "rot": {"base": 1000.0, "dims": 6}, "mask": {"size": 33}},
                "right": {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 36, "conv": 3}},
             "mlp": {"kind": "dense", "ff": 60}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.5, "diff": 0.9,
                                            "conv": 3},
             "mlp": None},
        ],
    }


def tiny_w():
    """One stream that still has its reading, writing and mixing numbers; a loop over the first layer alone, four
    times, and a span that runs once would be the same as none; a window of one token (a query sees itself only)."""
    return {
        "architecture": "Sagedra", "vocab": 130, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 7.0},
        "streams": 1, "loop": {"start": 0, "stop": 1, "times": 4}, "logit_softcap": 5.0,
        "layers": [
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 32, "scale": 0.25, "diff": 0.5,
                                            "conv": 2, "q_temp": {"coef": 1.0, "every": 3}},
             "mlp": {"kind": "dense", "ff": 80}},
            {"type": "parallel", "mixer": {
                "left": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.5,
                         "rot": {"base": 100.0, "dims": 8, "scaling": {"factor": 2.0, "low": 2.0, "high": 8.0, "original": 40}},
                         "mask": {"size": 1}},
                "right": {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 40, "conv": 4}},
             "mlp": {"kind": "dense", "ff": 96}},
        ],
    }


def write_model(raw, out_dir, seed, std=0.08, norm_std=0.1):
    """A model folder with random weights through the package's own writer; config.json is the raw dictionary."""
    import cpmcu_amd
    from cpmcu_amd.weights import write_model_dir
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    cfg = arch.config_class.from_dict(raw)
    write_model_dir(cfg, out_dir, seed, std=std, norm_std=norm_std)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    return out_dir
