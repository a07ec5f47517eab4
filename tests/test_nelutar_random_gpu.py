"""Nelutar models drawn at random (GPU): sizes, head counts, the order of the layers, windows, taps, ranks, constants
and seeds differ from draw to draw and from every tiny model of the other tests; each is stepped whole, with a
decoded tail and in an unequal batch by both engines against the plain implementation."""
import json
import os
import random

import pytest
import torch

import schedules
import tiny
from test_nelutar_gpu import Reference, check

pytestmark = pytest.mark.gpu


def _attention(rng, second):
    kv, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 4])
    dim = rng.choice([8, 16, 24, 32, 48, 64])
    m = {"heads": kv * group, "kv_heads": kv, "dim": dim, "vdim": rng.choice([8, 16, 24, 40, 64]),
         "scale": round(rng.uniform(0.05, 0.6), 3)}
    rot = rng.choice([0, 2, dim // 2 // 2 * 2, dim])
    if rot:
        m["rot"] = {"base": rng.choice([50.0, 1000.0, 500000.0]), "dims": rot}
    size = rng.choice([None, 1, 5, 17, 64, 100])
    if size:
        m["mask"] = {"size": size}
    if second:
        taps = rng.choice([0, 1, 2, 3, 4])
        if taps:
            m["conv"] = taps
        cap = rng.choice([None, 1.0, 10.0])
        if cap:
            m["softcap"] = cap
    return m


def _decays(rng, heads, none=True):
    """``none``: a decay of 0 (a head that keeps nothing of the past) may be drawn."""
    return [rng.choice([0.0 if none else 0.5, 1.0, round(rng.uniform(0.3, 0.999), 4), round(rng.uniform(0.9, 0.9999), 5)])
            for _ in range(heads)]


def _mixer(rng, kind):
    if kind == "retention":
        heads, dim = rng.choice([1, 2, 3, 5]), rng.choice([8, 16, 32, 64])
        # (no decay of 0 in front of the norm a head: the head's output would be one value row times a sign)
        m = {"heads": heads, "dim": dim, "vdim": rng.choice([8, 12, 32, 64]), "decay": _decays(rng, heads, none=False)}
        rot = rng.choice([0, 2, dim])
        if rot:
            m["rot"] = {"base": rng.choice([20.0, 10000.0]), "dims": rot}
        return m
    if kind == "parallel":
        kv, rep = rng.choice([1, 2]), rng.choice([1, 2, 3])
        return {"left": _attention(rng, False),
                "right": {"heads": kv * rep, "kv_heads": kv, "dim": rng.choice([8, 16, 32, 64]), "vdim": rng.choice([8, 20, 32, 64]),
                          "conv": rng.choice([1, 2, 3, 4])}}
    heads = rng.choice([1, 2, 4])
    return {"left": _attention(rng, True),
            "right": {"heads": heads, "dim": rng.choice([8, 16, 32]), "vdim": rng.choice([8, 24, 32]), "decay": _decays(rng, heads)},
            "left_scale": round(rng.uniform(0.2, 1.5), 2), "right_scale": round(rng.uniform(0.2, 1.5), 2)}


def _mlp(rng):
    kind = rng.choice([None, "dense", "moe", "moe"])
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": rng.choice([24, 40, 72, 128])}
    count = rng.choice([1, 2, 3, 4])
    per = rng.choice([1, 2, 3, 4])
    keep = rng.randint(1, count)
    router = {"experts": count * per, "top": rng.randint(1, keep * per), "scale": round(rng.uniform(0.5, 3.0), 2)}
    if count > 1 or rng.random() < 0.5:
        router["groups"] = {"count": count, "keep": keep}
    else:
        router["top"] = rng.randint(1, count * per)
    mlp = {"kind": "moe", "expert": {"ff": rng.choice([8, 20, 32]), "limit": round(rng.uniform(0.5, 3.0), 2)}, "router": router}
    if rng.random() < 0.6:
        mlp["shared"] = {"ff": rng.choice([8, 28, 48]), "limit": round(rng.uniform(0.5, 3.0), 2)}
    return mlp


def draw(seed):
    """(config.json dictionary, ranks of the low-rank products of every `parallel` layer with weights of its own)."""
    rng = random.Random(seed)
    raw = {"architecture": "Nelutar", "vocab": rng.randint(50, 300), "width": rng.choice([64, 72, 96, 128, 160]),
           "norm": {"eps": rng.choice([1e-5, 1e-6])}, "layers": []}
    if rng.random() < 0.7:
        raw["embedding"] = {"bigram": {"buckets": rng.choice([1, 31, 251]), "mul_prev": rng.randint(0, 40), "mul_cur": rng.randint(1, 40)}}
    ranks = {}
    for i in range(rng.randint(3, 5)):
        own = [j for j, l in enumerate(raw["layers"]) if "weights_of" not in l]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            raw["layers"].append(dict(json.loads(json.dumps(raw["layers"][j])), weights_of=j))
            continue
        kind = rng.choice(["parallel", "parallel_2", "retention"])
        raw["layers"].append({"type": kind, "mixer": _mixer(rng, kind), "mlp": _mlp(rng)})
        if kind == "parallel":
            ranks[i] = (rng.choice([3, 8, 12, 24]), rng.choice([5, 8, 16]))
    return raw, ranks


def write(raw, ranks, out_dir, seed):
    """Random weights through the package's writer, with the low-rank products redrawn at the ranks of the draw (the
    engine reads them from the checkpoint's shapes)."""
    import cpmcu_amd
    from cpmcu_amd.weights import random_tensors
    from safetensors.torch import save_file
    cfg = cpmcu_amd.get_architecture("Nelutar").config_class.from_dict(raw)
    tensors = random_tensors(cfg, seed, 0.08, 0.1)
    g = torch.Generator().manual_seed(seed)
    for i, (ra, rg) in ranks.items():
        p, W = f"l{i}.mix.right.", raw["width"]
        hk, hv = tensors[p + "a2"].shape[0], tensors[p + "g2"].shape[0]
        for name, shape in ((p + "a1", (ra, W)), (p + "a2", (hk, ra)), (p + "g1", (rg, W)), (p + "g2", (hv, rg))):
            tensors[name] = (torch.randn(shape, generator=g) * 0.15).bfloat16()
    # routers that spread their scores: with the writer's small weights every other token's choice of experts is a
    # close call, and after the first token that bfloat16 routes differently a recurrent layer compares nothing
    for name in tensors:
        if name.endswith(".mlp.router"):
            tensors[name] = (tensors[name].float() * 5.0).bfloat16()
    os.makedirs(out_dir, exist_ok=True)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16, 17, 18])
def test_a_drawn_model(seed, tmp_path):
    from cpmcu_amd import Engine, EngineOptions
    raw, ranks = draw(seed)
    d = str(tmp_path / "model")
    write(raw, ranks, d, seed)
    cfg, w = tiny.read_model(d)
    reqs = {"a": tiny.random_tokens(150, raw["vocab"], seed), "b": tiny.random_tokens(37, raw["vocab"], seed + 100),
            "c": tiny.random_tokens(2, raw["vocab"], seed + 200)}
    refs = {r: Reference(cfg, w, t, conditioning=True) for r, t in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512, max_slots=3, max_seq_len=256, hip_graph=True))
        check(schedules.whole(eng, reqs), refs, dtype, f"draw {seed} whole")
        check(schedules.tail(eng, {"a": reqs["a"]}, 110), {"a": refs["a"]}, dtype, f"draw {seed} tail")
        got = schedules.batched(eng, reqs, {"a": 70, "b": 36, "c": 1}, [("b", "a", "c")])
        check(got, refs, dtype, f"draw {seed} batched")
        eng.cache.check()
        assert not eng.cache.live
