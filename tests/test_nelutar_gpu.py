"""The Nelutar engine against the plain implementation (GPU): whole prompts, prefill against token-by-token decoding,
portions of several sizes down to two tokens, unequal batches against each request alone, slots and pages that are
used again, long decoding in which every window passes over decoded tokens, the first tokens of a sequence, the
residual stream after every layer run, and greedy generation through the package's own entry point, scheduler, replay
program and command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_nelutar as plain
import schedules
import tiny
import tiny_nelutar as tn

pytestmark = pytest.mark.gpu

# P: windows of 20 and 70, pages of 64, convolutions of 2 and 4 taps.  Lengths cross several windows and pages;
# requests of one and two tokens are shorter than every convolution and have no bigram beyond the first.
LENS = {"a": 13, "b": 171, "c": 85, "d": 41, "e": 1, "f": 2}
PROMPT = {"a": 5, "b": 130, "c": 64, "d": 39, "e": 1, "f": 1}
BATCHES = [("a", "b", "c"), ("d", "e", "f"), ("c", "a"), ("f", "b", "d")]
CONFIGS = (("P", tn.tiny_p, 271), ("Q", tn.tiny_q, 283), ("R", tn.tiny_r, 297))
NAMES = [c[0] for c in CONFIGS]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, raw, seed in CONFIGS:
        raw = raw()
        d = str(tmp_path_factory.mktemp(f"nelutar_{name}"))
        tn.write_model(raw, d, seed)
        cfg, w = tiny.read_model(d)
        reqs = {r: tiny.random_tokens(n, raw["vocab"], 2700 + i) for i, (r, n) in enumerate(LENS.items())}
        refs = {}
        for r, t in reqs.items():
            refs[r] = Reference(cfg, w, t)
        out[name] = (d, cfg, w, reqs, refs)
    return out


def deviation(got, ref):
    """A position's deviation as the bfloat16 checks measure it: root mean square of the logits' difference (its mean
    taken off) against the spread of the request's logits."""
    d = got - ref
    return (d - d.mean(1, keepdim=True)).pow(2).mean(1).sqrt() / ref.std()


class Reference:
    """The plain implementation's logits of a request, and which of its positions chose their experts by a margin
    that bfloat16's rounding of the router's input can overturn.  With ``conditioning`` also how far every position's
    logits move, in float64, when every matrix is disturbed by relative noise of bfloat16's size (2^-9): what a model
    with random weights and extreme constants (a head that keeps nothing of the past in front of a norm that divides
    by the head's own size, keys of 8 features) does to rounding at some positions whoever computes it."""

    def __init__(self, cfg, w, tokens, conditioning=False):
        margins = []
        self.logits = plain.forward(cfg, w, tokens, margins=margins).float()
        self.close = torch.zeros(len(tokens), dtype=torch.bool)
        for m in margins:
            self.close |= m < CLOSE_CALL
        self.moved = torch.zeros(len(tokens))
        if conditioning:
            g = torch.Generator().manual_seed(1)
            noisy = {k: v.double() * (1 + torch.randn(v.shape, generator=g, dtype=torch.float64) * 2.0 ** -9) if v.dim() == 2 else v
                     for k, v in w.items()}
            self.moved = deviation(plain.forward(cfg, noisy, tokens).float(), self.logits)

    def rows(self, rows):
        out = Reference.__new__(Reference)
        out.logits, out.close, out.moved = self.logits[rows], self.close[rows], self.moved[rows]
        return out


CLOSE_CALL = 0.02       # choice scores are sigmoids: bfloat16 rows move a logit by a few thousandths


_engines = {}


def engine_for(models, name, dtype, **kw):
    from cpmcu_amd import Engine, EngineOptions
    key = (name, dtype, tuple(sorted(kw.items())))
    if key not in _engines:
        opts = dict(dtype=dtype, max_tokens=1024, max_slots=3, max_seq_len=512)
        opts.update(kw)
        _engines[key] = Engine.from_dir(models[name][0], EngineOptions(**opts))
    return _engines[key]


def check(got, refs, dtype, what):
    """float32 (the sharp comparison): rounding of float sums, at every position.  bfloat16: the deviation of a
    position's logits (mean taken off) against the logits' spread: 0.08 at most and 0.04 in the median.  A position
    whose choice of experts was a close call in the plain implementation (Reference.close) may have gone to other
    experts in bfloat16 and is not held to a bound, and at most one position in fifty (or one) behind such a
    position, which reads its keys, values and state, is held to 0.5 only; where the reference knows how far noise of
    bfloat16's size moves a position in float64 (Reference.moved), the bound grows by six times that; the float32
    engine is held to every position."""
    for r, ref in refs.items():
        if isinstance(ref, Reference):
            ref, close, moved = ref.logits, ref.close, ref.moved
        else:
            close, moved = torch.zeros(ref.shape[0], dtype=torch.bool), torch.zeros(ref.shape[0])
        if dtype == "float32":
            err = (got[r] - ref).abs().max(dim=1).values
            bad = (err > 2e-4 * max(1.0, float(ref.abs().max()))).nonzero().flatten()
            assert bad.numel() == 0, (f"{what}: request {r}: first wrong position {int(bad[0])} of {ref.shape[0]} "
                                      f"(error {float(err[bad[0]]):.3g})")
            continue
        err = deviation(got[r], ref)
        over = ((err > 0.08 + 6.0 * moved) & ~close).nonzero().flatten()
        allowed = max(1, ref.shape[0] // 50) if (bool(close.any()) and over.numel() and int(over[0]) > int(close.nonzero()[0])) else 0
        clear = (err - 6.0 * moved)[~close]
        assert over.numel() <= allowed and (clear.numel() == 0 or float(clear.max()) <= 0.5) and float(err.median()) <= 0.04 + float(moved.median()), \
            (f"{what}: request {r}: {over.numel()} of {ref.shape[0]} positions over 0.08 whose choice of experts was "
             f"clear (first {int(over[0]) if over.numel() else -1}, worst {float(err.max()):.3g}, median "
             f"{float(err.median()):.3g}; close calls at {close.nonzero().flatten().tolist()[:12]})")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(models, name, dtype):
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, dtype)
    check(schedules.whole(eng, reqs), refs, dtype, "whole")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_prefill_then_token_by_token(models, name, dtype):
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, dtype)
    check(schedules.tail(eng, reqs, 45), refs, dtype, "tail-45")       # 45 tokens: a window of 20 passes over decoded tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_and_slots_used_again(models, name, dtype):
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, dtype)
    for part in (BATCHES[:2], BATCHES[2:]):
        used = {r for b in part for r in b}
        got = schedules.batched(eng, {r: reqs[r] for r in used}, PROMPT, part)
        check(got, {r: refs[r] for r in used}, dtype, "batched")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.parametrize("step", [2, 7, 33, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_portions(models, name, dtype, step):
    """Forward passes of at most `step` tokens: a prompt is cut into portions (two tokens are fewer than the taps of
    most convolutions), and a batch's sequences are split across passes; the previous token of the bigram table,
    recurrent state, convolution inputs and windows go on where the last portion ended."""
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, dtype, max_step_tokens=step)
    some = {r: reqs[r] for r in ("b", "d", "f")}
    check(schedules.whole(eng, some), {r: refs[r] for r in some}, dtype, f"portions of {step}")
    got = schedules.batched(eng, {r: reqs[r] for r in ("c", "a", "d")}, PROMPT, [("c", "a", "d")])
    check(got, {r: refs[r] for r in ("c", "a", "d")}, dtype, f"batch in portions of {step}")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_long_decoding_from_the_first_token(models, name, dtype):
    """One token, then 170 more one by one (captured graphs): every window slides past decoded tokens and over two
    page edges, windowed cache groups give pages back, and the recurrent states, the convolutions' inputs and the
    previous token are carried all the way, separately in every run of a layer whose weights are used twice."""
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, dtype, hip_graph=True)
    got = schedules.tail(eng, {"b": reqs["b"]}, len(reqs["b"]) - 1)
    check(got, {"b": refs["b"]}, dtype, "decoding from the first token")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_does_not_depend_on_its_neighbours_or_its_pages(models, dtype):
    from cpmcu_amd import StepEntry
    _, cfg, w, reqs, refs = models["P"]
    eng = engine_for(models, "P", dtype)
    alone = schedules.whole(eng, {"c": reqs["c"]})["c"]
    s = [eng.acquire() for _ in range(3)]
    lg = eng.step([StepEntry(s[0], reqs["b"], []), StepEntry(s[1], reqs["c"], list(range(LENS["c"]))),
                   StepEntry(s[2], reqs["a"], [0])]).cpu()
    for x in (s[1], s[0], s[2]):
        eng.release(x)
    again = schedules.whole(eng, {"c": reqs["c"]})["c"]
    assert torch.equal(again, alone)
    if dtype == "float32":
        assert float((lg[:LENS["c"]] - alone).abs().max()) <= 5e-5
    else:
        check({"c": lg[:LENS["c"]]}, {"c": alone}, dtype, "in a batch against alone")


def test_a_freed_slot_starts_from_nothing(models):
    """float32: a slot that held a long request is given to a short one: the previous token, the recurrent states and
    the convolutions' inputs of every layer run start at zero again, so the logits equal those of a fresh engine to
    the bit."""
    _, cfg, w, reqs, refs = models["P"]
    eng = engine_for(models, "P", "float32", max_slots=1)
    first = schedules.tail(eng, {"d": reqs["d"]}, 10)["d"]
    schedules.tail(eng, {"b": reqs["b"]}, 3)
    assert torch.equal(schedules.tail(eng, {"d": reqs["d"]}, 10)["d"], first)
    check({"d": first}, {"d": refs["d"]}, "float32", "one slot")


@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer_run(models, name):
    """float32: the residual after every layer run (a layer whose weights are used twice counts each time) equals the
    plain implementation's.  A layer leaves its result pending, so the stream is put together here from what the
    block left."""
    from cpmcu_amd import StepEntry
    from cpmcu_amd.parts.base import branch_tensor
    _, cfg, w, reqs, refs = models[name]
    eng = engine_for(models, name, "float32")
    _, res = plain.forward(cfg, w, reqs["d"], return_layers=True)
    seen = []
    blocks = eng.model.layers
    originals = [b.forward for b in blocks]

    def spy(i):
        def f(stream, ctx, cache, writes_cache=True):
            originals[i](stream, ctx, cache, writes_cache)
            y = branch_tensor(stream.take_pending()).double()
            seen.append((stream.x.double() + (y.sum(0) if y.dim() == 3 else y)).cpu())
        return f
    try:
        for i, b in enumerate(blocks):
            b.forward = spy(i)
        s = eng.acquire()
        eng.step([StepEntry(s, reqs["d"], [0])])
        eng.release(s)
    finally:
        for b, o in zip(blocks, originals):
            b.forward = o
    assert len(seen) == len(res) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, res)):
        err = float((a - b).abs().max())
        assert err < 2e-5 * max(1.0, float(b.abs().max())), f"residual after layer run {i}: {err:.3g}"


def test_borrowed_weights_are_held_once(models):
    """A layer that uses another's weights adds a cache entry, not tensors: the model has as many blocks as layers
    with weights of their own, and every run of the schedule its own entry."""
    eng = engine_for(models, "P", "float32")
    assert len(eng.model.layers) == 3 and [r.layer for r in eng.model.schedule] == [0, 1, 2, 0, 2]
    assert [r.cache for r in eng.model.schedule] == [0, 1, 2, 3, 4] and eng.model.embedding_entry == 5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_borrowing_layer_with_constants_of_its_own(dtype, tmp_path):
    """A layer that uses another's tensors but differs from it (a window of 9 instead of 20, other decays): it is
    built as a layer of its own on the owner's tensors."""
    from cpmcu_amd import Engine, EngineOptions
    raw = tn.tiny_p()
    raw["layers"][3]["mixer"]["left"]["mask"]["size"] = 9
    raw["layers"][4]["mixer"]["right"]["decay"] = [0.5, 0.9]
    raw["layers"][4]["mixer"]["left_scale"] = 0.2
    d = str(tmp_path / "m")
    tn.write_model(raw, d, 311, router_gain=5.0)
    cfg, w = tiny.read_model(d)
    reqs = {"a": tiny.random_tokens(90, raw["vocab"], 3200), "b": tiny.random_tokens(7, raw["vocab"], 3201)}
    refs = {r: Reference(cfg, w, t) for r, t in reqs.items()}
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512, max_slots=2, max_seq_len=256))
    assert len(eng.model.layers) == 5
    check(schedules.tail(eng, reqs, 30), refs, dtype, "borrowed tensors, own constants")


def _greedy(cfg, w, prompt, n):
    toks = list(prompt)
    out = []
    for _ in range(n):
        nxt = int(plain.forward(cfg, w, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


def test_greedy_generation_through_the_entry_point(models):
    from cpmcu_amd.llm import LLM
    d, cfg, w, reqs, refs = models["Q"]
    prompt = reqs["a"][:9]
    want = _greedy(cfg, w, prompt, 20)
    llm = LLM(d, dtype="float32", max_tokens=256)
    llm.init_storage()
    llm.load_from_hf()
    tokens, _, _ = llm.generate(torch.tensor(prompt, dtype=torch.int32), 20)
    assert tokens == want


def test_generation_loop_with_unequal_requests(models):
    """The scheduler's own loop: several prompts of unequal length in batches, greedy, against the plain
    implementation's tokens (float32); three slots, so slots and pages are used again.  The loop feeds sampled tokens
    from the device: the bigram table's previous token is the one the device chose."""
    from cpmcu_amd.engine.generate import generate
    d, cfg, w, reqs, refs = models["P"]
    eng = engine_for(models, "P", "float32")
    prompts = [reqs["a"][:7], reqs["c"][:50], reqs["d"][:3], reqs["b"][:90]]
    out = generate(eng, prompts, 12)
    for p, o in zip(prompts, out):
        assert list(o.tokens) == _greedy(cfg, w, p, 12)
    eng.cache.check()
    assert not eng.cache.live


def test_replay_program_with_a_tight_token_budget(models, tmp_path):
    """bin/trace_run as a user runs it (float32): an unequal batch, then decoding together with early leavers, with
    --max-tokens the bare sum of the requests' tokens; then a request that takes freed slots and pages."""
    import numpy as np
    d, cfg, w, reqs, refs = models["P"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    names = ["b", "c", "a", "f"]
    prompt = {"b": 160, "c": 66, "a": 2, "f": 1}
    steps = [{"step": 0, "entries": [{"id": r, "tokens": reqs[r][:prompt[r]], "want": [0, prompt[r] - 1]} for r in names],
              "end": []}]
    fed = dict(prompt)
    n = 1
    while any(fed[r] < LENS[r] for r in names):
        live = [r for r in names if fed[r] < LENS[r]]
        steps.append({"step": n, "entries": [{"id": r, "tokens": [reqs[r][fed[r]]], "want": [0]} for r in live],
                      "end": [r for r in live if fed[r] + 1 == LENS[r]]})
        for r in live:
            fed[r] += 1
        n += 1
    steps.append({"step": n, "entries": [{"id": "again", "tokens": reqs["d"], "want": [LENS["d"] - 1]}], "end": ["again"]})
    out = tmp_path / "out"
    budget = sum(LENS[r] for r in names)
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", str(budget)],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    V = cfg["vocab"]
    at = dict(prompt)
    for s in steps[:-1]:
        rows = []
        for e in s["entries"]:
            base = 0 if s["step"] == 0 else at[e["id"]]
            rows += [refs[e["id"]].logits[base + wpos] for wpos in e["want"]]
        if s["step"] > 0:
            for e in s["entries"]:
                at[e["id"]] += 1
        got = torch.from_numpy(np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(rows), V))
        assert float((got - torch.stack(rows)).abs().max()) < 2e-4, f"step {s['step']}"
    got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(1, V))
    assert float((got[0] - refs["d"].logits[-1]).abs().max()) < 2e-4


def test_command_line(models, tmp_path):
    """The command line on a Nelutar folder (greedy tokens equal the plain implementation's, the timers name the new
    kernel classes), and in random-weights mode from a config.json alone."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def run_cli(*args):
        env = dict(os.environ, PYTHONPATH=root)
        return subprocess.run([sys.executable, "-m", "cpmcu_amd.cli", *args], capture_output=True, text=True,
                              timeout=600, env=env)
    d, cfg, w, reqs, refs = models["P"]
    prompts = [reqs["a"][:6], reqs["c"][:45]]
    ids = tmp_path / "ids.txt"
    ids.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    p = run_cli("--model-path", d, "--dtype", "float32", "--prompt-ids", str(ids), "--num-generate", "6",
                "--ignore-eos", "true", "--max-tokens", "512", "--use_stream", "false", "--perf")
    assert p.returncode == 0, p.stderr[-1500:]
    assert "prefill_delta_scan" in p.stdout and "decode_linattn_scan" in p.stdout and "decode_layer_scale" in p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert [[int(t) for t in l.split(") ")[1].split()] for l in lines] == [_greedy(cfg, w, pr, 6) for pr in prompts]
    cfgp = tmp_path / "config.json"
    cfgp.write_text(json.dumps(tn.tiny_q()))
    out = tmp_path / "model"
    p = run_cli("--random-weights", "--config", str(cfgp), "--seed", "3", "--model-path", str(out), "--prompt-lens", "70,5",
                "--num-generate", "3", "--max-tokens", "512")
    assert p.returncode == 0, p.stderr[-1500:]
    assert sorted(os.listdir(out)) == ["config.json", "model.safetensors"]
    assert len([l for l in p.stdout.splitlines() if l.startswith("[")]) == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "R"])
def test_a_long_sequence(models, name, dtype):
    """1,300 tokens (21 pages): the prompt in passes of 512 tokens, then 40 tokens one by one.  The windowed layers
    have long since given their early pages back; the recurrent states (a head that never forgets among them) have
    been carried throughout."""
    from cpmcu_amd import StepEntry
    _, cfg, w, reqs, refs = models[name]
    toks = tiny.random_tokens(1300, cfg["vocab"], 2900)
    ref = Reference(cfg, w, toks)
    eng = engine_for(models, name, dtype, max_tokens=2048, max_seq_len=1408, max_step_tokens=512)
    s = eng.acquire()
    want = list(range(0, 1260, 97)) + [1259]
    got = [eng.step([StepEntry(s, toks[:1260], want)]).cpu()]
    for i in range(1260, 1300):
        got.append(eng.step([StepEntry(s, toks[i:i + 1], [0])]).cpu())
    held = [g.held(s) for g in eng.cache.groups if g.needs.window is not None]
    assert held and max(held) <= 4
    eng.release(s)
    rows = want + list(range(1260, 1300))
    check({"long": torch.cat(got)}, {"long": ref.rows(rows)}, dtype, "a long sequence")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_of_a_real_models_kind(dtype, tmp_path):
    """Width 1,024 and heads of 128: a prompt of 330 tokens (the library's products, attention and experts on the
    matrix cores, a window of 256 that has passed the first tokens), then 24 tokens one by one through captured
    graphs (strip and skinny products), and a batch of three unequal requests."""
    from cpmcu_amd import Engine, EngineOptions
    raw = tn.medium_m()
    d = str(tmp_path / "m")
    tn.write_model(raw, d, 301, std=0.03)
    cfg, w = tiny.read_model(d)
    reqs = {"a": tiny.random_tokens(354, raw["vocab"], 3100), "b": tiny.random_tokens(70, raw["vocab"], 3101),
            "c": tiny.random_tokens(9, raw["vocab"], 3102)}
    refs = {r: Reference(cfg, w, t, conditioning=(dtype == "bfloat16")) for r, t in reqs.items()}
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=1024, max_slots=3, max_seq_len=512, hip_graph=True))
    check(schedules.tail(eng, {"a": reqs["a"]}, 24), {"a": refs["a"]}, dtype, "prompt of 330, then 24 tokens")
    got = schedules.batched(eng, reqs, {"a": 300, "b": 66, "c": 2}, [("c", "a", "b")])
    check(got, refs, dtype, "batch of three")
    eng.cache.check()
    assert not eng.cache.live
