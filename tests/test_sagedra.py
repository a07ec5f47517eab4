"""Sagedra without a GPU: configuration, defaults, refusals, tensor names, the order of layer runs and what each run
asks of the cache; the plain implementation pinned by closed forms and invariants, one mechanism at a time."""
import copy
import math

import pytest
import torch

import plain_sagedra as plain
import tiny_sagedra as ts

F64 = torch.float64


def _cfg(raw):
    import cpmcu_amd
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    return arch, arch.config_class.from_dict(raw)


# ---------------------------------------------------------------------------
# configuration and model
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("raw", [ts.tiny_u(), ts.tiny_v(), ts.tiny_w()])
def test_configuration_reads_back(raw):
    arch, cfg = _cfg(raw)
    assert arch.config_class.from_dict(cfg.to_dict()) == cfg
    assert cfg.vocabulary_size == raw["vocab"] and len(cfg.layers) == len(raw["layers"])
    assert list(cfg.layer_runs()) == plain.layer_order(raw)


def test_defaults_of_absent_keys():
    _, cfg = _cfg(ts.tiny_v())
    assert cfg.streams is None and cfg.loop is None and cfg.logit_softcap is None and cfg.embedding_scale == 1.0
    a = cfg.layers[0].mixer
    assert a.conv == 0 and a.temp_every == 0 and a.kv_heads == 5
    left = cfg.layers[1].mixer.left
    assert left.rot_dims == 0 and left.window is None and left.rot_scaling is None
    assert cfg.layers[2].mixer.left.rot_scaling is None and cfg.layers[2].mixer.left.rot_dims == 6
    assert cfg.layers[3].ff is None
    raw = ts.tiny_u()
    del raw["layers"][1]["mixer"]["kv_heads"], raw["layers"][1]["mixer"]["vdim"]
    m = _cfg(raw)[1].layers[1].mixer
    assert m.kv_heads == m.heads == 2 and m.vdim == m.dim == 16


@pytest.mark.parametrize("change, word", [
    (lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=26), "rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"]["scaling"].update(high=1.0), "high"),
    (lambda r: r["layers"][0]["mixer"]["right"].update(conv=0), "conv"),
    (lambda r: r["layers"][0]["mixer"].pop("right"), "right"),
    (lambda r: r["layers"][1]["mixer"]["q_temp"].update(every=0), "every"),
    (lambda r: r["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda r: r["layers"][1].update(type="mamba2"), "type"),
    (lambda r: r["layers"][1]["mlp"].update(kind="experts"), "kind"),
    (lambda r: r["loop"].update(stop=5), "loop"),
    (lambda r: r["loop"].update(times=0), "times"),
    (lambda r: r.update(streams=0), "streams"),
    (lambda r: r.update(logit_softcap=0.0), "logit_softcap"),
    (lambda r: r.pop("norm"), "norm"),
])
def test_refusals(change, word):
    from cpmcu_amd import ConfigError
    raw = ts.tiny_u()
    change(raw)
    with pytest.raises(ConfigError, match=word):
        _cfg(raw)


def test_tensor_names_and_cache_needs():
    arch, cfg = _cfg(ts.tiny_u())
    model = arch.build_model(cfg)
    specs = {s.name: tuple(s.shape) for s in model.all_weight_specs()}
    assert specs["embed"] == (210, 96) and specs["head"] == (210, 96) and specs["final.norm"] == (96,)
    assert specs["l0.hc1.in"] == (2,) and specs["l0.hc2.mix"] == (2, 2) and specs["l0.norm2"] == (96,)
    assert specs["l0.mix.left.q"] == (6 * 24, 96) and specs["l0.mix.left.v"] == (2 * 40, 96)
    assert specs["l0.mix.left.g"] == (6 * 40, 96) and specs["l0.mix.left.o"] == (96, 6 * 40)
    assert specs["l0.mix.right.q"] == (2 * 24, 96) and specs["l0.mix.right.v"] == (4 * 20, 96)
    assert specs["l0.mix.right.q.conv"] == (48, 2) and specs["l0.mix.right.v.conv"] == (80, 2)
    assert specs["l0.mix.right.a"] == (4, 96) and specs["l0.mix.right.A_log"] == (4,) and specs["l0.mix.right.norm"] == (20,)
    assert specs["l0.mix.left.out"] == (96,) and specs["l0.mix.right.out"] == (96,)
    # two score maps a head: twice the query and key rows, one set of values
    assert specs["l1.mix.q"] == (2 * 2 * 16, 96) and specs["l1.mix.k"] == (1 * 2 * 16, 96) and specs["l1.mix.v"] == (24, 96)
    assert specs["l1.mix.q.b"] == (64,) and specs["l1.mix.o.b"] == (96,) and specs["l1.mix.k.conv"] == (32, 4)
    assert specs["l1.mix.lq1"] == (16,) and specs["l1.mix.lk2"] == (16,)
    # a layer without feed-forward has neither the second norm nor the second set of stream numbers
    assert "l2.norm2" not in specs and "l2.hc2.in" not in specs and "l2.mlp.gate" not in specs and "l2.hc1.mix" in specs
    assert arch.ignore_tensor(cfg, "l2.norm2") and arch.ignore_tensor(cfg, "l2.hc2.mix")
    assert not arch.ignore_tensor(cfg, "l1.norm2") and not arch.ignore_tensor(cfg, "l2.hc1.mix")
    # a cache entry a layer run: layers 1 and 2 run three times
    needs = model.cache_needs()
    assert len(needs) == 8 == len(cfg.layer_runs())
    assert needs[0].window == 20 and needs[2].window == 70 and needs[1].window is None
    assert needs[1] == needs[3] == needs[5] and needs[2] == needs[4] == needs[6]
    state0 = dict(needs[0].state)
    assert state0["right.delta"].shape == (4, 20, 24) and state0["right.delta"].dtype == torch.float32
    assert state0["right.conv"].shape == (1, 48 + 48 + 80)                 # taps - 1 rows of q | k | v
    assert dict(needs[1].state)["conv"].shape == (3, 64 + 32 + 24)
    assert dict(needs[0].streams)["left.v"].width >= 2 * 40 and dict(needs[0].streams)["left.k"].width >= 2 * 24


def test_plain_models_without_streams_conv_or_cap():
    """A configuration with nothing optional builds and asks for no convolution state where there is no convolution."""
    arch, cfg = _cfg(ts.tiny_v())
    model = arch.build_model(cfg)
    specs = {s.name for s in model.all_weight_specs()}
    assert not any(".hc" in n for n in specs) and "l0.mix.q.conv" not in specs and "l3.mix.q.conv" in specs
    needs = model.cache_needs()
    assert dict(needs[0].state) == {} and needs[1].window is None and needs[2].window == 33
    # one tap: the convolution is a multiplication and keeps nothing
    assert set(dict(needs[1].state)) == {"right.delta"} and dict(needs[1].state)["right.delta"].shape == (2, 7, 12)


# ---------------------------------------------------------------------------
# the plain implementation
# ---------------------------------------------------------------------------
def test_norms():
    torch.manual_seed(1)
    x = torch.randn(5, 40, dtype=F64) * 3 + 2
    w = torch.rand(40, dtype=F64)
    y = plain.layer_norm(x, w, 0.0) / w
    assert torch.allclose(y.mean(-1), torch.zeros(5, dtype=F64), atol=1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=F64), atol=1e-12)
    assert torch.allclose(plain.layer_norm(x + 7.0, w, 1e-5), plain.layer_norm(x, w, 1e-5))      # the mean is taken off
    assert not torch.allclose(plain.rms(x + 7.0, 1e-5), plain.rms(x, 1e-5))
    # eps lies inside the root
    z = torch.full((1, 4), 1e-3, dtype=F64)
    assert torch.allclose(plain.rms(z, 1e-6), z / math.sqrt(2e-6))


def test_activations():
    z = torch.linspace(-6, 6, 25, dtype=F64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(plain.softplus(z * 20), torch.nn.functional.softplus(z * 20, threshold=1e9))
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z))


def test_convolution_is_causal_and_ends_at_the_current_token():
    torch.manual_seed(2)
    u, w = torch.randn(9, 3, dtype=F64), torch.randn(3, 4, dtype=F64)
    y = plain.causal_conv(u, w)
    assert torch.allclose(y[0], u[0] * w[:, 3])                             # zeros before the start
    assert torch.allclose(y[5], u[5] * w[:, 3] + u[4] * w[:, 2] + u[3] * w[:, 1] + u[2] * w[:, 0])
    u2 = u.clone()
    u2[6:] += 1.0
    assert torch.equal(plain.causal_conv(u2, w)[:6], y[:6])
    # in two parts, the second one given the first one's last taps - 1 inputs
    tail = plain.causal_conv(u[2:], w)
    assert torch.allclose(tail[3:], y[5:])


def test_stretched_frequencies():
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}}
    f0 = plain.frequencies({"base": 10000.0, "dims": 32})
    f = plain.frequencies(rot)
    assert torch.allclose(f0, 10000.0 ** (-torch.arange(16, dtype=F64) / 16))
    wave = 2 * math.pi / f0
    fast, slow = wave < 256 / 4.0, wave > 256 / 1.0
    assert fast.any() and slow.any() and (~fast & ~slow).any()
    assert torch.equal(f[fast], f0[fast]) and torch.allclose(f[slow], f0[slow] / 8.0)
    mid = ~fast & ~slow
    assert ((f[mid] > f0[mid] / 8.0) & (f[mid] < f0[mid])).all()
    # continuous at both ends of the blend
    for wl, want in ((256 / 4.0, 1.0), (256 / 1.0, 1 / 8.0)):
        t = (256 / wl - 1.0) / 3.0
        assert math.isclose((1 - t) / 8.0 + t, want)


def test_rotation_depends_on_distance_and_leaves_the_rest():
    torch.manual_seed(3)
    rot = {"base": 100.0, "dims": 8}
    q, k = torch.randn(1, 1, 12, dtype=F64), torch.randn(1, 1, 12, dtype=F64)
    dot = lambda a, b: float((plain.rotate(q, torch.tensor([a]), rot) * plain.rotate(k, torch.tensor([b]), rot)).sum())
    assert math.isclose(dot(9, 4), dot(105, 100), rel_tol=1e-9) and not math.isclose(dot(9, 4), dot(9, 5), rel_tol=1e-3)
    r = plain.rotate(q, torch.tensor([17]), rot)
    assert torch.equal(r[..., 8:], q[..., 8:]) and not torch.allclose(r[..., :8], q[..., :8])
    # feature i is paired with feature i + dims/2
    e = torch.zeros(1, 1, 12, dtype=F64)
    e[0, 0, 1] = 1.0
    r = plain.rotate(e, torch.tensor([3]), rot)
    a = 3 * 100.0 ** (-2.0 / 8)
    assert math.isclose(float(r[0, 0, 1]), math.cos(a)) and math.isclose(float(r[0, 0, 5]), math.sin(a))
    assert float(r.abs().sum()) == pytest.approx(abs(math.cos(a)) + abs(math.sin(a)))


def test_window_counts_the_query_itself():
    m = plain.visible(10, 3)
    assert m[5].nonzero().flatten().tolist() == [3, 4, 5] and m[1].nonzero().flatten().tolist() == [0, 1]
    assert plain.visible(10)[7].sum() == 8 and plain.visible(10, 1).sum() == 10


def _one_layer(kind, mixer, width=32, streams=None, seed=4):
    raw = {"architecture": "Sagedra", "vocab": 50, "width": width, "norm": {"eps": 1e-5},
           "layers": [{"type": kind, "mixer": mixer, "mlp": None}]}
    if streams:
        raw["streams"] = streams
    arch, cfg = _cfg(raw)
    g = torch.Generator().manual_seed(seed)
    W = {s.name: torch.randn(tuple(s.shape), generator=g, dtype=F64) * 0.3 for s in arch.build_model(cfg).all_weight_specs()}
    return raw, W


def test_window_attention_loses_a_key_that_leaves_the_window():
    mixer = {"left": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.5, "mask": {"size": 4}},
             "right": {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "conv": 2}}
    raw, W = _one_layer("parallel", mixer)
    torch.manual_seed(5)
    h = torch.randn(9, 32, dtype=F64)
    base = plain.window_attention(h, W, "l0.mix.left.", mixer["left"], 1e-5)
    h2 = h.clone()
    h2[2] += 1.0
    moved = plain.window_attention(h2, W, "l0.mix.left.", mixer["left"], 1e-5)
    changed = ((moved - base).abs().max(-1).values > 1e-12).nonzero().flatten().tolist()
    assert changed == [2, 3, 4, 5]                                          # positions 2..5 see token 2; 6 does not


def test_delta_rule_writes_and_reads_back():
    """With orthonormal keys, beta 1 and no decay the state stores each value under its key; writing a key again
    replaces its value; a decay of zero empties the state before the write."""
    d, dv = 6, 3
    torch.manual_seed(6)
    keys = torch.linalg.qr(torch.randn(d, d, dtype=F64))[0]
    k = torch.stack([keys[0], keys[1], keys[2], keys[0], keys[3]])
    v = torch.randn(5, dv, dtype=F64)
    q = torch.stack([keys[0], keys[0], keys[1], keys[0], keys[2]])
    one = torch.ones(5, dtype=F64)
    o = plain.delta_rule(q, k, v, one, one)
    assert torch.allclose(o[0], v[0]) and torch.allclose(o[1], v[0]) and torch.allclose(o[2], v[1])
    assert torch.allclose(o[3], v[3])                                       # the read-out sees the current write
    assert torch.allclose(o[4], v[2])
    g = one.clone()
    g[4] = 0.0
    assert torch.allclose(plain.delta_rule(q, k, v, one, g)[4], torch.zeros(dv, dtype=F64))
    half = plain.delta_rule(q, k, v, one * 0.5, one)
    assert torch.allclose(half[1], 0.5 * v[0]) and torch.allclose(half[3], 0.5 * (0.5 * v[0]) + 0.5 * v[3])


def test_delta_rule_state_carries_across_a_cut():
    torch.manual_seed(7)
    T, d, dv = 12, 5, 4
    q, k, v = torch.randn(T, d, dtype=F64), torch.randn(T, d, dtype=F64) * 0.4, torch.randn(T, dv, dtype=F64)
    beta, g = torch.rand(T, dtype=F64), torch.rand(T, dtype=F64)
    whole = plain.delta_rule(q, k, v, beta, g)
    S = torch.zeros(d, dv, dtype=F64)
    for t in range(T):                                                      # the same steps written out once more
        S = g[t] * S
        S = S + torch.outer(k[t], beta[t] * (v[t] - S.T @ k[t]))
        assert torch.allclose(S.T @ q[t], whole[t])


def test_two_maps_combine():
    mixer = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.4, "diff": 0.3, "q_temp": {"coef": 0.5, "every": 2}}
    raw, W = _one_layer("attention", mixer)
    torch.manual_seed(8)
    h = torch.randn(7, 32, dtype=F64)
    p = "l0.mix."
    out = plain.differential_attention(h, W, p, mixer, 1e-5)
    # by hand for the last position of head 1
    T, H, d, dv = 7, 2, 8, 6
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, 2, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, 1, 2, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, 1, dv)
    temp = 1.0 + 0.5 * math.log(math.floor((6 + 1) / 2) + 1.0)
    a = []
    for n in (0, 1):
        s = (k[:, 0, n] @ (q[6, 1, n] * temp)) * 0.4
        a.append(torch.softmax(s, 0) @ v[:, 0])
    lam = math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + 0.3
    o = a[0] - lam * a[1]
    o = o / torch.sqrt((o * o).mean() + 1e-5) * 0.7
    heads = (out - W[p + "o.b"]) @ torch.linalg.pinv(W[p + "o"].T)
    assert torch.allclose(heads[6, dv:], o, atol=1e-9)
    # the temperature is 1 while floor((p + 1) / every) is 0
    assert math.floor((0 + 1) / 2) == 0


def test_streams_reduce_to_the_plain_residual():
    """One stream read with 1, written with 1 and mixed with 1 is the ordinary residual sum; with several streams
    the new rows come from the old ones all at once, and mix is indexed [from, to]."""
    raw = ts.tiny_w()
    arch, cfg = _cfg(raw)
    g = torch.Generator().manual_seed(9)
    W = {s.name: torch.randn(tuple(s.shape), generator=g) * 0.2 for s in arch.build_model(cfg).all_weight_specs()}
    for n in W:
        if ".hc" in n:
            W[n] = torch.ones_like(W[n])
    toks = [3, 9, 27, 81, 2, 6]
    with_streams = plain.forward(raw, W, toks)
    raw2 = copy.deepcopy(raw)
    del raw2["streams"]
    assert torch.allclose(with_streams, plain.forward(raw2, W, toks), atol=1e-10)
    # [from, to]: stream 0 feeds stream 1 and nothing else does
    X = torch.stack([torch.full((1, 4), 1.0, dtype=F64), torch.full((1, 4), 10.0, dtype=F64)])
    mix = torch.tensor([[0.0, 1.0], [0.0, 0.0]], dtype=F64)
    new = torch.einsum("st,snd->tnd", mix, X)
    assert float(new[1, 0, 0]) == 1.0 and float(new[0, 0, 0]) == 0.0


def test_loop_runs_the_span_in_place():
    raw = ts.tiny_u()
    assert plain.layer_order(raw) == [0, 1, 2, 1, 2, 1, 2, 3]
    raw["loop"] = {"start": 0, "stop": 4, "times": 2}
    assert plain.layer_order(raw) == [0, 1, 2, 3, 0, 1, 2, 3]
    raw["loop"] = {"start": 2, "stop": 2, "times": 5}
    assert plain.layer_order(raw) == [0, 1, 2, 3] == list(_cfg(raw)[1].layer_runs())
    del raw["loop"]
    assert plain.layer_order(raw) == [0, 1, 2, 3]


def test_logit_cap_bounds_the_logits():
    raw = ts.tiny_w()
    arch, cfg = _cfg(raw)
    g = torch.Generator().manual_seed(10)
    W = {s.name: torch.randn(tuple(s.shape), generator=g) * 0.5 for s in arch.build_model(cfg).all_weight_specs()}
    capped = plain.forward(raw, W, [1, 2, 3, 4])
    raw2 = copy.deepcopy(raw)
    del raw2["logit_softcap"]
    free = plain.forward(raw2, W, [1, 2, 3, 4])
    assert float(capped.abs().max()) < 5.0 and torch.allclose(capped, 5.0 * torch.tanh(free / 5.0))
    assert float(free.abs().max()) > 5.0
