"""Nelutar without a GPU: configuration, defaults, refusals, tensor names, layers that borrow weights and what each
run asks of the cache; the plain implementation pinned by closed forms and invariants, one mechanism at a time."""
import math

import pytest
import torch

import plain_nelutar as plain
import tiny_nelutar as tn

F64 = torch.float64


def _cfg(raw):
    import cpmcu_amd
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    return arch, arch.config_class.from_dict(raw)


def _rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, dtype=F64, generator=torch.Generator().manual_seed(seed)) * scale


# ---------------------------------------------------------------------------
# configuration and model
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("raw", [tn.tiny_p(), tn.tiny_q(), tn.tiny_r()])
def test_configuration_reads_back(raw):
    arch, cfg = _cfg(raw)
    assert arch.config_class.from_dict(cfg.to_dict()) == cfg
    assert cfg.vocabulary_size == raw["vocab"] and len(cfg.layers) == len(raw["layers"])
    assert list(cfg.layer_weights()) == [l.get("weights_of", i) for i, l in enumerate(raw["layers"])]


def test_defaults_of_absent_keys():
    _, cfg = _cfg(tn.tiny_q())
    assert cfg.bigram is None
    left = cfg.layers[1].mixer.left
    assert left.rot_dims == 0 and left.window is None and left.conv == 0 and left.softcap is None
    assert cfg.layers[0].mixer.rot_dims == 0
    moe = cfg.layers[0].mlp
    assert moe.groups is None and moe.shared_ff is None and moe.router_scale == 1.0
    raw = tn.tiny_p()
    del raw["layers"][0]["mixer"]["left"]["kv_heads"], raw["layers"][0]["mixer"]["left"]["vdim"]
    del raw["layers"][3]["mixer"]["left"]["kv_heads"], raw["layers"][3]["mixer"]["left"]["vdim"]
    m = _cfg(raw)[1].layers[0].mixer.left
    assert m.kv_heads == m.heads == 6 and m.vdim == m.dim == 24


@pytest.mark.parametrize("change, word", [
    (lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=26), "rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda r: r["layers"][0]["mixer"]["right"].update(conv=0), "conv"),
    (lambda r: r["layers"][0]["mixer"].pop("right"), "right"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=13), "top"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=5), "groups"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=4), "keep"),
    (lambda r: r["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda r: r["layers"][1]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda r: r["layers"][1]["mixer"].update(decay=[0.5, 0.5, 1.5]), "decays"),
    (lambda r: r["layers"][1].update(type="mamba2"), "type"),
    (lambda r: r["layers"][1]["mlp"].update(kind="experts"), "kind"),
    (lambda r: r["layers"][2]["mixer"]["left"].update(softcap=0.0), "softcap"),
    (lambda r: r["layers"][3].update(weights_of=3), "weights_of"),
    (lambda r: r["layers"][3].update(weights_of=4), "weights_of"),
    (lambda r: r["layers"][3].update(weights_of=1), "equal"),
    (lambda r: r["layers"][3].update(mlp=None), "equal"),
    (lambda r: r["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda r: r.pop("norm"), "norm"),
])
def test_refusals(change, word):
    from cpmcu_amd import ConfigError
    raw = tn.tiny_p()
    change(raw)
    with pytest.raises(ConfigError, match=word):
        _cfg(raw)


def test_a_borrowing_layer_may_leave_out_what_it_shares():
    raw = tn.tiny_p()
    full = _cfg(raw)[1]
    raw["layers"][3] = {"weights_of": 0}
    raw["layers"][4] = {"type": "parallel_2", "weights_of": 2, "mixer": raw["layers"][4]["mixer"]}
    assert _cfg(raw)[1] == full


def test_a_borrowing_layer_that_differs_is_a_layer_of_its_own_on_the_same_tensors():
    raw = tn.tiny_p()
    raw["layers"][3]["mixer"]["left"]["mask"]["size"] = 9
    arch, cfg = _cfg(raw)
    model = arch.build_model(cfg)
    assert len(model.layers) == 4 and [r.layer for r in model.schedule] == [0, 1, 2, 3, 2]
    assert {s.name for s in model.layers[3].all_weight_specs()} == {s.name for s in model.layers[0].all_weight_specs()}
    needs = model.cache_needs()
    assert needs[0].window == 20 and needs[3].window == 9


def test_the_pairing_belongs_to_the_position_encoding():
    from cpmcu_amd.parts import MIXERS, POSITION_ENCODINGS
    arch, cfg = _cfg(tn.tiny_p())
    model = arch.build_model(cfg)
    pair, retention = model.layers[0].mixer, model.layers[1].mixer
    assert pair.left.position.pairs == "interleaved" and pair.left.interleaved
    assert retention.position.pairs == "halves" and not retention.interleaved
    assert POSITION_ENCODINGS.build("rope", head_dim=8, theta=10.0).pairs == "halves"
    with pytest.raises(ValueError, match="pairs"):
        POSITION_ENCODINGS.build("rope", head_dim=8, theta=10.0, pairs="thirds")
    turned = POSITION_ENCODINGS.build("rope", head_dim=16, theta=100.0, pairs="interleaved")
    with pytest.raises(ValueError, match="interleaved"):
        MIXERS.build("gqa_attention", prefix="x.", hidden_size=64, num_heads=4, num_kv_heads=2, head_dim=16, position=turned)


def test_tensor_names_and_cache_needs():
    arch, cfg = _cfg(tn.tiny_p())
    model = arch.build_model(cfg, {"ranks": {0: (5, 7)}})
    specs = {s.name: tuple(s.shape) for s in model.all_weight_specs()}
    assert specs["embed"] == (211, 96) and specs["bigram"] == (98, 96) and specs["final.norm"] == (96,)
    assert specs["l0.ls1"] == (96,) and specs["l0.ls2"] == (96,) and "l2.ls2" not in specs and "l2.ls1" in specs
    assert specs["l0.mix.left.q"] == (6 * 24, 96) and specs["l0.mix.left.v"] == (2 * 40, 96)
    assert specs["l0.mix.right.q"] == (2 * 24, 96) and specs["l0.mix.right.v"] == (4 * 20, 96)
    assert specs["l0.mix.right.a1"] == (5, 96) and specs["l0.mix.right.a2"] == (4 * 24, 5)
    assert specs["l0.mix.right.g1"] == (7, 96) and specs["l0.mix.right.g2"] == (4 * 20, 7)
    assert specs["l0.mix.right.dt_bias"] == (4 * 24,) and specs["l0.mix.right.A_log"] == (4,)
    assert specs["l0.mix.right.norm"] == (20,) and specs["l0.mix.right.k.conv"] == (2 * 24, 2)
    assert specs["l0.mlp.router"] == (12, 96) and specs["l0.mlp.correction"] == (12,)
    assert specs["l0.mlp.e11.down"] == (96, 40) and specs["l0.mlp.shared.up"] == (56, 96)
    assert specs["l1.mix.g"] == (3 * 24, 96) and specs["l1.mix.k"] == (3 * 16, 96)
    assert specs["l2.mix.left.q.conv"] == (2 * 32, 4) and specs["l2.mix.right.norm"] == (2 * 32,)
    # layers 3 and 4 use the tensors of layers 0 and 2: none of their own, but a cache entry each
    assert not any(n.startswith(("l3.", "l4.")) for n in specs)
    needs = model.cache_needs()
    assert len(needs) == 6
    assert needs[0] == needs[3] and needs[2] == needs[4] and needs[0].window == 20 and needs[2].window == 70
    assert dict(needs[0].state)["right.delta"].shape == (4, 20, 24) and dict(needs[0].state)["right.conv"].shape == (1, 176)
    assert dict(needs[2].state)["left.conv"].shape == (3, 2 * 32 + 32 + 16) and dict(needs[2].state)["right.memory"].shape == (2, 32, 16)
    assert needs[1].streams == () and dict(needs[1].state)["memory"].shape == (3, 24, 16)
    assert dict(needs[5].state)["previous_token"].shape == () and dict(needs[5].state)["previous_token"].dtype == torch.int32


def test_ranks_come_from_the_checkpoints_shapes():
    arch, cfg = _cfg(tn.tiny_p())
    shapes = {"l0.mix.right.a1": (9, 96), "l0.mix.right.g1": (3, 96)}
    model = arch.build_model(cfg, None, shapes)
    specs = {s.name: tuple(s.shape) for s in model.all_weight_specs()}
    assert specs["l0.mix.right.a2"] == (4 * 24, 9) and specs["l0.mix.right.g2"] == (4 * 20, 3)


# ---------------------------------------------------------------------------
# the plain implementation, one mechanism at a time
# ---------------------------------------------------------------------------
def test_bigram_rows():
    W = {"embed": torch.zeros(10, 3, dtype=F64), "bigram": torch.arange(8, dtype=F64)[:, None].expand(8, 3).contiguous()}
    big = {"buckets": 7, "mul_prev": 3, "mul_cur": 5}
    x = plain.embed([4, 9, 9, 0], W, big)
    assert x[:, 0].tolist() == [7.0, (4 * 3 + 9 * 5) % 7, (9 * 3 + 9 * 5) % 7, (9 * 3) % 7]
    assert torch.equal(plain.embed([4, 9], W, None), torch.zeros(2, 3, dtype=F64))


def test_norm_has_eps_inside_the_root():
    x = torch.tensor([[3.0, 4.0]], dtype=F64)
    assert torch.allclose(plain.rms(x, 0.5), x / math.sqrt(12.5 + 0.5))


def test_convolution_is_causal_and_ends_at_the_current_token():
    u = _rand(9, 3, seed=1)
    w = torch.tensor([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0], [1.0, 0.0, 0.0]], dtype=F64)
    y = plain.causal_conv(u, w)
    assert torch.equal(y[:, 0], u[:, 0])                                    # the last tap is the current token's
    assert torch.equal(y[1:, 1], u[:-1, 1]) and y[0, 1] == 0                 # the one before it the previous token's
    assert torch.equal(y[2:, 2], u[:-2, 2]) and torch.equal(y[:2, 2], torch.zeros(2, dtype=F64))


@pytest.mark.parametrize("pairing", ["interleaved", "halves"])
def test_rotation_depends_on_distance_and_leaves_the_rest(pairing):
    rot = {"base": 100.0, "dims": 4}
    q, k = _rand(1, 1, 6, seed=2), _rand(1, 1, 6, seed=3)

    def score(pq, pk):
        n = max(pq, pk) + 1
        a = plain.rotate(q.expand(n, 1, 6), rot, pairing)[pq, 0]
        b = plain.rotate(k.expand(n, 1, 6), rot, pairing)[pk, 0]
        return float(a @ b)
    assert abs(score(7, 3) - score(11, 7)) < 1e-12 and abs(score(7, 3) - score(8, 3)) > 1e-6
    r = plain.rotate(q.expand(5, 1, 6), rot, pairing)
    assert torch.equal(r[:, :, 4:], q.expand(5, 1, 6)[:, :, 4:]) and torch.allclose(r[0], q[0])
    # which features form a pair: a vector with one pair set keeps its length in that pair alone
    e = torch.zeros(2, 1, 6, dtype=F64)
    e[:, 0, 0] = 1.0
    other = 1 if pairing == "interleaved" else 2
    moved = plain.rotate(e, rot, pairing)[1, 0]
    assert abs(float(moved[0]) - math.cos(1.0)) < 1e-12 and abs(float(moved[other]) - math.sin(1.0)) < 1e-12
    e = torch.zeros(2, 1, 6, dtype=F64)
    e[:, 0, 1 if pairing == "halves" else 2] = 1.0                           # the second pair turns by base^(-2/4)
    moved = plain.rotate(e, rot, pairing)[1, 0]
    assert abs(float(moved[1 if pairing == "halves" else 2]) - math.cos(0.1)) < 1e-12


def test_window_counts_the_query_itself_and_the_cap_bends_scores():
    T = 6
    q = torch.zeros(T, 1, 2, dtype=F64)
    k = torch.zeros(T, 1, 2, dtype=F64)
    v = torch.eye(T, dtype=F64).view(T, 1, T)
    o = plain.window_softmax_attention(q, k, v, 1.0, 3)
    assert torch.allclose(o[5], torch.tensor([0, 0, 0, 1 / 3, 1 / 3, 1 / 3], dtype=F64))
    assert torch.allclose(o[1], torch.tensor([0.5, 0.5, 0, 0, 0, 0], dtype=F64))
    assert torch.allclose(plain.window_softmax_attention(q, k, v, 1.0, 1), torch.eye(T, dtype=F64))
    assert torch.allclose(plain.window_softmax_attention(q, k, v, 1.0, None)[5], torch.full((T,), 1 / 6, dtype=F64))
    # one huge score: without a cap it takes everything, with a cap c it weighs e^c against e^0
    q[5, 0, 0], k[4, 0, 0] = 100.0, 100.0
    assert float(plain.window_softmax_attention(q, k, v, 1.0, 3)[5, 4]) > 0.999999
    capped = plain.window_softmax_attention(q, k, v, 1.0, 3, cap=2.0)[5]
    assert abs(float(capped[4]) - math.exp(2.0) / (math.exp(2.0) + 2)) < 1e-9


def test_decay_recurrence_is_a_weighted_sum_of_the_past():
    T, d, dv = 7, 3, 2
    q, k, v = _rand(T, d, seed=4), _rand(T, d, seed=5), _rand(T, dv, seed=6)
    for decay in (0.0, 0.6, 1.0):
        o = plain.decay_recurrence(q, k, v, decay)
        want = torch.stack([sum((decay ** (t - j)) * float(q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)])
        assert torch.allclose(o, want)
    assert torch.allclose(plain.decay_recurrence(q, k, v, 0.0), (q * k).sum(-1, keepdim=True) * v)


def test_delta_rule_writes_overwrites_and_forgets_by_channel():
    d, dv = 4, 3
    e = torch.eye(d, dtype=F64)
    v = _rand(5, dv, seed=7)
    ones, full = torch.ones(5, dtype=F64), torch.ones(5, d, dtype=F64)
    # orthonormal keys, beta 1, no decay: a value is stored under its key, and writing the key again replaces it
    k = torch.stack([e[0], e[1], e[0], e[2], e[1]])
    o = plain.delta_recurrence(k, k, v, ones, full)
    assert torch.allclose(o, v)                                              # the read-out sees the current write
    q = torch.stack([e[0]] * 5)
    o = plain.delta_recurrence(q, k, v, ones, full)
    assert torch.allclose(o[1], v[0]) and torch.allclose(o[2], v[2]) and torch.allclose(o[4], v[2])
    # a decay on channel 0 alone fades what key 0 holds and nothing else
    g = full.clone()
    g[:, 0] = 0.5
    o = plain.delta_recurrence(torch.stack([e[0] + e[1]] * 5), torch.stack([e[0], e[1], e[3], e[3], e[3]]), v, ones, g)
    assert torch.allclose(o[4], v[0] * 0.5 ** 4 + v[1])
    # beta scales the correction: half of the way from what is held to the new value
    o = plain.delta_recurrence(q, torch.stack([e[0]] * 5), v, 0.5 * ones, full)
    assert torch.allclose(o[1], 0.5 * (0.5 * v[0]) + 0.5 * v[1])


def test_experts_cut_off_and_raise():
    W = {"gate": torch.eye(2, dtype=F64), "up": torch.eye(2, dtype=F64), "down": torch.eye(2, dtype=F64)}
    h = torch.tensor([[5.0, -5.0], [0.5, 0.25]], dtype=F64)
    y = plain.expert(h, W, "", 2.0)
    sw = lambda g: g / (1 + math.exp(-1.702 * g))
    assert torch.allclose(y[0], torch.tensor([sw(2.0) * 3.0, sw(-5.0) * (-2.0 + 1.0)], dtype=F64))   # the gate has no floor
    assert torch.allclose(y[1], torch.tensor([sw(0.5) * 1.5, sw(0.25) * 1.25], dtype=F64))


def test_router_groups_correction_and_weights():
    E = 6
    logit = lambda s: math.log(s / (1 - s))
    scores = [0.9, 0.1, 0.5, 0.45, 0.6, 0.2]                                 # groups of 2: sums 1.0, 0.95, 0.8
    W = {"router": torch.diag(torch.tensor([logit(s) for s in scores], dtype=F64)), "correction": torch.zeros(E, dtype=F64)}
    h = torch.ones(1, E, dtype=F64)
    r = {"experts": E, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 2}}
    idx, w = plain.route(h, W, "", r)
    assert sorted(idx[0].tolist()) == [0, 2]                                 # expert 4 (0.6) lies in the group that lost
    assert abs(float(w.sum()) - 3.0) < 1e-9 and abs(float(w[0, idx[0].tolist().index(0)]) - 3.0 * 0.9 / 1.4) < 1e-9
    idx, _ = plain.route(h, W, "", {"experts": E, "top": 2, "scale": 1.0})
    assert sorted(idx[0].tolist()) == [0, 4]                                 # without groups the two largest win
    # the correction moves the choice, not the weights; it may push a whole group below the others
    W["correction"] = torch.tensor([-5.0, -5.0, 0, 0, 0, 0], dtype=F64)
    m = []
    idx, w = plain.route(h, W, "", r, margins=m)
    assert sorted(idx[0].tolist()) == [2, 4]
    assert abs(float(w[0, idx[0].tolist().index(4)]) - 3.0 * 0.6 / 1.1) < 1e-9
    assert abs(float(m[0][0]) - 0.05) < 1e-9                                 # 0.5 was taken, 0.45 was left


def test_a_layer_adds_both_results_times_their_vectors():
    raw = tn.tiny_q()
    raw["layers"] = raw["layers"][1:2]
    arch, cfg = _cfg(raw)
    from cpmcu_amd.weights.random_init import random_tensors
    W = {k: v.to(F64) for k, v in random_tensors(cfg, 11, std=0.1, norm_std=0.2).items()}
    toks = [3, 70, 12, 5]
    _, after = plain.forward(raw, W, toks, return_layers=True)
    x = plain.embed(toks, W, None)
    h = plain.rms(x, 1e-6) * W["l0.norm1"]
    want = x + W["l0.ls1"] * plain.parallel_2_mixer(h, W, "l0.mix.", raw["layers"][0]["mixer"], 1e-6) \
        + W["l0.ls2"] * plain.feed_forward(h, W, "l0.mlp.", raw["layers"][0]["mlp"])
    assert torch.allclose(after[0], want)


def test_borrowed_weights_give_the_same_layer_twice():
    raw = tn.tiny_r()
    arch, cfg = _cfg(raw)
    from cpmcu_amd.weights.random_init import random_tensors
    W = random_tensors(cfg, 12, std=0.1, norm_std=0.2)
    twice = dict(raw, layers=[raw["layers"][1], dict(raw["layers"][1], weights_of=0)])
    own = dict(raw, layers=[raw["layers"][1], raw["layers"][1]])
    W1 = {k.replace("l1.", "l0."): v for k, v in W.items() if not k.startswith(("l0.", "l3."))}
    W2 = dict(W1)
    W2.update({k.replace("l0.", "l1."): v for k, v in W1.items() if k.startswith("l0.")})
    toks = [1, 2, 3, 4, 5, 6, 7]
    assert torch.equal(plain.forward(twice, W1, toks), plain.forward(own, W2, toks))
