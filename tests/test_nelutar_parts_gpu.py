"""Nelutar's mechanisms alone, through their kernel entry points, against the plain implementation (GPU): the bigram
table with the previous token kept in slots; the sum of two results with numbers and vectors; rotation of neighbouring
pairs (alone, and followed by the unit-rms division, from float rows into a bfloat16 cache); capped scores under a
sliding window in the plain and the matrix-core attention kernels, with one key made to stand out just inside and
just outside the window, at page borders, at the first positions and far back; the delta rule with a decay a key
channel in portions and slots; linear attention with a fixed decay (decays of 0 and 1) and what prepares its inputs;
the sigmoid router with groups scored by their two best; experts with the clamped swish in every product that can run
them."""
import math

import pytest
import torch

import plain_nelutar as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def dev(t, dtype=None):
    return t.to(DEV, dtype) if dtype is not None else t.to(DEV)


def i32(x):
    return dev(torch.as_tensor(x, dtype=torch.int32))


def close(got, want, dtype, scale=None, what=""):
    want = want.to(F64)
    tol = (2e-5 if dtype == "float32" else 1.5e-2) * float(scale if scale is not None else want.abs().max())
    err = float((got.detach().cpu().to(F64) - want).abs().max())
    assert err <= tol, f"{what} error {err:.3g} > {tol:.3g}"


# ---------------------------------------------------------------------------
# embedding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("buckets, mul_prev, mul_cur", [(97, 13, 5), (1, 0, 1), (1000003, 40009, 30011)])
def test_bigram_table_in_portions_and_slots(dtype, buckets, mul_prev, mul_cur):
    """Two sequences in slots 2 and 0, cut into steps of unequal sizes down to one token; the first token reads the
    last row; a slot that is used again starts over; a hash beyond 32 bits."""
    from cpmcu_amd import ops
    torch.manual_seed(51)
    H, V = 24, 50000
    rows = min(buckets, 300)
    table = torch.randn(rows + 1, H).to(DT[dtype])
    if buckets > 300:                       # only the rows that the tokens hit exist in this test's table
        big = torch.zeros(buckets + 1, H, dtype=DT[dtype])
    else:
        big = table
    toks = {2: torch.randint(0, V, (23,)).tolist(), 0: torch.randint(0, V, (9,)).tolist()}
    if buckets > 300:
        for t in toks.values():
            for a, b in zip(t[:-1], t[1:]):
                big[(a * mul_prev + b * mul_cur) % buckets] = torch.randn(H).to(DT[dtype])
        big[buckets] = torch.randn(H).to(DT[dtype])
    W = {"embed": torch.zeros(V, H, dtype=F64), "bigram": big.double()}
    want = {s: plain.embed(t, W, {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}) for s, t in toks.items()}
    state = torch.full((3,), 7, dtype=torch.int32, device=DEV)
    state[2] = 0
    state[0] = 0
    cuts = {2: [0, 1, 2, 9, 22, 23], 0: [0, 5, 9]}
    got = {s: [] for s in toks}
    tab = dev(big)
    for step in range(5):
        batch = [(s, cuts[s][step], cuts[s][step + 1]) for s in (2, 0) if step + 1 < len(cuts[s])]
        ids, pos, slot, cu = [], [], [], [0]
        for s, a, b in batch:
            ids += toks[s][a:b]
            pos += list(range(a, b))
            slot += [s] * (b - a)
            cu.append(cu[-1] + b - a)
        x = torch.full((len(ids), H), 0.5, device=DEV)
        ops.bigram_add(tab, i32(ids), i32(pos), i32(slot), state, i32(cu), i32([s for s, _, _ in batch]), x, buckets,
                       mul_prev, mul_cur)
        for i, (s, _, _) in enumerate(batch):
            got[s].append(x[cu[i]:cu[i + 1]].cpu() - 0.5)
    for s in toks:
        close(torch.cat(got[s]), want[s], "float32", scale=1.0)
    assert state.tolist() == [toks[0][-1], 7, toks[2][-1]]


# ---------------------------------------------------------------------------
# joining two results
@pytest.mark.parametrize("case", [(5, 96, 3, "float32", 1, "float32", True, True), (200, 100, 1, "bfloat16", 4, "float32", False, True),
                                  (1, 4096, 16, "float32", 16, "float32", True, False), (7, 33, 1, "bfloat16", 1, "bfloat16", False, False),
                                  (3, 64, 2, "float32", 0, None, True, True)])
def test_sum_of_two_results_with_numbers_and_vectors(case):
    from cpmcu_amd import ops
    n, H, ap, adt, fp, fdt, biased, vectors = case
    torch.manual_seed(52)
    shape = lambda p: (p, n, H) if p > 1 else (n, H)
    a = torch.randn(shape(ap)).to(DT[adt])
    f = torch.randn(shape(fp)).to(DT[fdt]) if fp else None
    ab, fb = (torch.randn(H), torch.randn(H)) if biased else (None, None)
    wa, wf = (torch.randn(H), torch.randn(H)) if vectors else (None, None)
    sa, sf = (1.0, 1.0) if vectors else (0.7, -1.3)
    total = lambda t: t.double().sum(0) if t.dim() == 3 else t.double()
    want = sa * (wa.double() if vectors else 1.0) * (total(a) + (ab.double() if biased else 0.0))
    if f is not None:
        want = want + sf * (wf.double() if vectors else 1.0) * (total(f) + (fb.double() if biased else 0.0))
    out = torch.empty(n, H, device=DEV)
    g = lambda t: dev(t) if t is not None else None
    ops.scaled_branches(dev(a), g(ab), g(wa), sa, g(f), g(fb) if f is not None else None, g(wf) if f is not None else None, sf, out)
    close(out, want, "float32", scale=float(want.abs().max()) * (400 if "bfloat16" in (adt, fdt) else 1))


# ---------------------------------------------------------------------------
# rotation of neighbouring pairs
def _store_and_read(ops, row, H, G, d, dv, pos, dtype, page, table, store, window=0, scale=0.4, softcap=0.0):
    """Stores k and v of `row` through `store` and reads them back by attention with random queries."""
    T = row.shape[0]
    pk, pv = -(-d // 16) * 16, -(-dv // 16) * 16
    kp = torch.zeros(int(table.max()) + 1, page, G * pk, dtype=DT[dtype], device=DEV)
    vp = torch.zeros(int(table.max()) + 1, page, G * pv, dtype=DT[dtype], device=DEV)
    q_out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
    slot = i32([1] * T)
    store(q_out, kp, vp, slot)
    qq = torch.randn(T, H, d).to(DT[dtype])
    out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
    ops.attention_general(dev(qq.reshape(T, H * d)), out, H, G, d, dv, scale, kp, vp, dev(table), page, i32(pos.tolist()), slot,
                          0, window, 0, None, softcap=softcap)
    return q_out, qq, out, kp, vp


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(6, 2, 24, 40, 8), (2, 1, 32, 16, 32), (3, 1, 24, 24, 0), (5, 5, 20, 28, 6), (4, 2, 128, 128, 128), (4, 2, 16, 8, 2)])
@pytest.mark.parametrize("normed", [False, True])
def test_rotation_of_neighbouring_pairs(dtype, shape, normed):
    """q and k heads: pairs (2i, 2i + 1) of the first features rotate; with `normed` every head is then divided by
    its root mean square, and the rows come as float (what a convolution leaves) whatever the cache's type.  The
    pages are read back through attention with given queries."""
    from cpmcu_amd import ops
    H, G, d, dv, rd = shape
    torch.manual_seed(53)
    T, page, eps = 150, 64, 1e-5
    rot = {"base": 300.0, "dims": rd} if rd else None
    row = (torch.randn(T, H * d + G * d + G * dv) * 2).to(torch.float32 if normed else DT[dtype])
    q_raw, k_raw, v_raw = row.double().split([H * d, G * d, G * dv], 1)
    rows64 = lambda x, n: x.reshape(T, n, d)
    q_want, k_want = plain.rotate(rows64(q_raw, H), rot, "interleaved"), plain.rotate(rows64(k_raw, G), rot, "interleaved")
    if normed:
        q_want, k_want = plain.rms(q_want, eps), plain.rms(k_want, eps)
    table = torch.zeros(2, 4, dtype=torch.int32)
    table[1] = torch.tensor([3, 0, 4, 1])
    pos = torch.arange(T)
    inv = dev((300.0 ** (-torch.arange(0, rd, 2, dtype=F64) / rd)).float()) if rd else None

    def store(q_out, kp, vp, slot):
        if normed:
            ops.qkv_norm_rotate_store(dev(row), q_out, H, G, d, dv, rd, i32(pos.tolist()), slot, inv, 1.0, kp, vp, dev(table),
                                      page, eps=eps, norm_after=True, interleaved=True)
        else:
            ops.qkv_rotate_store(dev(row), q_out, H, G, d, dv, rd, i32(pos.tolist()), slot, inv, 1.0, kp, vp, dev(table), page,
                                 interleaved=True)
    q_out, qq, out, _, _ = _store_and_read(ops, row, H, G, d, dv, pos, dtype, page, table, store, window=30)
    close(q_out, q_want.reshape(T, H * d), dtype)
    want = plain.window_softmax_attention(qq.double(), k_want, v_raw.reshape(T, G, dv), 0.4, 30)
    close(out, want, dtype)


# ---------------------------------------------------------------------------
# capped scores under a sliding window
def _edge_case(T, H, G, d, dv, window, tall, seed):
    """Random q, k, v in which, for every query in `tall` (query position -> key position), that key alone has a huge
    score with every head of the query."""
    g = torch.Generator().manual_seed(seed)
    q, k = torch.randn(T, H, d, generator=g) * 0.3, torch.randn(T, G, d, generator=g) * 0.3
    v = torch.randn(T, G, dv, generator=g)
    for i, (qp, kp_) in enumerate(tall.items()):
        axis = i % d
        k[kp_, :, axis] = 14.0
        q[qp, :, axis] = 14.0
    return q, k, v


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(6, 2, 24, 40, 20, 5.0), (2, 1, 32, 16, 70, 3.0), (4, 4, 16, 16, 64, 0.0), (4, 2, 16, 8, 1, 0.5),
                                   (8, 1, 64, 64, 96, 8.0), (3, 1, 24, 24, 0, 2.0)])
def test_capped_scores_under_a_window(dtype, shape):
    """One key with a score of about 78 (the scale is 0.4): just inside the window it takes all the weight without a
    cap and e^c against the others' e^(about 0) with one; just outside it must not be seen at all.  Such keys stand
    at distances window - 1 and window, at page borders (63, 64, 127, 128), at position 0 and far back; prompts
    through the plain kernel and the matrix-core kernel (a token a tile, token tiles), single tokens with whole and
    with split keys."""
    from cpmcu_amd import ops
    H, G, d, dv, window, cap = shape
    T, page = 300, 64
    w = window or T
    tall = {}
    for qp in (w - 1, w, 150, 151, 190, 191, 255, 256, 299):
        if qp < T:
            tall[qp] = max(qp - w + 1, 0) if qp % 2 else max(qp - w, 0)      # odd queries: the oldest visible key; even: the first lost one
    tall[130] = 128
    tall[131] = 64 if w > 67 else 131 - min(w, 131) + 1
    q, k, v = _edge_case(T, H, G, d, dv, window, tall, 54)
    q, k, v = (t.to(DT[dtype]) for t in (q, k, v))
    want = plain.window_softmax_attention(q.double(), k.double(), v.double(), 0.4, window or None, cap or None)
    row = torch.cat([q.reshape(T, H * d), k.reshape(T, G * d), v.reshape(T, G * dv)], 1)
    table = torch.zeros(2, 5, dtype=torch.int32)
    table[1] = torch.tensor([3, 0, 4, 1, 5])
    pos = torch.arange(T)

    def store(q_out, kp, vp, slot):
        ops.qkv_rotate_store(dev(row), q_out, H, G, d, dv, 0, i32(pos.tolist()), slot, None, 1.0, kp, vp, dev(table), page)
    q_out, _, _, kp, vp = _store_and_read(ops, row, H, G, d, dv, pos, dtype, page, table, store)
    slot = i32([1] * T)
    out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
    ops.attention_general(q_out, out, H, G, d, dv, 0.4, kp, vp, dev(table), page, i32(pos.tolist()), slot, 0, window, 0, None,
                          softcap=cap)
    close(out, want, dtype, what="plain kernel")
    if dtype != "bfloat16":
        return
    pv = -(-dv // 16) * 16
    cases = [(0, T, 1, False), (T - 1, T, 1, False), (T - 1, T, 3, False), (255, 257, 2, False), (130, 132, 1, False)]
    if H // G <= 8:
        cases.append((0, T, 1, True))
    for a, b, splits, tiled in cases:
        out = torch.empty(b - a, H * dv, dtype=torch.bfloat16, device=DEV)
        po = torch.empty(b - a, H, splits, dv, device=DEV) if splits > 1 else None
        pm = torch.empty(b - a, H, splits, 2, device=DEV) if splits > 1 else None
        tiles, tpt = None, 1
        if tiled:
            tpt = ops.attention_general_tokens_per_tile(b - a, H, G, pv)
            assert tpt > 1
            tiles = ops.prefill_tiles([b - a], tpt, DEV)
        ops.attention_general_mfma(q_out[a:b], out, H, G, d, dv, 0.4, kp, vp, dev(table), page, i32(pos[a:b].tolist()), slot[a:b],
                                   0, splits, po, pm, tiles, tpt, window=window, softcap=cap)
        close(out, want[a:b], "bfloat16", what=f"matrix cores rows {a}..{b} splits {splits} tiled {tiled}")


# ---------------------------------------------------------------------------
# recurrences
def _channel_plain(qkv, a, b, A_log, dt_bias, H, G, d, dv):
    T = qkv.shape[0]
    q, k, v = qkv.double().split([G * d, G * d, H * dv], 1)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k, v = unit(q.reshape(T, G, d)) * d ** -0.5, unit(k.reshape(T, G, d)), v.reshape(T, H, dv)
    beta = torch.sigmoid(b.double())
    g = torch.exp(-torch.exp(A_log.double())[None, :, None] * plain.softplus(a.double() + dt_bias.double()).reshape(T, H, d))
    rep = H // G
    return torch.stack([plain.delta_recurrence(q[:, i // rep], k[:, i // rep], v[:, i], beta[:, i], g[:, i]) for i in range(H)],
                       1).reshape(T, H * dv)


def _decay_plain(qkv, decay, H, d, dv):
    T = qkv.shape[0]
    q, k, v = qkv.double().split([H * d, H * d, H * dv], 1)
    q, k, v = q.reshape(T, H, d), k.reshape(T, H, d), v.reshape(T, H, dv)
    return torch.stack([plain.decay_recurrence(q[:, i], k[:, i], v[:, i], float(decay[i])) for i in range(H)], 1).reshape(T, H * dv)


@pytest.mark.parametrize("lanes", [0, 8, 16])
@pytest.mark.parametrize("rule", ["channel", "decay"])
@pytest.mark.parametrize("shape", [(4, 2, 24, 20), (1, 1, 72, 8), (2, 1, 12, 7), (3, 3, 8, 36), (4, 1, 32, 40), (4, 2, 128, 128),
                                   (2, 2, 256, 16), (2, 1, 200, 50)])
def test_recurrences_in_portions_and_slots(rule, shape, lanes):
    """Two sequences in slots 3 and 1, in portions of unequal sizes down to one token: the state is carried in the
    slot; a slot that is freed (its state cleared) and used again starts from nothing; a pass that does not write
    leaves the state as it was.  The delta rule's decays differ from channel to channel, from nearly 1 to nearly 0;
    the fixed decays include 0 (nothing is kept) and 1 (nothing is lost)."""
    from cpmcu_amd import ops
    H, G, d, dv = shape
    if rule == "decay":
        G = H
    torch.manual_seed(55)
    lens = {3: 41, 1: 12}
    C = 2 * G * d + H * dv
    A_log = torch.linspace(-4.0, 1.5, H)
    dt_bias = torch.randn(H * d)
    decay = torch.tensor(([0.0, 1.0, 0.9, 0.5] * H)[:H])
    data, want = {}, {}
    for s, L in lens.items():
        qkv = torch.randn(L, C) * (1.0 if rule == "channel" else 0.5)
        gates = (torch.randn(L, 3 + H) * 2).bfloat16()                   # wider rows: beta's columns lie at offset 3
        wide = torch.randn(L, H * d + 5) * 2                             # and the decay's at offset 2 of other rows
        data[s] = (qkv, gates, wide)
        want[s] = (_channel_plain(qkv, wide[:, 2:2 + H * d], gates[:, 3:], A_log, dt_bias, H, G, d, dv) if rule == "channel"
                   else _decay_plain(qkv, decay, H, d, dv))
    state = torch.zeros(4, H, dv, d, device=DEV)
    state[0] = 5.0
    cuts = {3: [0, 1, 2, 9, 40, 41], 1: [0, 5, 12]}
    got = {s: [] for s in lens}

    def run(batch, write=True):
        cu = [0]
        for s, a, b in batch:
            cu.append(cu[-1] + b - a)
        qkv = dev(torch.cat([data[s][0][a:b] for s, a, b in batch]))
        y = torch.empty(cu[-1], H * dv, device=DEV)
        slots = i32([s for s, _, _ in batch])
        if rule == "channel":
            gates = dev(torch.cat([data[s][1][a:b] for s, a, b in batch]))
            wide = dev(torch.cat([data[s][2][a:b] for s, a, b in batch]))
            ops.delta_scan(qkv, gates, 0, 3, dev(dt_bias), dev(A_log), state, y, i32(cu), slots, H, G, d, dv, d ** -0.5,
                           write_state=write, lanes=lanes, rule="channel", channel_decay=wide[:, 2:2 + H * d])
        else:
            ops.delta_scan(qkv, None, 0, 0, None, dev(decay), state, y, i32(cu), slots, H, H, d, dv, 1.0, write_state=write,
                           lanes=lanes, rule="decay")
        return [y[cu[i]:cu[i + 1]].cpu() for i in range(len(batch))]

    for step in range(5):
        batch = [(s, cuts[s][step], cuts[s][step + 1]) for s in (3, 1) if step + 1 < len(cuts[s])]
        if step == 3:
            before = state.clone()
            run(batch, write=False)
            assert torch.equal(state, before)
        for (s, _, _), y in zip(batch, run(batch)):
            got[s].append(y)
    for s in lens:
        close(torch.cat(got[s]), want[s], "float32", scale=float(want[s].abs().max()))
    assert float((state[0] - 5.0).abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0
    state[3] = 0.0                                                        # the slot is given to another sequence
    close(run([(3, 0, 7)])[0], want[3][:7], "float32", scale=float(want[3].abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [(3, 16, 24, 16, "halves", False, 0.25), (2, 32, 8, 0, "halves", True, 1.0), (5, 20, 12, 6, "interleaved", True, 1.0),
                                  (1, 12, 7, 12, "interleaved", False, 2.0)])
def test_what_prepares_linear_attention(dtype, case):
    """From columns of a wider projection to float rows [q | k | v]: SiLU or nothing, a rotation of the first
    features in either pairing at positions away from zero, k times a number afterwards."""
    from cpmcu_amd import ops
    H, d, dv, rd, pairing, silu, ks = case
    torch.manual_seed(56)
    T = 37
    proj = (torch.randn(T, 3 + 2 * H * d + 2 * H * dv) * 1.5).to(DT[dtype])
    q_off, k_off, v_off = 3, 3 + H * d, 3 + 2 * H * d
    pos = torch.arange(T) + 1000
    rot = {"base": 500.0, "dims": rd} if rd else None
    act = (lambda z: plain.silu(z)) if silu else (lambda z: z)

    def turned(x):
        full = torch.zeros(T + 1000, H, d, dtype=F64)
        full[1000:] = x
        return plain.rotate(full, rot, pairing)[1000:]
    p64 = proj.double()
    q = turned(act(p64[:, q_off:q_off + H * d]).reshape(T, H, d))
    k = turned(act(p64[:, k_off:k_off + H * d]).reshape(T, H, d)) * ks
    v = act(p64[:, v_off:v_off + H * dv])
    out = torch.empty(T, 2 * H * d + H * dv, device=DEV)
    inv = dev((500.0 ** (-torch.arange(0, rd, 2, dtype=F64) / rd)).float()) if rd else None
    ops.linear_attention_prepare(dev(proj), q_off, k_off, v_off, out, H, d, dv, silu, i32(pos.tolist()), inv,
                                 pairing == "interleaved", ks)
    want = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v], 1)
    close(out, want, "float32", scale=float(want.abs().max()) * (20 if rd else 1))       # angles of a thousand radians in float


# ---------------------------------------------------------------------------
# routed experts
@pytest.mark.parametrize("case", [(12, 2, (3, 2), 1.7), (5, 5, None, 1.0), (8, 1, (8, 1), 0.5), (64, 6, (4, 2), 2.0), (16, 4, (4, 3), 2.2),
                                  (130, 4, (13, 5), 1.0)])
def test_sigmoid_router_with_groups_scored_by_their_two_best(case):
    """Choice scores s + correction (corrections large enough to turn choices, also below zero), groups by the sum of
    their two best, the others shut out, weights from s alone, times the scale.  Tokens whose choice is a close call
    in float64 are left out."""
    from cpmcu_amd import ops
    E, top, groups, scale = case
    torch.manual_seed(57)
    n, H = 300, 48
    h = torch.randn(n, H)
    W = {"router": torch.randn(E, H) * 0.3, "correction": torch.randn(E) * 0.8}
    r = {"experts": E, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    margins = []
    idx_want, w_want = plain.route(h.double(), {k: v.double() for k, v in W.items()}, "", r, margins)
    clear = margins[0] > 1e-4
    assert int(clear.sum()) > 250
    idx = torch.empty(n, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(n, top, device=DEV)
    ops.moe_route(dev(h), dev(W["router"]), dev(W["correction"]), None, groups[0] if groups else 1, groups[1] if groups else 1,
                  top, idx, wts, score="sigmoid", group_score="top2_sum", weight_scale=scale)
    got = torch.zeros(n, E, dtype=F64).scatter_(1, idx.cpu().long(), wts.cpu().double())
    want = torch.zeros(n, E, dtype=F64).scatter_(1, idx_want, w_want)
    assert float((got - want)[clear].abs().max()) < 1e-5
    assert float((got.sum(1) - scale).abs().max()) < 1e-4


def _experts_plain(h, gate_up, down, idx, wts, limit):
    n, top = idx.shape
    out = torch.zeros(n, down.shape[1], dtype=F64)
    F = gate_up.shape[1] // 2
    for t in range(n):
        for j in range(top):
            e = int(idx[t, j])
            W = {"gate": gate_up[e, :F].double(), "up": gate_up[e, F:].double(), "down": down[e].double()}
            out[t] += float(wts[t, j]) * plain.expert(h[t:t + 1].double(), W, "", limit)[0]
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [(5, 96, 40, 12, 2, 1.2), (3, 100, 28, 5, 5, 0.8), (200, 64, 16, 64, 6, 1.0), (130, 96, 40, 12, 2, 0.3)])
def test_experts_with_the_clamped_swish(dtype, case):
    """Few tokens (an expert's rows stream for every token that chose it) and many (pairs grouped by expert on the
    matrix cores), limits that cut off a good part of the products, a shared expert's result added without a gate."""
    from cpmcu_amd import ops
    n, H, F, E, top, limit = case
    torch.manual_seed(58)
    h = torch.randn(n, H).to(DT[dtype])
    gate_up = (torch.randn(E, 2 * F, H) * 0.3).to(DT[dtype])
    down = (torch.randn(E, H, F) * 0.3).to(DT[dtype])
    idx = torch.stack([torch.randperm(E)[:top] for _ in range(n)]).int()
    wts = torch.rand(n, top)
    shared = torch.randn(n, H)
    want = _experts_plain(h, gate_up, down, idx, wts, limit) + shared.double()
    act = torch.empty(n, top, F, dtype=DT[dtype], device=DEV)
    out = torch.empty(n, H, device=DEV)
    ops.moe_gated(dev(h), dev(gate_up), dev(idx), act, activation=("clamped_swish", limit))
    ops.moe_down(act, dev(down), dev(idx), dev(wts), out, dev(shared), None)
    close(out, want, dtype, what="few tokens")
    tiles = ops.moe_tiles(n, top, E)
    if dtype == "bfloat16" and ops.moe_experts_mfma_ok(dev(h), F, tiles):
        out2 = torch.empty(n, H, device=DEV)
        y = torch.empty(n, top, H, dtype=torch.bfloat16, device=DEV)
        rows = torch.empty(tiles * ops.MOE_TILE, dtype=torch.int32, device=DEV)
        ops.moe_experts_mfma(dev(h), dev(gate_up), dev(down), dev(idx), dev(wts), out2, act, y, rows,
                             torch.empty(tiles, dtype=torch.int32, device=DEV), torch.empty(1, dtype=torch.int32, device=DEV),
                             dev(shared), None, activation=("clamped_swish", limit))
        close(out2, want, dtype, what="many tokens", scale=float(want.abs().max()) * 1.5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n", [1, 9, 40, 200])
def test_gated_product_with_the_clamped_swish(dtype, n):
    """The shared expert is a gated feed-forward of the package: its nonlinearity in the strip kernel (up to 16 rows),
    the skinny product (up to 64), the elementwise kernel behind the library's product, and the float kernel."""
    from cpmcu_amd import ops
    torch.manual_seed(59)
    K, F, limit = 128, 64, 0.7
    x = torch.randn(n, K).to(DT[dtype])
    w = (torch.randn(2 * F, K) * 0.2).to(DT[dtype])
    g, u = (x.double() @ w.double().T).split([F, F], 1)
    g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
    want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    gu = torch.empty(n, 2 * F, dtype=DT[dtype], device=DEV)
    ops.linear(dev(x), dev(w), gu)
    out = torch.empty(n, F, dtype=DT[dtype], device=DEV)
    ops.silu_mul(gu, out, ("clamped_swish", limit))
    close(out, want, dtype, what="elementwise")
    if dtype == "bfloat16":
        tiled = ops.TiledWeight(dev(w))
        if n <= ops.STRIP_ROWS:
            out = torch.empty(n, F, dtype=torch.bfloat16, device=DEV)
            ops.gated_strip(dev(x), tiled, out, activation=("clamped_swish", limit))
            close(out, want, dtype, what="strip")
        if n <= ops.SKINNY_MAX_ROWS:
            out = torch.empty(n, F, dtype=torch.bfloat16, device=DEV)
            ops.gemm_skinny(dev(x), tiled, out, mode="gated", activation=("clamped_swish", limit))
            close(out, want, dtype, what="skinny")
    with pytest.raises(ops.KernelError):
        ops.silu_mul(gu, out, "clamped_swish")                            # the limit is part of the nonlinearity


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
def test_one_norm_over_all_heads_with_a_sigmoid_gate_behind_it(out_dtype):
    from cpmcu_amd import ops
    torch.manual_seed(60)
    n, W, eps = 9, 2 * 36, 1e-5
    y, w = torch.randn(n, W) * 3, torch.randn(W)
    wide = (torch.randn(n, W + 7) * 2).to(DT[out_dtype])
    out = torch.empty(n, W, dtype=DT[out_dtype], device=DEV)
    ops.rms_norm_groups(dev(y), dev(w), eps, out, groups=1, gate=dev(wide)[:, 5:5 + W], gate_after=True)
    want = plain.rms(y.double(), eps) * w.double() * torch.sigmoid(wide[:, 5:5 + W].double())
    close(out, want, out_dtype)
    ops.rms_norm_groups(dev(y), None, eps, out, groups=2, gate=dev(wide)[:, 5:5 + W], gate_after="silu")
    want = plain.rms(y.double().reshape(n, 2, 36), eps).reshape(n, W) * plain.silu(wide[:, 5:5 + W].double())
    close(out, want, out_dtype)
