"""Sagedra's mechanisms alone, through their kernel entry points, against the plain implementation (GPU): the norm
that reads and writes a residual of several streams (row kernels for few and many rows, odd widths, partial sums,
biases, chosen rows); the mean of two normed branches; convolutions with a pending bias and no activation, in
portions; rotation with stretched frequencies followed by the unit-rms division; attention with two score maps a
head over shared values (plain and matrix-core kernels, prompts in token tiles, single tokens with shared keys,
wide values), with one key far back that one map alone sees; the gated delta rule in portions and slots; the gated
group norm behind it; gates, the logit cap, the GELU-gated product and the scaled embedding."""
import math

import pytest
import torch

import plain_sagedra as plain

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
# residual streams and the norm that reads them

def _streams_plain(X, y, mix, outw, read, w, eps, rms):
    X = X.double()
    if y is not None:
        S = X.shape[0]
        m = mix.double() if mix is not None else torch.eye(S, dtype=F64)
        o = outw.double() if outw is not None else torch.ones(S, dtype=F64)
        X = torch.einsum("st,snh->tnh", m, X) + o[:, None, None] * y.double()[None]
    r = read.double() if read is not None else torch.ones(X.shape[0], dtype=F64)
    u = torch.einsum("s,snh->nh", r, X)
    return X, (plain.rms(u, eps) * w.double() if rms else plain.layer_norm(u, w.double(), eps))


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [
    # streams, rows, width, partial sums, branch type, bias, chosen rows
    (4, 8, 4096, 16, "float32", False, False),     # a decode step: a row over 1,024 threads, 16 partial sums
    (2, 3, 96, 5, "float32", True, False),
    (1, 7, 100, 1, "bfloat16", True, False),       # one stream with mixing numbers of its own
    (3, 5, 101, 3, "float32", False, False),       # a width no 16-byte access suits
    (4, 600, 512, 1, "bfloat16", False, False),    # a prompt: smaller workgroups, 2 vectors a thread
    (5, 40, 14000, 2, "float32", True, False),     # 4 vectors a thread of 1,024
    (8, 9, 64, 9, "float32", False, True),
    (4, 33, 2048, 8, "float32", True, True),
])
def test_norm_over_residual_streams(case, out_dtype):
    from cpmcu_amd import ops
    S, n, H, P, btype, with_bias, chosen = case
    torch.manual_seed(31)
    eps = 1e-5
    w = torch.rand(H) + 0.5
    for rms in (False, True):
        X = torch.randn(S, n, H) + 0.7                     # a mean away from zero: the norm must take it off
        parts = (torch.randn(P, n, H) * 0.5).to(DT[btype])
        bias = torch.randn(H) if with_bias else None
        mix, outw, read = torch.randn(S, S) * 0.6, torch.randn(S), torch.randn(S)
        y = parts.double().sum(0) * 0.5 + (bias.double() if with_bias else 0.0)
        rows = [n - 1, 0, n // 2] if chosen else None
        # first a read of fresh streams (no branch), then with a branch to add
        Xd = dev(X.clone())
        out = torch.empty(n, H, dtype=DT[out_dtype], device=DEV)
        ops.streams_norm(Xd, None, None, 1.0, None, None, dev(read), dev(w), eps, out, rms=rms)
        close(out, _streams_plain(X, None, None, None, read, w, eps, rms)[1], out_dtype, what="read")
        assert torch.equal(Xd.cpu(), X)
        X_want, h_want = _streams_plain(X, y, mix, outw, read, w, eps, rms)
        branch = dev(parts if P > 1 else parts[0])
        out = torch.empty(len(rows) if chosen else n, H, dtype=DT[out_dtype], device=DEV)
        ops.streams_norm(Xd, branch, dev(bias) if with_bias else None, 0.5, dev(mix), dev(outw), dev(read), dev(w), eps, out,
                         rows=i32(rows) if chosen else None, rms=rms)
        close(out, h_want[rows] if chosen else h_want, out_dtype, what="norm")
        if chosen:
            assert torch.equal(Xd.cpu(), X)
        else:
            close(Xd, X_want, "float32", what="streams")
    # a residual of one row a token ([n, H]) with a plain add: mixing numbers absent
    x = torch.randn(n, H)
    b = torch.randn(n, H)
    xd = dev(x.clone())
    out = torch.empty(n, H, dtype=DT[out_dtype], device=DEV)
    ops.streams_norm(xd, dev(b), None, 1.0, None, None, None, dev(w), eps, out)
    close(out, plain.layer_norm((x + b).double(), w.double(), eps), out_dtype)
    close(xd, (x + b).double(), "float32")


def test_streams_start_as_copies():
    from cpmcu_amd import ops
    x = torch.randn(11, 100)
    X = torch.empty(3, 11, 100, device=DEV)
    ops.streams_fill(dev(x), X)
    assert torch.equal(X.cpu(), x[None].expand(3, -1, -1))


@pytest.mark.parametrize("case", [(8, 4096, 8, 16, "float32", "float32"), (3, 100, 1, 1, "bfloat16", "float32"),
                                  (5, 101, 2, 3, "float32", "float32"), (700, 256, 1, 1, "bfloat16", "bfloat16"),
                                  (9, 96, 4, 1, "float32", "bfloat16"), (4, 14000, 2, 2, "float32", "float32")])
def test_mean_of_two_normed_branches(case):
    from cpmcu_amd import ops
    n, H, pa, pb, ta, tb = case
    torch.manual_seed(32)
    eps = 1e-6
    a = (torch.randn(pa, n, H) * 3).to(DT[ta])
    b = (torch.randn(pb, n, H) * 0.1).to(DT[tb])
    a_bias, wa, wb = torch.randn(H), torch.rand(H) + 0.5, torch.rand(H) + 0.5
    left, right = a.double().sum(0) + a_bias.double(), b.double().sum(0)
    want = 0.5 * (plain.rms(left, eps) * wa.double() + plain.rms(right, eps) * wb.double())
    out = torch.empty(n, H, device=DEV)
    ops.pair_norm_mean(dev(a if pa > 1 else a[0]), dev(a_bias), dev(b if pb > 1 else b[0]), None, dev(wa), dev(wb), eps, out)
    close(out, want, "float32" if ta == tb == "float32" else "bfloat16")


# ---------------------------------------------------------------------------
# convolution with a pending bias, without activation, in portions

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_convolution_without_activation_in_portions(dtype, taps):
    """Two sequences in slots 2 and 0, cut into portions of unequal sizes (also a single token, fewer than the
    taps): the slots' last inputs carry the convolution over the cuts; a slot used again starts from zeros."""
    from cpmcu_amd import ops
    torch.manual_seed(33)
    C, lens = 52, {2: 23, 0: 9}
    w = torch.randn(C, taps)
    bias = torch.randn(C)
    u = {s: torch.randn(L, C).to(DT[dtype]) for s, L in lens.items()}
    want = {s: plain.causal_conv(u[s].double() + bias.double(), w.double()) for s in lens}
    state = torch.full((3, taps - 1, C), 7.0, device=DEV) if taps > 1 else None
    if state is not None:
        state[[0, 2]] = 0.0                                              # what acquiring a slot does
    cuts = {2: [0, 1, 3, 4, 15, 23], 0: [0, 2, 9]}
    got = {s: [] for s in lens}
    for step in range(5):
        batch = [(s, cuts[s][step], cuts[s][step + 1]) for s in (2, 0) if step + 1 < len(cuts[s])]
        rows = torch.cat([u[s][a:b] for s, a, b in batch])
        cu = [0]
        for s, a, b in batch:
            cu.append(cu[-1] + b - a)
        out = torch.empty(rows.shape[0], C, device=DEV)
        ops.conv_silu(dev(rows), dev(w), None, state, out, i32(cu), i32([s for s, _, _ in batch]),
                      max(b - a for _, a, b in batch), update_state=True, in_bias=dev(bias), activation=False)
        for i, (s, a, b) in enumerate(batch):
            got[s].append(out[cu[i]:cu[i + 1]].cpu())
    for s in lens:
        close(torch.cat(got[s]), want[s], dtype)
    if state is not None:
        assert float((state[1] - 7.0).abs().max()) == 0.0                # a slot that no sequence used


# ---------------------------------------------------------------------------
# rotation with stretched frequencies, then the division by the root mean square

def test_stretched_frequencies():
    from cpmcu_amd.parts import POSITION_ENCODINGS
    from cpmcu_amd.parts.base import Runtime
    rt = Runtime(torch.device("cpu"), torch.float32, None, 4096)
    for dims, base, sc in ((16, 10000.0, (4.0, 1.0, 3.0, 64)), (64, 500000.0, (8.0, 1.0, 4.0, 8192)), (8, 100.0, (2.0, 2.0, 8.0, 40)),
                           (32, 50.0, (3.0, 0.5, 1.5, 16))):
        enc = POSITION_ENCODINGS.build("llama3", head_dim=dims, theta=base, factor=sc[0], low=sc[1], high=sc[2], original=sc[3])
        enc.bind({}, rt)
        rot = {"base": base, "dims": dims, "scaling": dict(zip(("factor", "low", "high", "original"), sc))}
        want = plain.frequencies(rot)
        assert float((enc.inv_freq.double() - want).abs().max() / want.max()) < 1e-6
        kinds = {("same" if abs(a - b) < 1e-12 else ("slow" if abs(a / sc[0] - b) < 1e-12 else "blend"))
                 for a, b in zip(plain.frequencies({"base": base, "dims": dims}).tolist(), want.tolist())}
        if dims >= 16:
            assert {"same", "slow"} <= kinds


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(6, 2, 24, 40, 16), (2, 2, 32, 16, 32), (3, 1, 24, 24, 0), (5, 5, 20, 28, 6), (4, 4, 128, 128, 128)])
def test_rotation_then_unit_rms(dtype, shape):
    """q and k heads: the first features rotate (stretched frequencies), then every head is divided by its root
    mean square; v is stored as projected.  The pages are read back through attention with given queries."""
    from cpmcu_amd import ops
    H, G, d, dv, rd = shape
    torch.manual_seed(34)
    T, page, eps = 150, 64, 1e-5
    rot = {"base": 300.0, "dims": rd, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 64}}
    row = (torch.randn(T, H * d + G * d + G * dv) * 2).to(DT[dtype])
    pos = torch.arange(T) + 70                                           # positions away from zero
    q_raw, k_raw, v_raw = row.double().split([H * d, G * d, G * dv], 1)
    q_want = plain.rms(plain.rotate(q_raw.reshape(T, H, d), pos, rot if rd else None), eps)
    k_want = plain.rms(plain.rotate(k_raw.reshape(T, G, d), pos, rot if rd else None), eps)
    pk, pv = -(-d // 16) * 16, -(-dv // 16) * 16
    kp = torch.zeros(5, page, G * pk, dtype=DT[dtype], device=DEV)
    vp = torch.zeros(5, page, G * pv, dtype=DT[dtype], device=DEV)
    table = torch.zeros(2, 4, dtype=torch.int32)
    table[1] = torch.tensor([3, 0, 4, 1])
    inv = dev(plain.frequencies(rot).float()) if rd else None
    q_out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
    slot = i32([1] * T)
    ops.qkv_norm_rotate_store(dev(row), q_out, H, G, d, dv, rd, i32(pos.tolist()), slot, inv, 1.0, kp, vp, dev(table), page,
                              eps=eps, norm_after=True)
    close(q_out, q_want.reshape(T, H * d), dtype)
    qq = torch.randn(T, H, d).to(DT[dtype])
    out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
    # the keys lie at cache rows pos; the first 70 rows hold nothing, so only queries whose window of 30 lies within
    # the stored rows are compared
    ops.attention_general(dev(qq.reshape(T, H * d)), out, H, G, d, dv, 0.4, kp, vp, dev(table), page, i32(pos.tolist()), slot,
                          0, 30, 0, None)
    mask = plain.visible(T, 30)
    want = plain.softmax_attention(qq.double(), k_want.repeat_interleave(H // G, 1),
                                   v_raw.reshape(T, G, dv).repeat_interleave(H // G, 1), 0.4, mask)
    close(out[29:], want.reshape(T, H * dv)[29:], dtype)


@pytest.mark.parametrize("shape", [(6, 2, 24, 40), (2, 2, 32, 16), (4, 1, 64, 64), (8, 8, 16, 24), (32, 8, 128, 128)])
def test_output_gate_in_the_attention_kernel(shape):
    """The matrix-core kernel multiplies what it writes with sigmoid of a gate row (a column slice of a wider
    projection): prompts a token a tile and in token tiles, single tokens with whole and with split keys."""
    from cpmcu_amd import ops
    H, G, d, dv = shape
    torch.manual_seed(39)
    T, page, eps = 300, 64, 1e-5
    row = torch.randn(T, H * d + G * d + G * dv).bfloat16()
    pos = torch.arange(T)
    q_raw, k_raw, v_raw = row.double().split([H * d, G * d, G * dv], 1)
    k_want = plain.rms(k_raw.reshape(T, G, d), eps)
    pk, pv = -(-d // 16) * 16, -(-dv // 16) * 16
    kp = torch.zeros(6, page, G * pk, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(6, page, G * pv, dtype=torch.bfloat16, device=DEV)
    table = torch.zeros(2, 5, dtype=torch.int32)
    table[1] = torch.tensor([3, 0, 4, 1, 5])
    slot = i32([1] * T)
    q_out = torch.empty(T, H * d, dtype=torch.bfloat16, device=DEV)
    ops.qkv_norm_rotate_store(dev(row), q_out, H, G, d, dv, 0, i32(pos.tolist()), slot, None, 1.0, kp, vp, dev(table), page,
                              eps=eps, norm_after=True)
    qq = torch.randn(T, H, d).bfloat16()
    wide = (torch.randn(T, H * dv + 9) * 2).bfloat16()                   # the gate's rows lie at column 4 of wider rows
    gate = dev(wide)[:, 4:4 + H * dv]
    want = plain.softmax_attention(qq.double(), k_want.repeat_interleave(H // G, 1),
                                   v_raw.reshape(T, G, dv).repeat_interleave(H // G, 1), 0.4, plain.visible(T, 90))
    want = want.reshape(T, H * dv) * torch.sigmoid(wide[:, 4:4 + H * dv].double())
    q = dev(qq.reshape(T, H * d))
    cases = [(0, T, 1, False), (T - 1, T, 1, False), (T - 1, T, 3, False), (150, 151, 2, False)]
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
        ops.attention_general_mfma(q[a:b], out, H, G, d, dv, 0.4, kp, vp, dev(table), page, i32(pos[a:b].tolist()), slot[a:b],
                                   0, splits, po, pm, tiles, tpt, window=90, gate=gate[a:b])
        close(out, want[a:b], "bfloat16", what=f"rows {a}..{b} splits {splits} tiled {tiled}")


# ---------------------------------------------------------------------------
# attention with two score maps a head

def _diff_plain(q, k, v, scale, lam, eps, post, temp, q_dtype=None):
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, dv]: the combined, normed heads [T, H*dv].  With q_dtype the
    tempered queries are rounded to it, as the kernel stores them: where the temperature makes the softmax sharp,
    that rounding alone moves the weights by more than every later step together."""
    T, H = q.shape[:2]
    rep = H // k.shape[1]
    q = q.double() * temp[:, None, None, None]
    if q_dtype is not None:
        q = q.to(q_dtype).double()
    k, v = k.double().repeat_interleave(rep, 1), v.double().repeat_interleave(rep, 1)
    mask = plain.visible(T)
    a1 = plain.softmax_attention(q[:, :, 0], k[:, :, 0], v, scale, mask)
    a2 = plain.softmax_attention(q[:, :, 1], k[:, :, 1], v, scale, mask)
    o = a1 - lam * a2
    size = lambda x: torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    # how much the division by the difference's size enlarges the rounding of its two terms (1: nothing cancels)
    amp = ((size(a1) + abs(lam) * size(a2)) / size(o)).expand_as(o).reshape(T, -1)
    return (plain.rms(o, eps) * post).reshape(T, -1), amp


def close_diff(got, want, amp, dtype, what=""):
    """float32: the plain tolerance.  bfloat16: where a head's two maps nearly cancel, the difference is small
    against its terms and the division by its root mean square enlarges their rounding by `amp`; the tolerance of
    an element grows with it."""
    if dtype == "float32":
        return close(got, want, dtype, what=what)
    err = (got.detach().cpu().to(F64) - want).abs()
    tol = 1.5e-2 * float(want.abs().max()) * torch.clamp(amp, min=1.0)
    bad = (err > tol).nonzero()
    assert bad.numel() == 0, f"{what}: {bad.shape[0]} elements, first {bad[0].tolist()}: {float(err[tuple(bad[0])]):.3g} > {float(tol[tuple(bad[0])]):.3g}"


def _temperature(T, coef, every):
    if not every:
        return torch.ones(T, dtype=F64)
    p = torch.arange(T, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def _diff_pools(T, G, d, dv, page, dtype, pages):
    pk, pv = -(-d // 16) * 16, -(-dv // 16) * 16
    kp = torch.zeros(max(pages) + 1, page, 2 * G * pk, dtype=dtype, device=DEV)
    vp = torch.zeros(max(pages) + 1, page, G * pv, dtype=dtype, device=DEV)
    table = torch.zeros(2, len(pages), dtype=torch.int32)
    table[1] = torch.tensor(pages, dtype=torch.int32)
    return kp, vp, dev(table)


def _diff_run(ops, src, H, G, d, dv, scale, lam, eps, post, coef, every, page, pages, dtype, mfma_checks=None):
    """Store, attend (plain kernel; and the matrix-core kernel over the given ranges) and combine."""
    T = src.shape[0]
    kp, vp, table = _diff_pools(T, G, d, dv, page, DT[dtype], pages)
    pos, slot = i32(range(T)), i32([1] * T)
    q = torch.empty(T, 2 * H * d, dtype=DT[dtype], device=DEV)
    ops.diff_qkv_store(dev(src), q, H, G, d, dv, coef, every, pos, slot, kp, vp, table, page)
    maps = torch.empty(T, 2 * H * dv, dtype=DT[dtype], device=DEV)
    ops.attention_general(q, maps, 2 * H, 2 * G, d, dv, scale, kp, vp, table, page, pos, slot, 0, 0, 0, None, 2)
    out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
    ops.diff_combine(maps, out, H, G, dv, lam, eps, post)
    outs = [(0, T, out)]
    for i, (a, b, splits, tiled) in enumerate(mfma_checks or []):
        # the maps leave the matrix-core kernel (and the merge of split keys) as float, as the mixer asks, or as bf16
        m2 = torch.empty(b - a, 2 * H * dv, dtype=torch.float32 if i != 1 else torch.bfloat16, device=DEV)
        po = torch.empty(b - a, 2 * H, splits, dv, device=DEV) if splits > 1 else None
        pm = torch.empty(b - a, 2 * H, splits, 2, device=DEV) if splits > 1 else None
        tiles, tpt = None, 1
        if tiled:
            tpt = ops.attention_general_tokens_per_tile(b - a, 2 * H, 2 * G, vp.shape[2] // G)
            assert tpt > 1
            tiles = ops.prefill_tiles([b - a], tpt, DEV)
        ops.attention_general_mfma(q[a:b], m2, 2 * H, 2 * G, d, dv, scale, kp, vp, table, page, pos[a:b], slot[a:b], 0, splits,
                                   po, pm, tiles, tpt, v_share=2)
        o2 = torch.empty(b - a, H * dv, dtype=torch.bfloat16, device=DEV)
        ops.diff_combine(m2, o2, H, G, dv, lam, eps, post)
        outs.append((a, b, o2))
    return outs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(2, 1, 16, 24, 0.3, 7), (3, 3, 40, 16, 0.7, 1), (5, 5, 24, 12, 0.2, 0), (4, 2, 8, 8, 0.9, 3),
                                   (4, 1, 16, 32, 0.5, 3), (8, 2, 64, 256, 0.4, 50), (2, 2, 32, 144, 0.6, 11)])
def test_two_score_maps_over_shared_values(dtype, shape):
    """q and k rows lie head by head as [map 1 | map 2]; both maps read one value head.  Prompts of 330 tokens (in
    the matrix-core kernel: a token a tile and, where a key head serves few query heads, several tokens a tile,
    also with values wider than one wavefront holds) and single tokens whose keys are shared out and merged."""
    from cpmcu_amd import ops
    H, G, d, dv, diff, every = shape
    torch.manual_seed(35)
    T, page, eps, coef, scale = 330, 64, 1e-5, 0.5, 0.3
    lam = math.exp(0.11) - math.exp(-0.2) + diff
    src = torch.randn(T, 2 * H * d + 2 * G * d + G * dv).to(DT[dtype]).float()    # numbers that the type holds exactly
    q, k, v = src.split([2 * H * d, 2 * G * d, G * dv], 1)
    want, amp = _diff_plain(q.reshape(T, H, 2, d), k.reshape(T, G, 2, d), v.reshape(T, G, dv), scale, lam, eps, 1.0 - diff,
                            _temperature(T, coef, every), DT[dtype] if dtype == "bfloat16" else None)
    checks = None
    if dtype == "bfloat16" and d % 8 == 0:
        checks = [(0, T, 1, False), (T - 40, T, 1, False), (T - 1, T, 5, False), (200, 201, 2, False), (T - 3, T, 1, False)]
        if H // G <= 8:
            checks.append((0, T, 1, True))
    for a, b, out in _diff_run(ops, src, H, G, d, dv, scale, lam, eps, 1.0 - diff, coef, every, page, [5, 2, 7, 0, 3, 6], dtype, checks):
        close_diff(out, want[a:b], amp[a:b], dtype, what=f"rows {a}..{b}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_that_one_map_alone_sees(dtype):
    """Among hundreds of keys one, far back, is made to dominate the first map of every later query; the second
    map stays spread.  The head's output is then a1 - lam * a2 with a1 the far key's value: whoever loses that key
    (a page border, a share of the keys, a tile's edge) loses the result.  Keys at page borders, at the sequence's
    first positions and directly before the query."""
    from cpmcu_amd import ops
    H, G, d, dv, page = 4, 2, 32, 48, 64
    T, eps, lam, post = 700, 1e-5, 0.8, 0.6
    torch.manual_seed(36)
    for star in (0, 1, 63, 64, 65, 127, 128, 511, 698):
        q = torch.randn(T, H, 2, d) * 0.2
        k = torch.randn(T, G, 2, d) * 0.2
        q[:, :, 0, 0] = 5.0
        k[star, :, 0, 0] = 5.0
        v = torch.randn(T, G, dv)
        v[star] = 3.0 * torch.sign(torch.randn(G, dv))
        src = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1)
        want, amp = _diff_plain(q, k, v, 1.0, lam, eps, post, _temperature(T, 0.0, 0))
        # the oracle itself depends on the far key: without it the rows after it change by far more than the tolerance
        k0 = k.clone()
        k0[star, :, 0, 0] = 0.0
        moved = (_diff_plain(q, k0, v, 1.0, lam, eps, post, _temperature(T, 0.0, 0))[0] - want)[star + 1:].abs().amax(1)
        assert float(moved.min()) > 0.2
        checks = None
        if dtype == "bfloat16":
            late = [(t, t + 1, s, False) for t, s in ((T - 1, 1), (T - 1, 4), (T - 1, 11), (max(star, 1), 1), (min(star + 1, T - 1), 3),
                                                      (min(star + 64, T - 1), 2))]
            checks = [(0, T, 1, False), (0, T, 1, True)] + late
        for a, b, out in _diff_run(ops, src, H, G, d, dv, 1.0, lam, eps, post, 0.0, 0, page, list(range(11, 0, -1)), dtype, checks):
            close_diff(out, want[a:b], amp[a:b], dtype, what=f"star {star} rows {a}..{b}")


# ---------------------------------------------------------------------------
# the gated delta rule

def _delta_plain(qkv, a, b, A_log, dt_bias, H, G, d, dv):
    T = qkv.shape[0]
    q, k, v = qkv.double().split([G * d, G * d, H * dv], 1)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k, v = unit(q.reshape(T, G, d)) * d ** -0.5, unit(k.reshape(T, G, d)), v.reshape(T, H, dv)
    beta = torch.sigmoid(b.double())
    g = torch.exp(-torch.exp(A_log.double()) * plain.softplus(a.double() + dt_bias.double()))
    rep = H // G
    return torch.stack([plain.delta_rule(q[:, i // rep], k[:, i // rep], v[:, i], beta[:, i], g[:, i]) for i in range(H)], 1).reshape(T, H * dv)


@pytest.mark.parametrize("lanes", [0, 8, 16])
@pytest.mark.parametrize("gates_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 24, 20), (1, 1, 72, 8), (2, 1, 12, 7), (3, 3, 8, 36), (4, 1, 32, 40), (4, 2, 128, 128),
                                   (2, 2, 256, 16), (2, 1, 200, 50)])
def test_delta_rule_in_portions_and_slots(gates_dtype, shape, lanes):
    """Two sequences in slots 3 and 1, in portions of unequal sizes down to one token: the state is carried in the
    slot; a slot that is freed (its state cleared) and used again starts from nothing; a pass that does not write
    leaves the state as it was.  Decays from nearly 1 to nearly 0, steps from nearly 0 to nearly 1.  A column of
    the state over 8 and over 16 lanes, and as the kernel chooses by the batch."""
    from cpmcu_amd import ops
    H, G, d, dv = shape
    torch.manual_seed(37)
    lens = {3: 41, 1: 12}
    C = 2 * G * d + H * dv
    A_log = torch.linspace(-4.0, 1.5, H)
    dt_bias = torch.randn(H)
    data, want = {}, {}
    for s, L in lens.items():
        qkv = torch.randn(L, C)
        gates = (torch.randn(L, 3 + 2 * H) * 2).to(DT[gates_dtype])      # wider rows: the columns lie at offsets
        data[s] = (qkv, gates)
        want[s] = _delta_plain(qkv, gates[:, 3:3 + H], gates[:, 3 + H:], A_log, dt_bias, H, G, d, dv)
    state = torch.zeros(4, H, dv, d, device=DEV)
    state[0] = 5.0
    cuts = {3: [0, 1, 2, 9, 40, 41], 1: [0, 5, 12]}
    got = {s: [] for s in lens}

    def run(batch, write=True):
        cu = [0]
        for s, a, b in batch:
            cu.append(cu[-1] + b - a)
        qkv = dev(torch.cat([data[s][0][a:b] for s, a, b in batch]))
        gates = dev(torch.cat([data[s][1][a:b] for s, a, b in batch]))
        y = torch.empty(cu[-1], H * dv, device=DEV)
        ops.delta_scan(qkv, gates, 3, 3 + H, dev(dt_bias), dev(A_log), state, y, i32(cu), i32([s for s, _, _ in batch]),
                       H, G, d, dv, d ** -0.5, write_state=write, lanes=lanes)
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


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
def test_head_norm_with_a_silu_gate_behind_it(out_dtype):
    from cpmcu_amd import ops
    torch.manual_seed(38)
    for n, H, dv in ((9, 4, 20), (1, 1, 8), (70, 3, 36), (8, 32, 128)):
        y = torch.randn(n, H * dv) * 3
        proj = torch.randn(n, H * dv + 5).to(DT[out_dtype])              # the gate is a column slice of a wider row
        w = torch.rand(dv) + 0.5
        want = (plain.rms(y.double().reshape(n, H, dv), 1e-5) * w.double()).reshape(n, H * dv) * plain.silu(proj[:, 2:2 + H * dv].double())
        out = torch.empty(n, H * dv, dtype=DT[out_dtype], device=DEV)
        ops.rms_norm_groups(dev(y), dev(w.repeat(H)), 1e-5, out, groups=H, gate=dev(proj)[:, 2:2 + H * dv], gate_after="silu")
        close(out, want, out_dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gates_cap_activation_and_embedding(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(39)
    n, W = 13, 84
    a = torch.randn(n, W).to(DT[dtype])
    g = (torch.randn(n, W + 4) * 3).to(DT[dtype])
    out = torch.empty(n, W, dtype=DT[dtype], device=DEV)
    ops.sigmoid_gate(dev(a), dev(g)[:, 4:], out)
    close(out, a.double() * torch.sigmoid(g[:, 4:].double()), dtype)
    gu = (torch.randn(n, 2 * W) * 2).to(DT[dtype])
    out = torch.empty(n, W, dtype=DT[dtype], device=DEV)
    ops.silu_mul(dev(gu), out, "gelu_tanh")
    close(out, plain.gelu_tanh(gu[:, :W].double()) * gu[:, W:].double(), dtype)
    lg = torch.randn(5, 301) * 20
    ld = dev(lg.clone())
    ops.softcap(ld, 12.0)
    close(ld, 12.0 * torch.tanh(lg.double() / 12.0), "float32")
    table = torch.randn(50, 36).to(DT[dtype])
    ids = [3, 49, 0, 3]
    out = torch.empty(4, 36, device=DEV)
    ops.embed(dev(table), i32(ids), out, 3.5)
    close(out, table[ids].double() * 3.5, "float32")
