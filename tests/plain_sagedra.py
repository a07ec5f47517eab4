"""Plain implementation of the Sagedra design: whole sequences, no cache, float64, one function per mechanism.

It reads the raw config.json dictionary and the checkpoint's tensors by name and shares no code with the
package: every formula is restated here.  Positions count from 0; "rms" always has eps inside the root.

    norm            layer norm without bias: (x - mean) / sqrt(mean((x - mean)^2) + eps) * w
    layer           x += mixer(norm1(x)); x += ff(norm2(x))  (a layer may have no feed-forward)
    streams         with `streams` = s the residual is s rows X_1..X_s, all equal to the embedding at the start.
                    A sub-layer with numbers in[s], out[s], mix[s, s]:  u = sum_s in[s] X_s;  y = sub(norm(u));
                    X_t' = sum_s mix[s, t] X_s + out[t] y  (all t at once from the old rows); the model's
                    output norm reads sum_t X_t
    loop            layers start..stop-1 run `times` times in a row (same weights, separate state), then the rest
    rotation        first `dims` features of a head, feature i with i + dims/2:
                    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = p * f_i, f_i = base^(-2i/dims); with
                    `scaling` {factor, low, high, original}: wavelength l = 2 pi / f; f stays where
                    l < original/high, becomes f/factor where l > original/low, and in between
                    (1 - t) f/factor + t f with t = (original/l - low) / (high - low)
    window          q, k, v = W h; q, k rotated, then divided by their rms per head; score = q.k * scale;
    attention       query p sees key j with 0 <= p - j < size; softmax; heads * sigmoid(Wg h); Wo
    delta rule      q, k, v = W h, each through a causal convolution per channel (taps weights, the last one
                    the current token's, zeros before the start) and silu; q, k / sqrt(sum squares + 1e-6) per
                    head, q / sqrt(dim); beta = sigmoid(Wb h); g = exp(-exp(A_log) softplus(Wa h + dt_bias));
                    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
                    o / rms(o) per head * w * silu(Wg h); Wo
    parallel        (rms(left) * w_left + rms(right) * w_right) / 2 over the model width
    differential    q, k rows lie head by head as [map 1 | map 2]; q, k, v = W h + b, then a causal convolution
    attention       per channel; q * (1 + coef ln(floor((p + 1)/every) + 1)); two causal softmax attentions over
                    the same values, a1 and a2; lam = exp(lq1.lk1) - exp(lq2.lk2) + diff;
                    o = rms(a1 - lam a2) (no weight) * (1 - diff); Wo (.) + bo
    feed-forward    Wd (gelu_tanh(Wg h) * (Wu h))
    output          logits = head . norm(x); with a cap c: c tanh(logits / c)
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    return y


def frequencies(rot):
    dims = rot["dims"]
    i = torch.arange(dims // 2, dtype=F64)
    f = float(rot["base"]) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc is None:
        return f
    factor, low, high, original = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = []
    for fi in f.tolist():
        wave = 2.0 * math.pi / fi
        if wave < original / high:
            out.append(fi)
        elif wave > original / low:
            out.append(fi / factor)
        else:
            t = (original / wave - low) / (high - low)
            out.append((1.0 - t) * fi / factor + t * fi)
    return torch.tensor(out, dtype=F64)


def rotate(x, positions, rot):
    """x [T, heads, d]: the first rot.dims features rotated by position, the others unchanged."""
    if rot is None or rot["dims"] == 0:
        return x
    dims = rot["dims"]
    a = positions.to(F64)[:, None] * frequencies(rot)[None, :]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def visible(T, size=None):
    p = torch.arange(T)
    m = p[:, None] >= p[None, :]
    if size is not None:
        m = m & ((p[:, None] - p[None, :]) < size)
    return m


def softmax_attention(q, k, v, scale, mask):
    """q [T, H, d], k [T, H, d], v [T, H, dv] (already one key/value head a query head) -> [T, H, dv]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    p = torch.softmax(s.masked_fill(~mask, -math.inf), -1)
    return torch.einsum("hij,jhd->ihd", p, v)


def window_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rms(rotate((h @ W[p + "q"].T).view(T, H, d), pos, m.get("rot")), eps)
    k = rms(rotate((h @ W[p + "k"].T).view(T, G, d), pos, m.get("rot")), eps)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    rep = H // G
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    size = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(q, k, v, m["scale"], visible(T, size)).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def delta_rule(q, k, v, beta, g):
    """One head: q, k [T, d], v [T, dv], beta, g [T].  S [d, dv] starts at zero."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def gated_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    branch = lambda n: silu(causal_conv(h @ W[p + n].T, W[p + n + ".conv"]))
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q = unit(branch("q").view(T, G, d)) * d ** -0.5
    k = unit(branch("k").view(T, G, d))
    v = branch("v").view(T, H, dv)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    rep = H // G
    o = torch.stack([delta_rule(q[:, i // rep], k[:, i // rep], v[:, i], beta[:, i], g[:, i]) for i in range(H)], 1)
    o = rms(o, eps) * W[p + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    left = window_attention(h, W, p + "left.", m["left"], eps)
    right = gated_delta(h, W, p + "right.", m["right"], eps)
    return 0.5 * (rms(left, eps) * W[p + "left.out"] + rms(right, eps) * W[p + "right.out"])


def differential_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    diff = float(m["diff"])

    def branch(n):
        u = h @ W[p + n].T + W[p + n + ".b"]
        return causal_conv(u, W[p + n + ".conv"]) if m.get("conv") else u
    q = branch("q").view(T, H, 2, d)
    k = branch("k").view(T, G, 2, d)
    v = branch("v").view(T, G, dv)
    if m.get("q_temp"):
        pos = torch.arange(T, dtype=F64)
        temp = 1.0 + m["q_temp"]["coef"] * torch.log(torch.floor((pos + 1) / m["q_temp"]["every"]) + 1.0)
        q = q * temp[:, None, None, None]
    rep = H // G
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    mask = visible(T)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, m["scale"], mask)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, m["scale"], mask)
    lam = torch.exp((W[p + "lq1"] * W[p + "lk1"]).sum()) - torch.exp((W[p + "lq2"] * W[p + "lk2"]).sum()) + diff
    o = rms(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * dv) @ W[p + "o"].T + W[p + "o.b"]


def feed_forward(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


MIXERS = {"parallel": parallel_mixer, "attention": differential_attention}


def layer_order(raw):
    n = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(raw, tensors, tokens, return_layers=False):
    """float64 logits [T, vocab] of the whole sequence (and the residual stream after every layer run, the sum of
    the streams where there are several)."""
    W = {k: v.to(F64) for k, v in tensors.items()}
    eps = float(raw["norm"]["eps"])
    emb = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((raw.get("embedding") or {}).get("scale", 1.0))
    s = raw.get("streams")
    X = emb.unsqueeze(0).repeat(s, 1, 1) if s else emb
    after = []

    def sub(X, q, norm_w, fn):
        if not s:
            return X + fn(layer_norm(X, norm_w, eps))
        u = torch.einsum("s,std->td", W[q + ".in"], X)
        y = fn(layer_norm(u, norm_w, eps))
        return torch.einsum("st,snd->tnd", W[q + ".mix"], X) + W[q + ".out"][:, None, None] * y[None]

    for i in layer_order(raw):
        layer, p = raw["layers"][i], f"l{i}."
        X = sub(X, p + "hc1", W[p + "norm1"],
                lambda h: MIXERS[layer["type"]](h, W, p + "mix.", layer["mixer"], eps))
        if layer.get("mlp") is not None:
            X = sub(X, p + "hc2", W[p + "norm2"], lambda h: feed_forward(h, W, p + "mlp."))
        after.append(X.sum(0) if s else X)
    x = X.sum(0) if s else X
    logits = layer_norm(x, W["final.norm"], eps) @ W["head"].T
    cap = raw.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return (logits, after) if return_layers else logits
