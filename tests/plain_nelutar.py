"""Plain implementation of the Nelutar design: whole sequences, no cache, float64, one function per mechanism.

It reads the raw config.json dictionary and the checkpoint's tensors by name and shares no code with the
package: every formula is restated here.  Positions count from 0; "rms" always has eps inside the root.

    embedding       x_t = embed[tok_t] + bigram[(tok_{t-1} * mul_prev + tok_t * mul_cur) mod buckets]; the first
                    token of a sequence reads row `buckets` (the table's last row) instead
    layer           h = rms(x) * w;  x += ls1 * mixer(h) + ls2 * ff(h)   (one norm, both read it; a layer may have
                    no feed-forward); a layer with `weights_of`: j reads layer j's tensors
    rotation        first `dims` features of a head; pairs (2i, 2i+1) ("interleaved") or (i, i + dims/2)
                    ("halves"): (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = p f_i, f_i = base^(-2i/dims)
    window          query p sees key j with 0 <= p - j < size; softmax over those
    parallel        left: q, k, v = W h; q, k rotated (interleaved); score = q.k * scale; window; Wo.
                    right: the gated delta rule with a decay per key channel: q, k, v through a causal convolution
                    per channel and silu; q, k / sqrt(sum squares + 1e-6) per head, q / sqrt(dim); beta =
                    sigmoid(Wb h); g = exp(-exp(A_log_h) softplus(Wa2 Wa1 h + dt_bias)) [heads, dim];
                    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
                    o / rms(o) per head * w * sigmoid(Wg2 Wg1 h); Wo.
                    result (rms(left) * w_left + rms(right) * w_right) / 2 over the model width
    retention       q, k rotated (halves), k / sqrt(dim); S <- decay_h S + k v^T; o = S^T q; o / rms(o) per head
                    (no weight); heads side by side * silu(Wg h); Wo
    parallel_2      left: q, k, v = W h, each through a causal convolution (no activation), q, k rotated
                    (interleaved), then divided by their rms per head; score = cap tanh(q.k * scale / cap);
                    window; Wo.  right: q, k, v = silu(W h); S <- decay_h S + k v^T; o = S^T q; all heads
                    together rms * w * sigmoid(Wg h); Wo.  result left_scale left + right_scale right
    feed-forward    dense: Wd (silu(Wg h) * (Wu h)).  experts: g = min(Wg h, limit), u = clamp(Wu h, +-limit),
                    Wd (g sigmoid(1.702 g) (u + 1)).  router: s = sigmoid(Wr h); choice c = s + correction;
                    groups of neighbours scored by the sum of their two largest c, the best `keep` groups stay,
                    the others' c = -inf; the `top` largest c are chosen; weights s / (sum of chosen s + 1e-20)
                    * scale; plus the shared expert (same form, limit of its own) for every token
    output          logits = head . (rms(x) * w_final)
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def embed(tokens, W, big):
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"][tok].clone()
    if big is not None:
        buckets = int(big["buckets"])
        rows = torch.full_like(tok, buckets)
        rows[1:] = (tok[:-1] * int(big["mul_prev"]) + tok[1:] * int(big["mul_cur"])) % buckets
        x = x + W["bigram"][rows]
    return x


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y


def rotate(x, rot, pairing):
    """x [T, heads, dim]."""
    if not rot or not rot.get("dims"):
        return x
    dims, T = int(rot["dims"]), x.shape[0]
    i = torch.arange(dims // 2, dtype=F64)
    ang = torch.arange(T, dtype=F64)[:, None] * float(rot["base"]) ** (-2.0 * i / dims)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if pairing == "interleaved":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * c - b * s
        out[..., dims // 2:dims] = b * c + a * s
    return out


def window_softmax_attention(q, k, v, scale, size, cap=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H * dv]."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    idx = torch.arange(T)
    dist = idx[:, None] - idx[None, :]
    mask = (dist >= 0) & ((dist < size) if size else True)
    outs = []
    for h in range(H):
        g = h // (H // G)
        sc = q[:, h] @ k[:, g].T * scale
        if cap:
            sc = cap * torch.tanh(sc / cap)
        sc = sc.masked_fill(~mask, -math.inf)
        outs.append(torch.softmax(sc, -1) @ v[:, g])
    return torch.cat(outs, -1)


def attention_side(h, W, p, m, eps, normed):
    T, H, G, d, dv = h.shape[0], int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if m.get("conv"):
        q, k, v = (causal_conv(t, W[p + n + ".conv"]) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    q = rotate(q.view(T, H, d), m.get("rot"), "interleaved")
    k = rotate(k.view(T, G, d), m.get("rot"), "interleaved")
    if normed:
        q, k = rms(q, eps), rms(k, eps)
    size = int(m["mask"]["size"]) if m.get("mask") else None
    o = window_softmax_attention(q, k, v.view(T, G, dv), float(m["scale"]), size, m.get("softcap"))
    return o @ W[p + "o"].T


def decay_recurrence(q, k, v, decay):
    """One head: S <- decay S + k v^T; o = S^T q.  q, k [T, d], v [T, dv]."""
    S = torch.zeros(q.shape[1], v.shape[1], dtype=F64)
    out = []
    for t in range(q.shape[0]):
        S = decay * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta_recurrence(q, k, v, beta, g):
    """One head: g [T, d] a decay per key channel."""
    S = torch.zeros(q.shape[1], v.shape[1], dtype=F64)
    out = []
    for t in range(q.shape[0]):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def channel_delta(h, W, p, m, eps):
    T, H, G, d, dv = h.shape[0], int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = (silu(causal_conv(h @ W[p + n].T, W[p + n + ".conv"])) for n in ("q", "k", "v"))
    q, k, v = q.view(T, G, d), k.view(T, G, d), v.view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    a = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]
    g = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * softplus(a).view(T, H, d))
    gate = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).view(T, H, dv)
    outs = []
    for i in range(H):
        j = i // (H // G)
        o = delta_recurrence(q[:, j], k[:, j], v[:, i], beta[:, i], g[:, i])
        outs.append(rms(o, eps) * W[p + "norm"] * gate[:, i])
    return torch.cat(outs, -1) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    a = attention_side(h, W, p + "left.", m["left"], eps, normed=False)
    b = channel_delta(h, W, p + "right.", m["right"], eps)
    return 0.5 * (rms(a, eps) * W[p + "left.out"] + rms(b, eps) * W[p + "right.out"])


def retention(h, W, p, m, eps):
    T, H, d, dv = h.shape[0], int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = rotate((h @ W[p + "q"].T).view(T, H, d), m.get("rot"), "halves")
    k = rotate((h @ W[p + "k"].T).view(T, H, d), m.get("rot"), "halves") * d ** -0.5
    v = (h @ W[p + "v"].T).view(T, H, dv)
    outs = [rms(decay_recurrence(q[:, i], k[:, i], v[:, i], float(m["decay"][i])), eps) for i in range(H)]
    return (torch.cat(outs, -1) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def lightning_side(h, W, p, m, eps):
    T, H, d, dv = h.shape[0], int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = silu(h @ W[p + "q"].T).view(T, H, d), silu(h @ W[p + "k"].T).view(T, H, d), silu(h @ W[p + "v"].T).view(T, H, dv)
    o = torch.cat([decay_recurrence(q[:, i], k[:, i], v[:, i], float(m["decay"][i])) for i in range(H)], -1)
    return (rms(o, eps) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel_2_mixer(h, W, p, m, eps):
    a = attention_side(h, W, p + "left.", m["left"], eps, normed=True)
    b = lightning_side(h, W, p + "right.", m["right"], eps)
    return float(m["left_scale"]) * a + float(m["right_scale"]) * b


def expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def route(h, W, p, r, margins=None):
    """(chosen experts [T, top], weights [T, top]).  ``margins`` (a list) receives, per token, how clear the choice
    was: the smallest gap between what was taken and what was left, among the groups and among the experts."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ W[p + "router"].T)
    c = s + W[p + "correction"] if (p + "correction") in W else s.clone()
    clear = torch.full((h.shape[0],), math.inf, dtype=F64)
    groups = r.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = c.view(-1, count, E // count)
        score = per.topk(min(2, E // count), -1).values.sum(-1)
        kept = torch.zeros_like(score, dtype=torch.bool)
        kept.scatter_(1, score.topk(keep, -1).indices, True)
        if keep < count:
            ranked = score.sort(-1, descending=True).values
            clear = torch.minimum(clear, ranked[:, keep - 1] - ranked[:, keep])
        c = per.masked_fill(~kept[:, :, None], -math.inf).reshape(-1, E)
    idx = c.topk(top, -1).indices
    if top < E:
        ranked = c.sort(-1, descending=True).values
        gap = ranked[:, top - 1] - ranked[:, top]
        clear = torch.minimum(clear, torch.where(torch.isfinite(gap), gap, torch.full_like(gap, math.inf)))
    if margins is not None:
        margins.append(clear)
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))


def feed_forward(h, W, p, mlp, margins=None):
    if mlp["kind"] == "dense":
        return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T
    idx, w = route(h, W, p, mlp["router"], margins)
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), w[t]):
            out[t] += a * expert(h[t:t + 1], W, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        out = out + expert(h, W, p + "shared.", float(mlp["shared"]["limit"]))
    return out


MIXERS = {"parallel": parallel_mixer, "retention": retention, "parallel_2": parallel_2_mixer}


def forward(raw, tensors, tokens, return_layers=False, margins=None):
    """Logits [T, vocab] of one sequence (and the residual after every layer run).  ``margins`` (a list) receives one
    tensor [T] for every routed layer run: how clear each token's choice of experts was (route)."""
    W = {k: v.to(F64) for k, v in tensors.items()}
    eps = float(raw["norm"]["eps"])
    x = embed(tokens, W, (raw.get("embedding") or {}).get("bigram"))
    after = []
    for i, layer in enumerate(raw["layers"]):
        p = f"l{layer['weights_of'] if layer.get('weights_of') is not None else i}."
        h = rms(x, eps) * W[p + "norm1"]
        y = W[p + "ls1"] * MIXERS[layer["type"]](h, W, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            y = y + W[p + "ls2"] * feed_forward(h, W, p + "mlp.", layer["mlp"], margins)
        x = x + y
        after.append(x)
    logits = (rms(x, eps) * W["final.norm"]) @ W["head"].T
    return (logits, torch.stack(after)) if return_layers else logits
