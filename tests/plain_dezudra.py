"""The Dezudra design, plainly: float64 on the CPU, whole sequences, no cache, one function per mechanism.

Nothing here is shared with the engine.  `forward(cfg, weights, tokens)` takes the configuration as the dict that
config.json holds and the tensors by their checkpoint names, and returns the logits of every position (and, if
asked, the residual stream after every layer).

    layer      x += norm1b(mixer(norm1(x)));  x += norm2b(ff(norm2(x)))            (four RMS norms a layer)
    delta      q, k, v <- silu(conv(W h));  q, k unit vectors per head, q / sqrt(dim);
               S <- g S;  S += k (beta (v - S^T k))^T;  o = S^T q;  rms(o) * w * silu(W_g h);  W_o
    attention  two score maps per head over one set of values, window with kept first tokens,
               o = a1 - lambda a2, rms(o) (1 - diff);  W_o
    ff         experts of relu^2, chosen among the best groups of neighbours, weights = softmax scores as they are
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def silu(x):
    return x / (1.0 + np.exp(-x))


def softplus(x):
    return np.logaddexp(0.0, x)


def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), u], axis=0)
    y = np.zeros_like(u)
    for j in range(taps):
        y += padded[j:j + T] * w[:, j][None, :]
    return y


def rotate(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` elements of every head, element i paired with i + dims/2."""
    if dims <= 0:
        return x
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = positions[:, None].astype(np.float64) * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(T, size, keep_first):
    """[T, T] bool: query i sees key j."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def exact(x):
    return x


def bfloat16(x):
    """x rounded to bfloat16 (nearest even) and back: what storing an activation in 16 bits does to it."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).to(torch.float64).numpy()


def delta_mixer(h, m, W, eps, store=exact):
    """m: the layer's `mixer` dict; W: name -> array for this mixer ('q', 'q.conv', ...).  `store`: what keeping an
    activation between two operations does to it (`exact`, or `bfloat16` for a model of a 16-bit run)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(silu(short_conv(store(h @ W["q"].T), W["q.conv"]))).reshape(T, G, D)
    k = store(silu(short_conv(store(h @ W["k"].T), W["k.conv"]))).reshape(T, G, D)
    v = store(silu(short_conv(store(h @ W["v"].T), W["v.conv"]))).reshape(T, H, V)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-(h @ W["b"].T)))                                   # [T, H]
    g = np.exp(-np.exp(W["A_log"])[None, :] * softplus(h @ W["a"].T + W["dt_bias"][None, :]))
    gate = silu(store(h @ W["g"].T)).reshape(T, H, V)
    o = np.zeros((T, H, V))
    for hd in range(H):
        kv = hd // (H // G)
        S = np.zeros((D, V))
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + np.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    o = store(rms_norm(o, W["norm"], eps) * gate)
    return store(o.reshape(T, H * V) @ W["o"].T)


def diff_attention(h, m, W, eps, store=exact):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv(store(h @ W["q"].T) + W["q.b"], W["q.conv"]).reshape(T, H * 2, D)
    k = short_conv(store(h @ W["k"].T) + W["k.b"], W["k.conv"]).reshape(T, G * 2, D)
    v = store(short_conv(store(h @ W["v"].T) + W["v.b"], W["v.conv"])).reshape(T, G, V)
    pos = np.arange(T)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = store(rotate(q, pos, rot["dims"], rot["base"]))
    k = store(rotate(k, pos, rot["dims"], rot["base"]))
    window = m.get("mask") or {"size": T, "keep_first": 0}  # no mask: every earlier token is seen
    mask = visible(T, window["size"], window.get("keep_first", 0))
    lam = math.exp(float(np.sum(W["lq1"] * W["lk1"]))) - math.exp(float(np.sum(W["lq2"] * W["lk2"]))) + m["diff"]
    o = np.zeros((T, H, V))
    for hd in range(H):
        kv = hd // (H // G)
        a = []
        for mp in range(2):
            s = q[:, 2 * hd + mp] @ k[:, 2 * kv + mp].T * m["scale"]
            s = np.where(mask, s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            p = p / p.sum(axis=1, keepdims=True)
            a.append(p @ v[:, kv])
        o[:, hd] = a[0] - lam * a[1]
    o = store(rms_norm(o, None, eps) * (1.0 - m["diff"]))
    return store(o.reshape(T, H * V) @ W["o"].T)


def route(h, r, w_router, margins=None):
    """Scores, and per token the chosen experts with their weights: ([T, E], [T, top] ids, [T, top] weights).
    `margins`: a list that receives, per token, how far the choice is from another one: the smaller of the relative
    gaps between the last expert taken and the first left out, and between the last group kept and the first
    dropped."""
    z = h @ w_router.T
    z = z - z.max(axis=1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(axis=1, keepdims=True)
    T, E = s.shape
    groups = r.get("groups") or {"count": 1, "keep": 1}
    n, keep = groups["count"], groups["keep"]
    per = E // n
    best = s.reshape(T, n, per).max(axis=2)
    order = np.argsort(-best, axis=1, kind="stable")[:, :keep]
    allowed = np.zeros((T, n), dtype=bool)
    np.put_along_axis(allowed, order, True, axis=1)
    masked = np.where(np.repeat(allowed, per, axis=1), s, -1.0)
    ranked = np.argsort(-masked, axis=1, kind="stable")
    ids = ranked[:, :r["top"]]
    if margins is not None:
        gap = np.full(T, np.inf)
        if r["top"] < keep * per:
            last = np.take_along_axis(masked, ranked[:, r["top"] - 1:r["top"]], axis=1)[:, 0]
            nxt = np.take_along_axis(masked, ranked[:, r["top"]:r["top"] + 1], axis=1)[:, 0]
            gap = (last - nxt) / last
        if keep < n:
            by_group = -np.sort(-best, axis=1)
            gap = np.minimum(gap, (by_group[:, keep - 1] - by_group[:, keep]) / by_group[:, keep - 1])
        margins.append(gap)
    return s, ids, np.take_along_axis(s, ids, axis=1)


def moe(h, mlp, W, margins=None, store=exact, chosen=None, scores_out=None):
    """`chosen` [T, top]: experts to use instead of the router's own choice (their weights are still their scores);
    `scores_out`: a list that receives (scores [T, E], the router's own choice [T, top])."""
    r = mlp["router"]
    s, ids, wts = route(h, r, W["router"], margins)
    if scores_out is not None:
        scores_out.append((s, ids))
    if chosen is not None:
        ids = np.asarray(chosen)
        wts = np.take_along_axis(s, ids, axis=1)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t], wts[t]):
            a = store(np.maximum(W[f"e{e}.up"] @ h[t], 0.0) ** 2)
            out[t] += w * store(W[f"e{e}.down"] @ a)
    return store(out)


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, layers_out=None, margins=None, store=exact, experts=None, scores_out=None):
    """Logits [T, vocab] in float64.  `weights`: name -> float64 array.  `layers_out`: a list that receives the
    residual stream after every layer; `margins`: one that receives every routed layer's margins (see `route`);
    `store=bfloat16`: a model of a 16-bit run, in which every activation kept between two operations is rounded
    (the residual stream, norms' sums, scores, the recurrence and the router stay exact): how far that moves the
    logits is what 16-bit storage alone costs.  `experts`: per routed layer, in order, the experts [T, top] to use
    instead of the router's choice; `scores_out`: receives every routed layer's (scores, own choice)."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"][np.asarray(tokens)]
    routed = 0
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mix = {"delta": delta_mixer, "attention": diff_attention}[layer["type"]]
        y = mix(store(rms_norm(x, weights[p + "norm1"], eps)), layer["mixer"], sub(weights, p + "mix."), eps, store)
        x = x + rms_norm(y, weights[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            y = moe(store(rms_norm(x, weights[p + "norm2"], eps)), layer["mlp"], sub(weights, p + "mlp."), margins, store,
                    None if experts is None else experts[routed], scores_out)
            routed += 1
            x = x + rms_norm(y, weights[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    x = store(rms_norm(x, weights["final.norm"], eps))
    return x @ weights["head"].T * cfg.get("logit_scale", 1.0)
