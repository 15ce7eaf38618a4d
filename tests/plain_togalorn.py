"""Togalorn, plainly: whole sequences, no cache, float64, one function per mechanism.

Shares nothing with the package.  ``weights`` maps tensor names (``embed``, ``loop.in``, ``loop.step``,
``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``) to float64 arrays, ``cfg`` is
the design's config.json as a dictionary.

Notation: ``T`` tokens of one sequence, positions ``0 .. T-1``; matrices are stored ``(out, in)`` and applied as
``x @ W.T``.
"""
from __future__ import annotations

import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def embedding(table, ids, scale):
    return table[np.asarray(ids)] * scale


def rms(x, eps):
    """Each row divided by the root of (its mean square + eps)."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def group_norm(x, weight, eps, groups):
    """The row in ``groups`` equal consecutive parts, each divided by its own root mean square; then the weight."""
    T, W = x.shape
    parts = x.reshape(T, groups, W // groups)
    return rms(parts, eps).reshape(T, W) * weight


def causal_conv(x, taps, bias=None):
    """``y_t = sum_j taps[:, j] * x_(t - K + 1 + j)`` per channel (the last column meets the current token), zeros
    before the sequence's start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), x], 0)
    y = np.zeros((T, C))
    for j in range(K):
        y += padded[j:j + T] * taps[:, j]
    return y if bias is None else y + bias


def rotate_interleaved(x, positions, base, dims):
    """Pairs ``(2i, 2i + 1)`` of the first ``dims`` features of the last axis turned by ``p * base^(-2i/dims)``."""
    out = np.array(x, dtype=np.float64, copy=True)
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(a).reshape(shape), np.sin(a).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, w, p, m, eps):
    """``w``: the mixer's tensors by their short names (``dq``, ``dq.norm``, ``uq``, ``dkv``, ``dkv.norm``, ``uk``,
    ``uv``, ``g``, ``o``); ``m``: its sizes; ``p``: positions."""
    T = h.shape[0]
    H, n, r, dv, c = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, n + r)
    down = h @ w["dkv"].T
    lat = rms(down[:, :c], eps) * w["dkv.norm"]
    k_rot = rotate_interleaved(down[:, c:], p, base, dims)                  # (T, r), one for all heads
    q_plain, q_rot = q[..., :n], rotate_interleaved(q[..., n:], p, base, dims)
    k_plain = (lat @ w["uk"].T).reshape(T, H, n)
    v = (lat @ w["uv"].T).reshape(T, H, dv)
    scores = (np.einsum("ihd,jhd->hij", q_plain, k_plain) + np.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    seen = np.tril(np.ones((T, T), dtype=bool))
    scores = np.where(seen[None], scores, -np.inf)
    scores = scores - scores.max(-1, keepdims=True)
    pr = np.exp(scores)
    pr = pr / pr.sum(-1, keepdims=True)
    mixed = np.einsum("hij,jhd->ihd", pr, v).reshape(T, H * dv)
    return (mixed * sigmoid(h @ w["g"].T)) @ w["o"].T


def state_space(x, B, C, dt, a_log, d_skip, heads_per_group):
    """Per head ``S_t = exp(-exp(a_log) dt_t) S_(t-1) + dt_t B_t x_t^T`` (state x vdim), ``y_t = S_t^T C_t + D x_t``.
    ``x (T, H, P)``, ``B, C (T, G, N)``, ``dt (T, H)``."""
    T, H, P = x.shape
    N = B.shape[2]
    y = np.zeros((T, H, P))
    for hd in range(H):
        g = hd // heads_per_group
        S = np.zeros((N, P))
        rate = math.exp(a_log[hd])
        for t in range(T):
            S = math.exp(-rate * dt[t, hd]) * S + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + d_skip[hd] * x[t, hd]
    return y


def mamba2(h, w, m, eps):
    """``w``: ``in``, ``conv``, ``conv.b``, ``dt_bias``, ``A_log``, ``D``, ``norm``, ``o``."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    rows = h @ w["in"].T
    z, xbc, dt = rows[:, :inner], rows[:, inner:2 * inner + 2 * G * N], rows[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    y = state_space(x, B, C, dt, w["A_log"], w["D"], H // G).reshape(T, inner)
    y = y * silu(z)
    y = group_norm(y, w["norm"], eps, m["norm_groups"])
    return y @ w["o"].T


def expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, router, correction, top):
    """``(chosen (T, top), weights (T, top))``: softmax over all router outputs; the choice looks at scores +
    correction, the weights are the plain scores of the chosen, divided by their sum."""
    z = h @ router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(-1, keepdims=True)
    chosen = np.argsort(-(s + correction), axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, -1)
    return chosen, picked / (picked.sum(-1, keepdims=True) + 1e-20)


def moe(h, w, m):
    """``w``: ``router``, ``correction``, ``e<k>.gate/up/down``, ``shared.gate/up/down``; ``m``: the ``mlp`` entry."""
    E, top = m["router"]["experts"], m["router"]["top"]
    chosen, weights = route(h, w["router"], w["correction"], top)
    y = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            if e >= E:                                   # an identity expert: the input itself
                y[t] += a * h[t]
            else:
                y[t] += a * expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], m["expert"]["limit"])[0]
    if m.get("shared") is not None:
        y = y + expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], m["shared"]["limit"])
    return y


def under(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer(x, weights, i, entry, cfg, positions):
    """``x + mixer(h + conv(h)) + ff(h)`` with ``h`` the group norm of ``x``."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    p = f"l{i}."
    h = group_norm(x, weights[p + "norm1"], eps, groups)
    hm = h + causal_conv(h, weights[p + "canon1"]) if p + "canon1" in weights else h
    if entry["type"] == "latent_attention":
        a = latent_attention(hm, under(weights, p + "mix."), positions, entry["mixer"], eps)
    else:
        a = mamba2(hm, under(weights, p + "mix."), entry["mixer"], eps)
    out = x + a
    if entry.get("mlp") is not None:
        out = out + moe(h, under(weights, p + "mlp."), entry["mlp"])
    return out


def run_order(cfg):
    """``[(layer, pass or None if the layer is outside the loop, first of its pass)]`` in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None, False) for i in range(a)]
    for t in range(times):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def forward(weights, cfg, ids, trace=None):
    """Logits ``(T, vocab)`` of one sequence; ``trace``: a list that receives the stream after every layer run."""
    T = len(ids)
    positions = np.arange(T)
    x0 = embedding(weights["embed"], ids, cfg.get("embedding", {}).get("scale", 1.0))
    x = x0
    for i, t, first in run_order(cfg):
        if first:
            x = np.concatenate([x, x0], 1) @ weights["loop.in"].T + weights["loop.step"][t]
        x = layer(x, weights, i, cfg["layers"][i], cfg, positions)
        if trace is not None:
            trace.append(x.copy())
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    return group_norm(x, weights["final.norm"], eps, groups) @ weights["head"].T
