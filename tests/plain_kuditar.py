"""Plain Kuditar: a slow, whole-sequence, cache-free implementation used as the oracle.

Nothing is imported from ``gesso_amd``: a model folder is read with ``json`` and the ``safetensors`` package, the
arithmetic is explicit torch on the CPU in float64 (or another type on request).  One function per mechanism:

    embedding  layer_norm  rms  frequencies  rotate_half  visible  softmax_attention  gated_attention  windowed_branch
    chunked_branch  causal_conv  delta_rule  delta_branch  gated_linear  gated_linear_branch  pair  clamped_glu  route
    moe  layer  forward

Notation.  Rows are tokens: activations are ``(T, features)``, a linear weight ``W`` is ``(out, in)`` and acts as
``y = x @ W.T``; positions count from 0.  ``rms(x) = x / sqrt(mean(x^2) + eps)``, eps under the root.

The model.  ``x = E[token] * scale``.  A layer: ``x <- x + mixer(ln1(x))``, then ``x <- x + ff(ln2(x))`` with
``ln(x) = (x - mean) / sqrt(var + eps) * w + b``.  Logits are ``E ln_final(x)``.

Mixer ``attention``: grouped-query attention without biases; q and k are turned by the position over their first
``rot.dims`` features (feature ``i`` with ``i + dims/2``, angle ``p base^(-2i/dims) / factor``), then each head's q and k
are divided by their root mean square; scores ``cap tanh((q . k) scale / cap)``; causal softmax; values of every layer
that says ``v_mix`` but the first such are blended with that first layer's values of the same token,
``(1 - lam) v + lam v_first``; the heads side by side are multiplied by ``sigmoid(W_g h)`` and projected by ``W_o``.

Mixer ``parallel``: half the sum of two branches, each normed over the model width (``rms(.) w``).  Left: attention with
biases on q, k, v, a weighted RMS norm of each head's q and k before the turn, capped scores, a view of the last
``mask.size`` positions plus the first ``mask.keep_first``, and a learned number per head whose exponential joins the
softmax's denominator.  Right: the gated delta rule: q, k, v through a causal convolution per channel and silu, q and k
made unit vectors (q also times ``dim^-0.5``), ``beta = sigmoid(W_b h)``,
``g = exp(-exp(A_log) softplus(W_a h + dt_bias))``, per head ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
o = S^T q``; each head's ``o`` normed with a weight, times ``silu(W_g h)``, then ``W_o``.

Mixer ``parallel_2``: the same sum of two normed branches.  Left: attention with biases and head norms, no turn, no cap,
a query sees the keys of its own run of ``mask.size`` positions.  Right: gated linear attention, a decay per key channel
``alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau)``, ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T (q_t dim^-0.5)``,
each head's ``o`` normed with a weight, the heads times ``silu(W_g h)``, then ``W_o``.

Feed-forward.  ``dense``: ``W_down (g sigmoid(1.702 g) (u + 1))`` with ``g = min(W_gate h, limit)``,
``u = clamp(W_up h, -limit, limit)``.  ``moe``: scores ``s = sigmoid(W_router h)``; the ``top`` experts with the largest
``s + correction`` are chosen and weighted by ``s * router.scale``; an expert has the dense form.
"""
from __future__ import annotations

import json
import math
import os

import torch

ACTIVATION_SLOPE = 1.702
UNIT_EPS = 1e-6


def _keep(x):
    return x


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and widen back: what a pipeline with bfloat16 activations does where it stores one."""
    return x.to(torch.bfloat16).to(x.dtype)


def linear(x, W, b=None):
    y = x @ W.T
    return y if b is None else y + b


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- small mechanisms

def embedding(table, ids, scale: float):
    rows = []
    for tok in ids:
        tok = int(tok)
        if not 0 <= tok < table.shape[0]:
            raise ValueError(f"token id {tok} outside the vocabulary of {table.shape[0]}")
        rows.append(table[tok])
    return torch.stack(rows, 0) * scale


def layer_norm(x, w, b, eps: float):
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x, eps: float):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def frequencies(dims: int, base: float, factor: float = 1.0):
    """``f_i = base^(-2i/dims) / factor`` for ``i`` below ``dims / 2``."""
    return torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=torch.float64)


def rotate_half(x, positions, freqs):
    """``x (T, heads, d)``: the first ``2 len(freqs)`` features of every head turned, feature ``i`` with
    ``i + len(freqs)``; the rest as they are."""
    n = len(freqs)
    if n == 0:
        return x
    ang = torch.tensor([float(p) for p in positions], dtype=torch.float64)[:, None] * freqs[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], dim=-1)


def visible(i: int, j: int, window=None, keep_first: int = 0, chunk=None) -> bool:
    """Whether the query at position ``i`` sees the key at position ``j``."""
    if j > i:
        return False
    if window is not None and not (i - j < window or j < keep_first):
        return False
    if chunk is not None and i // chunk != j // chunk:
        return False
    return True


def softmax_attention(q, k, v, positions, scale, cap=None, window=None, keep_first=0, chunk=None, sink=None):
    """``q (T, H, d)``, ``k (T, G, d)``, ``v (T, G, vd)``: every head's weighted sums ``(T, H, vd)``.  ``sink (H,)``: one
    more term ``exp(sink_h)`` in the denominator."""
    T, H, d = q.shape
    G = k.shape[1]
    seen = torch.tensor([[visible(positions[a], positions[b], window, keep_first, chunk) for b in range(T)]
                         for a in range(T)], dtype=torch.bool)
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, -math.inf)
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h])
        e = torch.exp(s - top)
        den = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - top)
        out[:, h] = (e / den) @ v[:, g]
    return out


def causal_conv(x, taps):
    """``x (T, C)``, ``taps (C, n)``: ``y_t = sum_j taps[:, j] x_(t - n + 1 + j)``, zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros((n - 1, C), dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(n):
        y = y + padded[j:j + T] * taps[:, j]
    return y


def unit(x):
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + UNIT_EPS)


def delta_rule(q, k, v, beta, g):
    """One head: ``q, k (T, n)``, ``v (T, m)``, ``beta, g (T,)``.  ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q``."""
    T, n = q.shape
    S = torch.zeros((n, v.shape[1]), dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out, 0)


def gated_linear(q, k, v, alpha):
    """One head: ``q, k, alpha (T, n)``, ``v (T, m)``.  ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``."""
    T, n = q.shape
    S = torch.zeros((n, v.shape[1]), dtype=q.dtype)
    out = []
    for t in range(T):
        S = alpha[t][:, None] * S + torch.outer(k[t], v[t])
        out.append(S.T @ q[t])
    return torch.stack(out, 0)


# --------------------------------------------------------------------------- mixers

def _rot_freqs(m):
    rot = m.get("rot")
    if not rot:
        return frequencies(0, 1.0)
    factor = (rot.get("scaling") or {}).get("factor") or 1.0
    return frequencies(int(rot["dims"]), float(rot["base"]), float(factor))


def gated_attention(h, W, p, m, positions, eps, v_first=None, store=_keep):
    """Mixer ``attention``.  Returns ``(output, this layer's own values)``.  ``store``: applied wherever a pipeline with
    activations of another type would store one (here and in the functions below)."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(linear(h, W[p + "q"])).reshape(T, H, d)
    k = store(linear(h, W[p + "k"])).reshape(T, G, d)
    v = store(linear(h, W[p + "v"])).reshape(T, G, vd)
    f = _rot_freqs(m)
    q, k = store(rms(rotate_half(q, positions, f), eps)), store(rms(rotate_half(k, positions, f), eps))
    own = v
    if v_first is not None:
        lam = W[p + "vmix"]
        v = store((1 - lam) * v + lam * v_first)
    o = store(softmax_attention(q, k, v, positions, m["scale"], cap=m.get("softcap")))
    o = store(o.reshape(T, H * vd) * torch.sigmoid(store(linear(h, W[p + "g"]))))
    return store(linear(o, W[p + "o"])), own


def _normed_biased_heads(h, W, p, m, eps, store=_keep):
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(linear(h, W[p + "q"], W[p + "q.b"])).reshape(T, H, d)
    k = store(linear(h, W[p + "k"], W[p + "k.b"])).reshape(T, G, d)
    v = store(linear(h, W[p + "v"], W[p + "v.b"])).reshape(T, G, vd)
    return rms(q, eps) * W[p + "q.norm"], rms(k, eps) * W[p + "k.norm"], v


def windowed_branch(h, W, p, m, positions, eps, store=_keep):
    """Left side of ``parallel``."""
    q, k, v = _normed_biased_heads(h, W, p, m, eps, store)
    f = _rot_freqs(m)
    q, k = store(rotate_half(q, positions, f)), store(rotate_half(k, positions, f))
    mask = m.get("mask") or {}
    o = softmax_attention(q, k, v, positions, m["scale"], cap=m.get("softcap"), window=mask.get("size"),
                          keep_first=mask.get("keep_first") or 0, sink=W[p + "sink"])
    return linear(store(o).reshape(h.shape[0], -1), W[p + "o"])


def chunked_branch(h, W, p, m, positions, eps, store=_keep):
    """Left side of ``parallel_2``."""
    q, k, v = _normed_biased_heads(h, W, p, m, eps, store)
    o = softmax_attention(store(q), store(k), v, positions, m["scale"], chunk=(m.get("mask") or {}).get("size"))
    return linear(store(o).reshape(h.shape[0], -1), W[p + "o"])


def delta_branch(h, W, p, m, eps, store=_keep):
    """Right side of ``parallel``."""
    T = h.shape[0]
    H, G, n, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(store(linear(h, W[p + "q"])), W[p + "q.conv"])).reshape(T, G, n)
    k = silu(causal_conv(store(linear(h, W[p + "k"])), W[p + "k.conv"])).reshape(T, G, n)
    v = silu(causal_conv(store(linear(h, W[p + "v"])), W[p + "v.conv"])).reshape(T, H, vd)
    q, k = unit(q) * n ** -0.5, unit(k)
    beta = torch.sigmoid(store(linear(h, W[p + "b"])))
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(store(linear(h, W[p + "a"])) + W[p + "dt_bias"]))
    heads = []
    for hd in range(H):
        j = hd // (H // G)
        heads.append(rms(delta_rule(q[:, j], k[:, j], v[:, hd], beta[:, hd], g[:, hd]), eps) * W[p + "norm"])
    o = store(torch.stack(heads, 1).reshape(T, H * vd) * silu(store(linear(h, W[p + "g"]))))
    return linear(o, W[p + "o"])


def gated_linear_branch(h, W, p, m, eps, store=_keep):
    """Right side of ``parallel_2``."""
    T = h.shape[0]
    H, n, vd = m["heads"], m["dim"], m["vdim"]
    q = (store(linear(h, W[p + "q"])) * n ** -0.5).reshape(T, H, n)
    k = store(linear(h, W[p + "k"])).reshape(T, H, n)
    v = store(linear(h, W[p + "v"])).reshape(T, H, vd)
    z = linear(store(linear(h, W[p + "a1"])), W[p + "a2"], W[p + "a2.b"])
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, n)
    heads = [rms(gated_linear(q[:, hd], k[:, hd], v[:, hd], alpha[:, hd]), eps) * W[p + "norm"] for hd in range(H)]
    o = store(torch.stack(heads, 1).reshape(T, H * vd) * silu(store(linear(h, W[p + "g"]))))
    return linear(o, W[p + "o"])


def pair(left, right, W, p, eps, store=_keep):
    return store(0.5 * (rms(left, eps) * W[p + "left.out"] + rms(right, eps) * W[p + "right.out"]))


# --------------------------------------------------------------------------- feed-forward

def clamped_glu(h, W, p, limit, store=_keep):
    g = torch.clamp(store(linear(h, W[p + "gate"])), max=limit)
    u = torch.clamp(store(linear(h, W[p + "up"])), -limit, limit)
    return linear(store(g * torch.sigmoid(ACTIVATION_SLOPE * g) * (u + 1)), W[p + "down"])


def route(h, W, p, top: int, scale: float):
    """``(chosen experts (T, top), their weights (T, top))``; ties go to the lower index."""
    s = torch.sigmoid(linear(h, W[p + "router"]))
    choice = s + W[p + "correction"]
    chosen = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    return chosen, torch.gather(s, 1, chosen) * scale


def moe(h, W, p, mlp, store=_keep):
    r = mlp["router"]
    chosen, weights = route(h, W, p, r["top"], r.get("scale") or 1.0)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            out[t] = out[t] + w * clamped_glu(h[t:t + 1], W, f"{p}e{e}.", mlp["expert"]["limit"], store)[0]
    return store(out)


def feed_forward(h, W, p, mlp, store=_keep):
    if mlp["kind"] == "dense":
        return store(clamped_glu(h, W, p, mlp["limit"], store))
    return moe(h, W, p, mlp, store)


# --------------------------------------------------------------------------- the model

def layer(x, W, i: int, entry, positions, eps, shared, store=_keep):
    """One layer on ``x (T, width)``; ``shared`` carries the first ``v_mix`` layer's values through the model."""
    p = f"l{i}."
    m = entry["mixer"]
    h = store(layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps))
    if entry["type"] == "attention":
        if m.get("v_mix"):
            y, own = gated_attention(h, W, p + "mix.", m, positions, eps, shared.get("v_first"), store)
            shared.setdefault("v_first", own)
        else:
            y, _ = gated_attention(h, W, p + "mix.", m, positions, eps, None, store)
    elif entry["type"] == "parallel":
        y = pair(windowed_branch(h, W, p + "mix.left.", m["left"], positions, eps, store),
                 delta_branch(h, W, p + "mix.right.", m["right"], eps, store), W, p + "mix.", eps, store)
    elif entry["type"] == "parallel_2":
        y = pair(chunked_branch(h, W, p + "mix.left.", m["left"], positions, eps, store),
                 gated_linear_branch(h, W, p + "mix.right.", m["right"], eps, store), W, p + "mix.", eps, store)
    else:
        raise ValueError(f"unknown layer type {entry['type']!r}")
    x = x + y
    if entry.get("mlp") is not None:
        h = store(layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps))
        x = x + feed_forward(h, W, p + "mlp.", entry["mlp"], store)
    return x


def forward(cfg: dict, W: dict, ids, store=_keep, layers_out=None):
    """Logits ``(T, vocab)`` of one whole sequence from position 0, in the tensors' type.  ``layers_out``: a list that
    receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    positions = list(range(len(ids)))
    x = embedding(W["embed"], ids, float((cfg.get("embedding") or {}).get("scale") or 1.0))
    shared = {}
    for i, entry in enumerate(cfg["layers"]):
        x = layer(x, W, i, entry, positions, eps, shared, store)
        if layers_out is not None:
            layers_out.append(x.clone())
    return linear(store(layer_norm(x, W["final.norm"], W["final.norm.b"], eps)), W["embed"])


def greedy(cfg: dict, W: dict, prompt, n_new: int):
    """The prompt and ``n_new`` tokens after it, each the largest logit's (the lowest id among equals), every step from
    the whole sequence anew."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, W, ids)[-1])))
    return ids


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json"), encoding="utf-8") as f:
        return json.load(f)


def read_weights(folder: str, dtype=torch.float64) -> dict:
    from safetensors.torch import load_file
    return {k: (v.to(dtype) if v.is_floating_point() else v)
            for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
