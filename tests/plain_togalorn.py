"""Plain Togalorn: a slow, whole-sequence, cache-free implementation used as the oracle.

Nothing is imported from ``gesso_amd``: a model folder is read with ``json`` and the ``safetensors`` package, the
arithmetic is explicit torch on the CPU in float64 (or another type on request).  One function per mechanism:

    embedding  rms  group_norm  causal_conv  rotate_interleaved  latent_attention  state_space  mamba2  expert  route
    moe  layer  run_order  forward

Notation.  Rows are tokens: activations are ``(T, features)``, a linear weight ``W`` is ``(out, in)`` and acts as
``y = x @ W.T``; positions count from 0.  ``rms(x) = x / sqrt(mean(x^2) + eps)``, eps under the root.

The model.  ``x0 = E[token] * scale``.  Layers run in the order ``run_order`` gives: the layers ``start .. stop - 1`` of
``loop`` run ``times`` times in a row with the same weights; right before the first layer of pass ``t`` (the first pass
too) ``x <- W_in [x; x0] + step[t]``.  A layer: ``a = group_norm(x)`` (the row in ``groups`` equal consecutive parts, each
divided by its own root mean square, the whole times a weight); ``x <- x + mixer(a + conv(a)) + ff(a)`` with ``conv`` a
causal convolution over time per channel, ``conv(a)_t = sum_j w[:, j] a_(t - taps + 1 + j)``, zeros before the start.
Logits are ``W_head group_norm(x)``.

Mixer ``latent_attention``: ``c_q = rms(W_dq h) g_q``, ``q = W_uq c_q`` laid out head by head as ``[dim plain | rot_dim
rotated]``; ``W_dkv h`` gives ``kv_rank`` features that, normed (``rms(.) g_kv``), are the latent ``c``, and ``rot_dim``
more that are one rotated key part for all heads; per head ``k_plain = W_uk c``, ``v = W_uv c``; the rotated parts of q
and k are turned by the position, feature ``2i`` paired with ``2i + 1``, angle ``p base^(-2i/dims)``; causal softmax of
``(q_plain . k_plain + q_rot . k_rot) scale``; the heads side by side times ``sigmoid(W_g h)``, then ``W_o``.

Mixer ``mamba2``: ``W_in h = [z | x | B | C | dt]`` (``inner = heads vdim``, ``inner``, ``groups state``, ``groups state``,
``heads``); x, B, C together pass a causal convolution per channel with a bias and silu; ``dt <- softplus(dt + dt_bias)``;
per head ``h`` with group ``h // (heads / groups)``: ``S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T``
(``state x vdim``, from 0), ``y_t = S_t^T C_t + D_h x_t``; ``y silu(z)`` is normed in ``norm_groups`` equal parts (each by
its own root mean square) times a weight, then ``W_o``.

Feed-forward ``moe``: scores ``s = softmax(W_router h)`` over ``experts + identity`` outputs; the ``top`` outputs with the
largest ``s + correction`` are chosen, weighted by their ``s`` over the chosen's sum (+ 1e-20); an expert is
``W_down (g sigmoid(1.702 g) (u + 1))`` with ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, -limit, limit)``; the last
``identity`` outputs are experts without tensors that give back ``h``; a shared expert of the same form (its own width
and limit) runs for every token and is added.
"""
from __future__ import annotations

import json
import math
import os

import torch


def _keep(x):
    return x


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and widen back: what a pipeline with bfloat16 activations does where it stores one."""
    return x.to(torch.bfloat16).to(x.dtype)


def linear(x, W):
    return x @ W.T


def silu(z):
    return z * torch.sigmoid(z)


# --------------------------------------------------------------------------- small mechanisms

def embedding(table: torch.Tensor, ids, scale: float) -> torch.Tensor:
    rows = []
    for tok in ids:
        tok = int(tok)
        if not 0 <= tok < table.shape[0]:
            raise ValueError(f"token id {tok} outside the vocabulary of {table.shape[0]}")
        rows.append(table[tok])
    return torch.stack(rows, 0) * scale


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def group_norm(x, weight, eps: float, groups: int):
    """The row in ``groups`` equal consecutive parts, each divided by its own root mean square; then the weight."""
    T, W = x.shape
    return rms(x.reshape(T, groups, W // groups), eps).reshape(T, W) * weight


def causal_conv(x, taps, bias=None):
    """``y_t = sum_j taps[:, j] x_(t - K + 1 + j)`` per channel (the last column meets the current token), zeros before
    the sequence's start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros((K - 1, C), dtype=x.dtype), x], 0)
    y = torch.zeros((T, C), dtype=x.dtype)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y if bias is None else y + bias


def rotate_interleaved(x, positions, base: float, dims: int):
    """Pairs ``(2i, 2i + 1)`` of the first ``dims`` features of the last axis turned by ``p base^(-2i/dims)``; ``x`` is
    ``(T, ..., features)``."""
    out = x.clone()
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    a = torch.tensor([float(p) for p in positions], dtype=torch.float64)[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.dim() - 2) + (half,)
    c, s = torch.cos(a).reshape(shape).to(x.dtype), torch.sin(a).reshape(shape).to(x.dtype)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# --------------------------------------------------------------------------- mixers

def latent_attention(h, w, p, m, eps, positions, store=_keep):
    T = h.shape[0]
    H, n, r, dv, c = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = store(rms(store(linear(h, w[p + ".dq"])), eps) * w[p + ".dq.norm"])
    q = store(linear(cq, w[p + ".uq"])).reshape(T, H, n + r)
    down = store(linear(h, w[p + ".dkv"]))
    lat = store(rms(down[:, :c], eps) * w[p + ".dkv.norm"])
    k_rot, q_rot = down[:, c:], q[..., n:]
    if r:
        base, dims = m["rot"]["base"], m["rot"]["dims"]
        k_rot = store(rotate_interleaved(k_rot, positions, base, dims))             # (T, r), one for all heads
        q_rot = store(rotate_interleaved(q_rot, positions, base, dims))
    k_plain = linear(lat, w[p + ".uk"]).reshape(T, H, n)
    v = linear(lat, w[p + ".uv"]).reshape(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q[..., :n], k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    seen = torch.ones((T, T), dtype=torch.bool).tril()
    pr = torch.softmax(scores.masked_fill(~seen[None], -math.inf), dim=-1)
    mixed = store(torch.einsum("hij,jhd->ihd", pr, v).reshape(T, H * dv))
    return store(linear(store(mixed * torch.sigmoid(store(linear(h, w[p + ".g"])))), w[p + ".o"]))


def state_space(x, B, C, dt, a_log, d_skip, heads_per_group: int):
    """Per head ``S_t = exp(-exp(a_log) dt_t) S_(t-1) + dt_t B_t x_t^T`` (state x vdim), ``y_t = S_t^T C_t + D x_t``.
    ``x (T, H, P)``, ``B, C (T, G, N)``, ``dt (T, H)``."""
    T, H, P = x.shape
    N = B.shape[2]
    y = torch.zeros((T, H, P), dtype=x.dtype)
    for hd in range(H):
        g = hd // heads_per_group
        S = torch.zeros((N, P), dtype=x.dtype)
        rate = math.exp(float(a_log[hd]))
        for t in range(T):
            S = math.exp(-rate * float(dt[t, hd])) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + d_skip[hd] * x[t, hd]
    return y


def mamba2(h, w, p, m, eps, store=_keep):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    rows = store(linear(h, w[p + ".in"]))
    z, xbc, dt = rows[:, :inner], rows[:, inner:2 * inner + 2 * G * N], rows[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + ".conv"], w[p + ".conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + ".dt_bias"], threshold=1e9)
    y = state_space(x, B, C, dt, w[p + ".A_log"], w[p + ".D"], H // G).reshape(T, inner)
    y = store(group_norm(y * silu(z), w[p + ".norm"], eps, m["norm_groups"]))
    return store(linear(y, w[p + ".o"]))


# --------------------------------------------------------------------------- feed-forward

def expert(h, gate, up, down, limit: float, store=_keep):
    g = torch.clamp(store(linear(h, gate)), max=limit)
    u = torch.clamp(store(linear(h, up)), -limit, limit)
    return linear(store(g * torch.sigmoid(1.702 * g) * (u + 1.0)), down)


def route(h, router, correction, top: int):
    """``(chosen (T, top), weights (T, top), scores (T, outputs))``: softmax over all router outputs; the choice looks at
    scores + correction (of equal ones the lowest index), the weights are the plain scores of the chosen over their sum."""
    s = torch.softmax(linear(h, router), dim=-1)
    chosen = torch.sort(-(s + correction), dim=-1, stable=True).indices[:, :top]
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20), s


def choice_margin(scores, correction, top: int):
    """Per token: by how much the last chosen output's corrected score leads the best one left out (inf: all chosen)."""
    ranked = torch.sort(scores + correction, dim=-1, descending=True).values
    if top >= ranked.shape[1]:
        return torch.full((ranked.shape[0],), math.inf, dtype=ranked.dtype)
    return ranked[:, top - 1] - ranked[:, top]


def moe(h, w, p, m, store=_keep, margins=None):
    E, top = m["router"]["experts"], m["router"]["top"]
    chosen, weights, scores = route(h, w[p + ".router"], w[p + ".correction"], top)
    if margins is not None:
        margins.append(choice_margin(scores, w[p + ".correction"], top))
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            if e >= E:                                   # an identity expert: the input itself
                y[t] = y[t] + a * h[t]
            else:
                q = f"{p}.e{e}"
                y[t] = y[t] + a * expert(h[t:t + 1], w[q + ".gate"], w[q + ".up"], w[q + ".down"], m["expert"]["limit"], store)[0]
    if m.get("shared") is not None:
        q = p + ".shared"
        y = y + store(expert(h, w[q + ".gate"], w[q + ".up"], w[q + ".down"], m["shared"]["limit"], store))
    return store(y)


# --------------------------------------------------------------------------- layers, the model

def layer(x, w, i, cfg, positions, store=_keep, margins=None):
    """``x + mixer(a + conv(a)) + ff(a)`` with ``a`` the norm in parts of ``x``."""
    L = cfg["layers"][i]
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups") or 1)
    a = store(group_norm(x, w[f"l{i}.norm1"], eps, groups))
    hm = a
    if (cfg.get("canon") or {}).get("taps") is not None:
        hm = store(a + causal_conv(a, w[f"l{i}.canon1"]))
    if L["type"] == "latent_attention":
        y = latent_attention(hm, w, f"l{i}.mix", L["mixer"], eps, positions, store)
    elif L["type"] == "mamba2":
        y = mamba2(hm, w, f"l{i}.mix", L["mixer"], eps, store)
    else:
        raise ValueError(f"unknown layer type {L['type']!r}")
    if L.get("mlp") is not None:
        y = y + moe(a, w, f"l{i}.mlp", L["mlp"], store, margins)
    return x + y


def run_order(cfg):
    """``[(layer, pass or None if the layer stands outside the loop, whether it is the first of its pass)]`` in the order
    the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None, False) for i in range(a)]
    for t in range(times):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        return json.load(f)


def read_weights(model_dir: str, dtype=torch.float64) -> dict:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            out[name] = t.to(dtype) if t.is_floating_point() else t.to(torch.int64)
    return out


def forward(cfg: dict, w: dict, ids, store=_keep, layers_out=None, margins=None) -> torch.Tensor:
    """Logits ``(T, vocab)`` of the whole sequence ``ids``, positions from 0.  ``layers_out``: a list that receives the
    residual stream after every layer run.  ``margins``: a list that receives, for every feed-forward run, each token's
    :func:`choice_margin`."""
    ids = [int(t) for t in ids]
    positions = list(range(len(ids)))
    x0 = embedding(w["embed"], ids, float((cfg.get("embedding") or {}).get("scale") or 1.0))
    x = x0
    for i, t, first in run_order(cfg):
        if first:
            x = linear(torch.cat([store(x), store(x0)], 1), w["loop.in"]) + w["loop.step"][t]
        x = layer(x, w, i, cfg, positions, store, margins)
        if layers_out is not None:
            layers_out.append(x.clone())
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups") or 1)
    return linear(store(group_norm(x, w["final.norm"], eps, groups)), w["head"])


def greedy(cfg: dict, w: dict, prompt, max_new_tokens: int):
    ids = [int(t) for t in prompt]
    for _ in range(max_new_tokens):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids
