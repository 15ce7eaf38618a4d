"""Attention through low-rank latents, over a cache of one latent row per token.

With ``x`` the mixer's input (``T`` rows):

    a      = rms(W_dq x) * g_q                       query latent                       (T, q_rank)
    q      = W_uq a                                   head h: [n plain | r rotated]      (T, H (n + r))
    [z~|u] = W_dkv x;  z = rms(z~) * g_kv;  k_rot = rotate(u)                            (T, c), (T, r)
    k_h    = [W_uk[h] z | k_rot],  v_h = W_uv[h] z
    o_h    = softmax_j((q_h . k_h,j) * scale) v_h,j  over the keys the window lets a query see
    y      = W_o concat_h(sigmoid(W_g x)_h * o_h)

Only ``[z | k_rot]`` is cached: one key head of width ``c + r`` and no value rows (``PagedKV(1, c + r, window,
value_dim=0)``).  Keys and values of single heads are never formed.  Since ``q_plain . (W_uk[h] z) =
(W_uk[h]^T q_plain) . z``, the query takes ``W_uk`` along (``q~_h = [W_uk[h]^T q_plain | rotate(q_rot)]``), every head
attends over the cached rows themselves, and because the softmax weights sum over rows before ``W_uv`` is applied,
``o_h = W_uv[h] (sum_j p_j z_j)``.  A step of any shape (prompt portions, single tokens, both) takes this one route,
so a position's result does not depend on how its sequence was cut.

``W_dq``, ``W_dkv`` and ``W_g`` read the same input and are laid side by side at load: one product.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, PagedKV, Part, TensorSpec
from .registry import build, register


def _pad_rows(w: torch.Tensor, multiple: int = 16) -> torch.Tensor:
    """``w`` with rows of zeros appended up to a multiple: the products' fast paths want whole tiles of outputs."""
    extra = -w.shape[0] % multiple
    if extra:
        w = torch.cat([w, torch.zeros((extra, w.shape[1]), dtype=w.dtype, device=w.device)], 0)
    return w.contiguous()


class LatentAttention(Part):
    graph_safe = True
    stage, out_stage = "attn_mixer", "attn_outproj"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.rot_dim % 2:
            raise ValueError("rotated features come in pairs")
        self.position = build("position", spec.position, rt)
        if spec.rot_dim and self.position.rotary_dim != spec.rot_dim:
            raise ValueError("the rotated part of a head is rotated whole")
        # The kernels turn half-split pairs (i, i + r/2).  An encoding whose pairs are neighbours (2i, 2i + 1) is served
        # by reordering, at load, the rows of the two products that make the rotated features (evens first, then odds):
        # queries and the shared key part are reordered alike, so every score is the same sum in another order, and
        # nobody else reads these features (the cache holds the key part in the kernels' order).
        self.reorder = bool(spec.rot_dim) and getattr(self.position, "layout", "half") == "interleaved"

    @staticmethod
    def tensor_specs(spec):
        W, H, n, r, dv, qr, c = spec.hidden, spec.n_heads, spec.plain_dim, spec.rot_dim, spec.value_dim, spec.q_rank, spec.kv_rank
        out = {"q_down.weight": TensorSpec((qr, W), MATRIX), "q_norm.weight": TensorSpec((qr,), VECTOR, "one_plus_normal"),
               "q_up.weight": TensorSpec((H * (n + r), qr), MATRIX), "kv_down.weight": TensorSpec((c + r, W), MATRIX),
               "kv_norm.weight": TensorSpec((c,), VECTOR, "one_plus_normal"), "k_up.weight": TensorSpec((H * n, c), MATRIX),
               "v_up.weight": TensorSpec((H * dv, c), MATRIX), "out.weight": TensorSpec((W, H * dv), MATRIX)}
        if spec.gated:
            out["gate.weight"] = TensorSpec((H * dv if getattr(spec, "gate_each", False) else H, W), MATRIX)
        return out

    @staticmethod
    def cache_need(spec):
        return PagedKV(1, spec.kv_rank + spec.rot_dim, spec.window, value_dim=0)

    def bind(self, tensors):
        s, rt = self.spec, self.rt
        H, n, r, dv, c = s.n_heads, s.plain_dim, s.rot_dim, s.value_dim, s.kv_rank
        w_dkv, w_uq = tensors["kv_down.weight"], tensors["q_up.weight"]
        if self.reorder:
            order = torch.cat([torch.arange(0, r, 2), torch.arange(1, r, 2)]).to(w_dkv.device)
            w_dkv = torch.cat([w_dkv[:c], w_dkv[c:][order]], 0)
            per_head = torch.cat([torch.arange(n, device=order.device), n + order])
            rows = (torch.arange(H, device=order.device)[:, None] * (n + r) + per_head[None, :]).reshape(-1)
            w_uq = w_uq[rows].contiguous()
        ws = [tensors["q_down.weight"], w_dkv] + ([tensors["gate.weight"]] if s.gated else [])
        if len({w.dtype for w in ws}) > 1:
            ws = [w.float() for w in ws]
        self.w_in = rt.prepare(_pad_rows(torch.cat(ws, 0)))
        self.q_norm, self.kv_norm = tensors["q_norm.weight"], tensors["kv_norm.weight"]
        self.w_uq = rt.prepare(w_uq)
        # W_uk[h]^T as the weight of a per-head product: (H, c, n); W_uv[h]: (H, dv, c)
        self.uk_t = tensors["k_up.weight"].reshape(H, n, c).transpose(1, 2).contiguous() if n else None
        self.uv = tensors["v_up.weight"].reshape(H, dv, c).contiguous()
        self.w_out = rt.prepare(tensors["out.weight"])

    def forward(self, x, ctx, cache):
        s, rt, ops, pos = self.spec, self.rt, self.rt.ops, self.position
        H, n, r, dv, qr, c = s.n_heads, s.plain_dim, s.rot_dim, s.value_dim, s.q_rank, s.kv_rank
        x = rt.dense(x)
        T = x.shape[0]
        with rt.stage("attn_proj"):
            down = rt.linear(x, self.w_in)                     # [query latent | kv latent | shared rotated key | gate]
            a = ops.latent_prep(down, 0, qr, qr, c, r, self.q_norm, self.kv_norm, s.eps, pos.cos, pos.sin, ctx.positions,
                                ctx.seq_of_token, cache.block_table, cache.page_size, cache.k, write_kv=cache.write)
            q = rt.linear(a, self.w_uq)
            qa = (torch.empty if n else torch.zeros)((T, H * (c + r)), dtype=q.dtype, device=q.device)
            if n:
                ops.heads_product(q, n + r, self.uk_t, qa, c + r, n)
            ops.latent_q_rot(q, H, n, r, c, pos.cos, pos.sin, ctx.positions, qa)
        with rt.stage("attn_core"):
            mixed = self.attend(qa, ctx, cache)
        o = torch.empty((T, H * dv), dtype=mixed.dtype, device=mixed.device)
        ops.heads_product(mixed, c, self.uv, o, dv, c, gate=down[:, qr + c + r:] if s.gated else None,
                          gate_each=bool(s.gated and getattr(s, "gate_each", False)))
        return rt.linear(o, self.w_out)

    def attend(self, qa, ctx, cache) -> torch.Tensor:
        """The step's queries (absorbed form) over the cached rows: ``(T, H c)``."""
        s, ops = self.spec, self.rt.ops
        if (qa.dtype == torch.bfloat16 and self.rt.options.latent_attention != "general"
                and ops.attention_latent_mfma_supports(s.n_heads, s.kv_rank, s.rot_dim)):
            # the matrix cores, whatever the step holds: tiles of consecutive tokens of one sequence, all heads of a
            # tile in one block (a step of single tokens needs no list: sequence i is token i)
            tiles = None if ctx.all_single else ctx.query_tiles(ops.attention_latent_mfma_tokens(s.n_heads))
            nsplit = 1
            if ctx.all_single:
                # single tokens: few blocks, each with a long walk; the keys are shared out over blocks until the chip
                # is full, a part at least 64 keys long (the bound on the keys is the longest sequence's, or what the
                # block tables hold where the host does not know it, cut by the window)
                longest = ctx.max_kv_len if ctx.max_kv_len is not None else cache.block_table.shape[1] * cache.page_size
                if s.window:
                    longest = min(longest, s.window)
                blocks = ctx.T * -(-s.n_heads // 64)
                nsplit = max(1, min(longest // 64, 64, self.rt.compute_units // max(1, blocks)))
            return ops.attention_latent_mfma(qa, cache.k, ctx.positions, tiles, cache.block_table, cache.page_size,
                                             s.window, s.scale, s.n_heads, s.kv_rank, s.rot_dim, ctx.T, nsplit=nsplit)
        return ops.attention_latent(qa, cache.k, ctx.positions, ctx.seq_of_token, cache.block_table, cache.page_size,
                                    s.window, s.scale, s.n_heads, s.kv_rank, s.rot_dim, ctx.T)


register("mixer", "latent_attention", LatentAttention)
