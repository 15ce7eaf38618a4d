"""Linear attention through a fading matrix state, and two mixers side by side.

``LinearAttention``: ``q, k, v, g = x W_q^T, x W_k^T, x W_v^T, x W_g^T`` (one product); per head a state
``S_t = decay_h S_(t-1) + k_t v_t^T`` (``key_dim x value_dim``) and ``o_t = S_t^T q_t``; the heads' outputs are normed,
multiplied by a function of ``g`` and projected by ``W_o``.  The spec says whether q, k and v are activated, whether q
and k are turned by the position, by what k is scaled, how the output is normed (all heads as one row with a weight, or
each head by its own root mean square) and which function gates it.  The state is the request's: one slot, float32 in
both precisions, zero at a request's start.  Between the input product and the norm nothing is rounded to the activation
type: activation, turn and scale are applied where the state kernel reads its operands, and its output stays float32
until norm and gate have been applied.

``MixerPair``: two mixers that read the same rows, each with a cache of its own; the result is
``left_scale * left(x) + right_scale * right(x)``, summed in float32 and rounded once; with ``branch_norm_eps`` each side
is first RMS-normed over the model width with a weight of its own.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, Part, SlotState, TensorSpec, sub_tensors
from .registry import build, part_class, register


class LinearAttention(Part):
    graph_safe = True
    stage, out_stage = "linear_mixer", "linear_out"
    RUNS_FROM = 8       # sequences that bring at least this many tokens to a step go to the kernel on the matrix cores
    SEGMENT = 128       # tokens of a segment where long portions are cut to fill the chip

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if len(spec.decay) != spec.n_heads:
            raise ValueError(f"{len(spec.decay)} decay factors for {spec.n_heads} heads")
        if spec.out_norm not in ("joint", "head"):
            raise ValueError(f"out_norm is 'joint' or 'head', not {spec.out_norm!r}")
        if spec.key_dim > rt.ops.LINEAR_ATTENTION_MAX_KEY:
            raise ValueError(f"keys of {spec.key_dim} features: the state kernel holds up to {rt.ops.LINEAR_ATTENTION_MAX_KEY}")
        self.position = build("position", spec.position, rt)
        if self.position.rotary_dim and getattr(self.position, "layout", "half") != "half":
            raise ValueError("the state kernel turns half-split pairs only")
        if self.position.rotary_dim > spec.key_dim:
            raise ValueError("more turned features than a key has")

    @staticmethod
    def tensor_specs(spec):
        W, H, n, m = spec.hidden, spec.n_heads, spec.key_dim, spec.value_dim
        out = {"q_proj.weight": TensorSpec((H * n, W), MATRIX), "k_proj.weight": TensorSpec((H * n, W), MATRIX),
               "v_proj.weight": TensorSpec((H * m, W), MATRIX), "gate_proj.weight": TensorSpec((H * m, W), MATRIX),
               "out_proj.weight": TensorSpec((W, H * m), MATRIX)}
        if spec.out_norm == "joint":
            out["out_norm.weight"] = TensorSpec((H * m,), VECTOR, "one_plus_normal")
        return out

    @staticmethod
    def cache_need(spec):
        return SlotState((("state", (spec.n_heads, spec.key_dim, spec.value_dim), "float32"),))

    def bind(self, tensors):
        ws = [tensors[k + "_proj.weight"] for k in ("q", "k", "v", "gate")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.float() for w in ws]
        self.w_in = self.rt.prepare(torch.cat(ws, 0).contiguous())
        self.w_out = self.rt.prepare(tensors["out_proj.weight"])
        self.norm_weight = tensors.get("out_norm.weight")
        self.decay = torch.tensor([float(d) for d in self.spec.decay], dtype=torch.float32, device=self.rt.device)

    def heads(self, x, ctx, cache, scale: float = 1.0):
        """The rows that the output projection takes: the heads' normed and gated outputs ``(T, H m)``."""
        s, rt, ops, pos = self.spec, self.rt, self.rt.ops, self.position
        H, n, m = s.n_heads, s.key_dim, s.value_dim
        with rt.stage("linear_in"):
            rows = rt.linear(rt.dense(x), self.w_in)                   # q | k | v | g
        with rt.stage("linear_state"):
            args = (rows, 0, H * n, 2 * H * n, H, n, m, self.decay, cache.state["state"], ctx.q_start, ctx.slots,
                    ctx.positions, ctx.nseq)
            kw = dict(activation=s.activation, cos=pos.cos, sin=pos.sin, rotary_dim=pos.rotary_dim, key_scale=s.key_scale)
            runs = (rt.options.linear_attention == "auto" and rows.dtype == torch.bfloat16 and not ctx.all_single
                    and n <= ops.LINEAR_ATTENTION_CHUNKS_MAX_KEY and ctx.max_q_len >= self.RUNS_FROM)
            if runs:
                # prompt portions 32 tokens at a time on the matrix cores; what brings fewer tokens, token by token
                # few long portions: cut into segments that run side by side (a block a sequence and head would leave
                # most of the chip idle)
                blocks = sum(1 for L in ctx.q_lens if L >= self.RUNS_FROM) * H * -(-m // 128)
                cut = self.SEGMENT if ctx.max_q_len >= 2 * self.SEGMENT and blocks < rt.compute_units else 0
                o = ops.linear_attention_scan(*args, chunks_from=self.RUNS_FROM, segment=cut, longest=ctx.max_q_len, **kw)
                if min(ctx.q_lens) < self.RUNS_FROM:
                    ops.linear_attention_scan(*args, below=self.RUNS_FROM, out=o, **kw)
            else:
                o = ops.linear_attention_scan(*args, **kw)
        with rt.stage("linear_norm"):
            return ops.gated_outnorm(o, rows, 2 * H * n + H * m, self.norm_weight, s.eps, H, m, s.out_norm == "joint",
                                     s.gate, rt.dtype)

    takes_out_dtype = True

    def forward(self, x, ctx, cache, out_dtype=None):
        return self.rt.linear(self.heads(x, ctx, cache), self.w_out, out_dtype=out_dtype)


class MixerPair(Part):
    stage = "pair_mixer"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.left = build("mixer", spec.left, rt)
        self.right = build("mixer", spec.right, rt)

    @staticmethod
    def tensor_specs(spec):
        out = {}
        for side, sub in (("left", spec.left), ("right", spec.right)):
            for name, ts in part_class("mixer", sub).tensor_specs(sub).items():
                out[f"{side}.{name}"] = ts
        if getattr(spec, "branch_norm_eps", None) is not None:
            if spec.hidden is None:
                raise ValueError("a pair that norms its branches must know the model width")
            out["left_norm.weight"] = TensorSpec((spec.hidden,), VECTOR, "one_plus_normal")
            out["right_norm.weight"] = TensorSpec((spec.hidden,), VECTOR, "one_plus_normal")
        return out

    @staticmethod
    def cache_need(spec):
        needs = []
        for sub in (spec.left, spec.right):
            cls = part_class("mixer", sub)
            needs.append(cls.cache_need(sub) if hasattr(cls, "cache_need") else None)
        return tuple(needs)

    def bind(self, tensors):
        self.left.bind(sub_tensors(tensors, "left"))
        self.right.bind(sub_tensors(tensors, "right"))
        self.left_norm, self.right_norm = tensors.get("left_norm.weight"), tensors.get("right_norm.weight")

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    def forward(self, x, ctx, cache):
        rt, s = self.rt, self.spec
        x = rt.dense(x)
        # a mixer that can leaves its last product's float32 sums, so that the weighted sum is rounded once
        wide = all(getattr(p, "takes_out_dtype", False) for p in (self.left, self.right))
        kw = {"out_dtype": torch.float32} if wide else {}
        a = rt.dense(self.left.forward(x, ctx, cache[0], **kw))
        b = rt.dense(self.right.forward(x, ctx, cache[1], **kw))
        eps = getattr(s, "branch_norm_eps", None)
        if eps is not None:
            # each side normed over the model width with its own weight, float32 from the products' sums to the one
            # rounding of the weighted sum
            if not wide:
                a, b = a.float(), b.float()
            return rt.ops.normed_pair_sum(a, self.left_norm, float(s.left_scale), b, self.right_norm, float(s.right_scale),
                                          float(eps), rt.dtype)
        return rt.ops.scaled_sum(a, float(s.left_scale), b, float(s.right_scale), rt.dtype)


register("mixer", "linear_attention", LinearAttention)
register("mixer", "mixer_pair", MixerPair)
