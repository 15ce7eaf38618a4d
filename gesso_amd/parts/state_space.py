"""A state-space mixer whose decay and step size depend on the token.

With ``x`` the mixer's input (``T`` rows), ``inner = H P`` (``H`` heads of ``P`` features), ``N`` state rows and ``G``
groups of heads that share their B and C:

    [z | u | B~ | C~ | d] = W_in x                        inner, inner, G N, G N, H columns
    [u' | B | C] = silu(conv([u | B~ | C~]) + b)          a causal convolution over time per channel
    dt = softplus(d + dt_bias),  a = exp(-exp(A_log) dt)                         per head, float32
    S_t = a_t S_(t-1) + dt_t B_t u'_t^T,   y_t = S_t^T C_t + D u'_t              S: N x P per head, float32
    out = W_o (norm_parts(y * silu(z)) * w)               the gate before the norm; norm_parts: RMS norm in equal parts

The request's state is one slot: the convolution's last ``taps - 1`` inputs and the matrices ``S``, float32 in both
precisions, zero at a request's start.  From the convolution's output to the norm nothing is rounded to the
activation type.  A portion of ``2 * SEGMENT`` tokens or more is walked in segments side by side (the state a segment
starts from is put together from what the segments before it add); results then differ from the walk in one piece by
float32 rounding.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, Part, SlotState, TensorSpec
from .registry import register


SEGMENT = 128      # tokens a segment: long portions are walked in segments of this many (or half), side by side


class StateSpace(Part):
    graph_safe = True
    stage, out_stage = "state_mixer", "state_out"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.n_heads % spec.groups:
            raise ValueError(f"{spec.n_heads} heads do not share {spec.groups} groups evenly")
        if (spec.n_heads * spec.head_dim) % spec.norm_groups:
            raise ValueError(f"{spec.norm_groups} norm parts do not divide {spec.n_heads * spec.head_dim} features")
        if spec.state > rt.ops.ssd_max_state(spec.head_dim):
            raise ValueError(f"a state of {spec.state} rows: the state kernel holds up to "
                             f"{rt.ops.ssd_max_state(spec.head_dim)} for heads of {spec.head_dim}")

    @staticmethod
    def sizes(spec):
        inner = spec.n_heads * spec.head_dim
        return inner, inner + 2 * spec.groups * spec.state

    @staticmethod
    def tensor_specs(spec):
        W, H = spec.hidden, spec.n_heads
        inner, chan = StateSpace.sizes(spec)
        return {"in_proj.weight": TensorSpec((inner + chan + H, W), MATRIX),
                "conv.weight": TensorSpec((chan, spec.conv_taps), VECTOR), "conv.bias": TensorSpec((chan,), VECTOR),
                "dt_bias": TensorSpec((H,), VECTOR), "A_log": TensorSpec((H,), VECTOR), "D": TensorSpec((H,), VECTOR),
                "norm.weight": TensorSpec((inner,), VECTOR, "one_plus_normal"),
                "out_proj.weight": TensorSpec((W, inner), MATRIX)}

    @staticmethod
    def cache_need(spec):
        inner, chan = StateSpace.sizes(spec)
        return SlotState((("conv_history", (max(spec.conv_taps - 1, 1), chan), "float32"),
                          ("state", (spec.n_heads, spec.state, spec.head_dim), "float32")))

    def bind(self, tensors):
        rt = self.rt
        self.w_in = rt.prepare(tensors["in_proj.weight"])
        self.w_out = rt.prepare(tensors["out_proj.weight"])
        self.taps, self.conv_bias = tensors["conv.weight"].contiguous(), tensors["conv.bias"]
        self.dt_bias, self.a_log, self.d_skip = tensors["dt_bias"], tensors["A_log"], tensors["D"]
        self.norm_weight = tensors["norm.weight"]

    def forward(self, x, ctx, cache):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        H, P, N, G = s.n_heads, s.head_dim, s.state, s.groups
        inner, chan = self.sizes(s)
        with rt.stage("state_in"):
            rows = rt.linear(rt.dense(x), self.w_in)                   # z | u | B | C | d
        with rt.stage("state_conv"):
            xbc = ops.channel_conv(rows[:, inner:inner + chan], self.taps, self.conv_bias, cache.state["conv_history"],
                                   ctx.seq_of_token, ctx.q_start, ctx.slots, ctx.nseq, ctx.all_single, torch.float32,
                                   activation="silu")
        with rt.stage("state_scan"):
            # a step that brings a long portion: its segments side by side instead of one walk a sequence and head
            segments = None
            if ctx.max_q_len >= 2 * SEGMENT:
                # shorter segments while the longer ones would leave compute units with fewer than four blocks
                blocks = (ctx.T // SEGMENT) * H * -(-P // 64)
                segments = ctx.state_segments(SEGMENT if blocks >= 4 * rt.compute_units else SEGMENT // 2)
            y = ops.ssd_scan(xbc, rows, inner + chan, self.dt_bias, self.a_log, self.d_skip, cache.state["state"],
                             ctx.q_start, ctx.slots, ctx.nseq, H, P, N, G, segments=segments)
        with rt.stage("state_norm"):
            g = ops.gated_group_norm(y, rows[:, :inner], self.norm_weight, s.eps, s.norm_groups, rt.dtype)
        return rt.linear(g, self.w_out)


register("mixer", "state_space", StateSpace)
