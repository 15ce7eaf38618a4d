"""Recurrent mixers whose matrix state fades by a factor that depends on the token.

Both keep, per head, a state ``S`` (``key_dim x value_dim``, float32 in both precisions, zero at a request's start) in the
request's slot and advance it token by token with one kernel (``ops.gated_state_scan``), whose sums run in one order
whatever the step's cut.  A step that brings a portion of ``2 * SEGMENT`` tokens or more walks its portions in segments
side by side (over a segment the state goes ``S -> M S + B``; ``ops.gated_state_scan_segments``); results then differ
from the walk in one piece by float32 rounding.

``GatedDelta`` (the gated delta rule): with ``x`` the mixer's input,

    [q | k | v | z | b | a] = W_in x                 one product; q, k: ``qk_heads`` heads of ``key_dim``, v, z: ``n_heads`` of ``value_dim``
    q, k, v <- silu(conv(.))                         a causal convolution over time per channel, no bias
    q <- q / sqrt(sum(q^2) + unit_eps) * key_dim^-0.5,   k <- k / sqrt(sum(k^2) + unit_eps)        per head
    beta = sigmoid(b),   g = exp(-exp(A_log) softplus(a + dt_bias))                                  per head
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    out = W_o (rms(o) * w * silu(z))                 the norm per head, its weight shared by the heads

The convolutions' last ``taps - 1`` inputs belong to the request's state too.

``GatedLinear`` (linear attention with a decay per key channel):

    [q | k | v | z] = W_in x,   alpha = sigmoid(W_up (W_down x) + b)^(1/tau)           n_heads x key_dim decays
    S <- diag(alpha) S + k v^T;  o = S^T (q key_dim^-0.5)
    out = W_o (rms(o) * w * silu(z))

From the convolutions' outputs (or the input product) to the gated norm nothing is rounded to the activation type:
unit norms, gates, decays and the state are float32.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, Part, SlotState, TensorSpec
from .registry import register


SEGMENT = 128      # tokens a segment: a step that brings a portion of twice as many walks its portions in segments


def _scan(ops, ctx, args, state, **kw):
    """The recurrence over this step's tokens: token by token a sequence, or, when a long portion is among them, the
    portions' segments side by side."""
    if not ctx.all_single and ctx.max_q_len >= 2 * SEGMENT:
        return ops.gated_state_scan_segments(*args, state, ctx.q_lens, ctx.slots, SEGMENT, **kw)
    return ops.gated_state_scan(*args, state, ctx.q_start, ctx.slots, ctx.nseq, **kw)


def _stacked(ws, pad_to: int = 16):
    """The weights one above the other, with rows of zeros below so that the row count is a multiple of ``pad_to``."""
    if len({w.dtype for w in ws}) > 1:
        ws = [w.float() for w in ws]
    rows = sum(w.shape[0] for w in ws)
    spare = -rows % pad_to
    if spare:
        ws = list(ws) + [torch.zeros((spare, ws[0].shape[1]), dtype=ws[0].dtype, device=ws[0].device)]
    return torch.cat(ws, 0).contiguous()


class GatedDelta(Part):
    graph_safe = True
    stage, out_stage = "delta_mixer", "delta_out"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.n_heads % spec.qk_heads:
            raise ValueError(f"{spec.n_heads} heads do not share {spec.qk_heads} queries and keys evenly")
        if spec.key_dim > rt.ops.GATED_STATE_MAX_KEY:
            raise ValueError(f"keys of {spec.key_dim} features: the state kernel holds up to {rt.ops.GATED_STATE_MAX_KEY}")

    @staticmethod
    def channels(spec) -> int:
        return 2 * spec.qk_heads * spec.key_dim + spec.n_heads * spec.value_dim

    @staticmethod
    def tensor_specs(spec):
        W, H, G, n, m, K = spec.hidden, spec.n_heads, spec.qk_heads, spec.key_dim, spec.value_dim, spec.conv_taps
        return {"q_proj.weight": TensorSpec((G * n, W), MATRIX), "k_proj.weight": TensorSpec((G * n, W), MATRIX),
                "v_proj.weight": TensorSpec((H * m, W), MATRIX), "gate_proj.weight": TensorSpec((H * m, W), MATRIX),
                "beta_proj.weight": TensorSpec((H, W), MATRIX), "decay_proj.weight": TensorSpec((H, W), MATRIX),
                "q_conv.weight": TensorSpec((G * n, K), VECTOR), "k_conv.weight": TensorSpec((G * n, K), VECTOR),
                "v_conv.weight": TensorSpec((H * m, K), VECTOR), "A_log": TensorSpec((H,), VECTOR),
                "dt_bias": TensorSpec((H,), VECTOR), "out_norm.weight": TensorSpec((m,), VECTOR, "one_plus_normal"),
                "out_proj.weight": TensorSpec((W, H * m), MATRIX)}

    @staticmethod
    def cache_need(spec):
        # (a single tap has no history; a row is kept all the same, which nobody reads)
        return SlotState((("conv_history", (max(spec.conv_taps - 1, 1), GatedDelta.channels(spec)), "float32"),
                          ("state", (spec.n_heads, spec.key_dim, spec.value_dim), "float32")))

    def bind(self, tensors):
        rt, s = self.rt, self.spec
        self.w_in = rt.prepare(_stacked([tensors[k + "_proj.weight"] for k in ("q", "k", "v", "gate", "beta", "decay")]))
        self.w_out = rt.prepare(tensors["out_proj.weight"])
        self.taps = torch.cat([tensors[k + "_conv.weight"] for k in ("q", "k", "v")], 0).contiguous()
        self.a_log, self.dt_bias = tensors["A_log"], tensors["dt_bias"]
        self.norm_weight = tensors["out_norm.weight"].repeat(s.n_heads).contiguous()      # one weight for every head

    takes_out_dtype = True

    def forward(self, x, ctx, cache, out_dtype=None):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        H, G, n, m = s.n_heads, s.qk_heads, s.key_dim, s.value_dim
        C = self.channels(s)
        with rt.stage("delta_in"):
            rows = rt.linear(rt.dense(x), self.w_in)                  # q | k | v | z | b | a (| spare columns)
        with rt.stage("delta_conv"):
            qkv = ops.channel_conv(rows[:, :C], self.taps, None, cache.state["conv_history"], ctx.seq_of_token,
                                   ctx.q_start, ctx.slots, ctx.nseq, ctx.all_single, torch.float32, activation="silu")
            gates = ops.delta_rule_prep(qkv, G, n, float(n) ** -0.5, s.unit_eps, rows, C + H * m + H, C + H * m,
                                        self.a_log, self.dt_bias, H)
        with rt.stage("delta_state"):
            o = _scan(ops, ctx, (qkv, 0, G * n, 2 * G * n, H, G, n, m, gates, 0, False), cache.state["state"], beta=gates, ob=H)
        with rt.stage("delta_norm"):
            y = ops.gated_outnorm(o, rows, C, self.norm_weight, s.eps, H, m, False, "silu", rt.dtype)
        return rt.linear(y, self.w_out, out_dtype=out_dtype)


class GatedLinear(Part):
    graph_safe = True
    stage, out_stage = "decay_mixer", "decay_out"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.key_dim > rt.ops.GATED_STATE_MAX_KEY:
            raise ValueError(f"keys of {spec.key_dim} features: the state kernel holds up to {rt.ops.GATED_STATE_MAX_KEY}")
        if not spec.tau > 0:
            raise ValueError("tau must be positive")

    @staticmethod
    def tensor_specs(spec):
        W, H, n, m, r = spec.hidden, spec.n_heads, spec.key_dim, spec.value_dim, spec.decay_rank
        return {"q_proj.weight": TensorSpec((H * n, W), MATRIX), "k_proj.weight": TensorSpec((H * n, W), MATRIX),
                "v_proj.weight": TensorSpec((H * m, W), MATRIX), "gate_proj.weight": TensorSpec((H * m, W), MATRIX),
                "decay_down.weight": TensorSpec((r, W), MATRIX), "decay_up.weight": TensorSpec((H * n, r), MATRIX),
                "decay_up.bias": TensorSpec((H * n,), VECTOR), "out_norm.weight": TensorSpec((m,), VECTOR, "one_plus_normal"),
                "out_proj.weight": TensorSpec((W, H * m), MATRIX)}

    @staticmethod
    def cache_need(spec):
        return SlotState((("state", (spec.n_heads, spec.key_dim, spec.value_dim), "float32"),))

    def bind(self, tensors):
        rt, s = self.rt, self.spec
        self.w_in = rt.prepare(_stacked([tensors[k + "_proj.weight"] for k in ("q", "k", "v", "gate")]))
        self.w_down = rt.prepare(_stacked([tensors["decay_down.weight"]]))
        up = tensors["decay_up.weight"]
        spare = self.w_down.shape[0] - up.shape[1]                     # the bottleneck's spare rows are zeros: columns of
        if spare:                                                      # zeros here change no sum
            up = torch.cat([up, torch.zeros((up.shape[0], spare), dtype=up.dtype, device=up.device)], 1)
        self.w_up = rt.prepare(up.contiguous())
        self.b_up = tensors["decay_up.bias"]
        self.w_out = rt.prepare(tensors["out_proj.weight"])
        self.norm_weight = tensors["out_norm.weight"].repeat(s.n_heads).contiguous()

    takes_out_dtype = True

    def forward(self, x, ctx, cache, out_dtype=None):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        H, n, m = s.n_heads, s.key_dim, s.value_dim
        x = rt.dense(x)
        with rt.stage("decay_in"):
            rows = rt.linear(x, self.w_in)                             # q | k | v | z
            alpha = rt.linear(rt.linear(x, self.w_down), self.w_up, self.b_up, out_dtype=torch.float32)
            ops.channel_decay(alpha, s.tau)
        with rt.stage("decay_state"):
            o = _scan(ops, ctx, (rows, 0, H * n, 2 * H * n, H, H, n, m, alpha, 0, True), cache.state["state"],
                      q_scale=float(n) ** -0.5)
        with rt.stage("decay_norm"):
            y = ops.gated_outnorm(o, rows, 2 * H * n + H * m, self.norm_weight, s.eps, H, m, False, "silu", rt.dtype)
        return rt.linear(y, self.w_out, out_dtype=out_dtype)


register("mixer", "gated_delta", GatedDelta)
register("mixer", "gated_linear", GatedLinear)
