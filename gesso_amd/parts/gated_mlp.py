"""Gated feed-forward with a choice of activation and optional biases:
``W_down (act(W_gate x + b_gate) * (W_up x + b_up)) + b_down``; ``act`` is silu or the tanh form of gelu.

W_gate and W_up are laid side by side at load so that one product feeds both (as :mod:`gesso_amd.parts.swiglu` does);
biases, activation and the product of the two halves are one pass in float32 over the product's rows.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, Part, TensorSpec
from .registry import register


class GatedMLP(Part):
    graph_safe = True
    stage, out_stage = "dense_ffn", "ffn_down"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.activation not in rt.ops.GATED_ACTS:
            raise ValueError(f"activation {spec.activation!r}; the kernel has {sorted(rt.ops.GATED_ACTS)}")

    @staticmethod
    def tensor_specs(spec):
        H, F = spec.hidden, spec.intermediate
        out = {"gate.weight": TensorSpec((F, H), MATRIX), "up.weight": TensorSpec((F, H), MATRIX),
               "down.weight": TensorSpec((H, F), MATRIX)}
        if spec.bias:
            out.update({"gate.bias": TensorSpec((F,), VECTOR), "up.bias": TensorSpec((F,), VECTOR),
                        "down.bias": TensorSpec((H,), VECTOR)})
        return out

    def bind(self, tensors):
        g, u = tensors["gate.weight"], tensors["up.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gu = self.rt.prepare(torch.cat([g, u], 0).contiguous(), unit=g.shape[0])
        self.w_down = self.rt.prepare(tensors["down.weight"])
        self.b_gu = self.b_down = None
        if self.spec.bias:
            self.b_gu = torch.cat([tensors["gate.bias"], tensors["up.bias"]], 0).contiguous()
            self.b_down = tensors["down.bias"]

    defers_bias = True

    def forward(self, x, ctx, defer_bias: bool = False):
        """``defer_bias``: returns ``(product without the last bias, that bias or None)``, for a block that adds the
        bias where it adds the product."""
        rt = self.rt
        with rt.stage("ffn_gateup"):
            gu = rt.linear(rt.dense(x), self.w_gu)
            a = rt.ops.gated_act(gu, self.b_gu, self.spec.activation, rt.dtype)
        if defer_bias:
            return rt.linear(a, self.w_down), self.b_down
        return rt.linear(a, self.w_down, self.b_down)


class ClampedGLU(Part):
    """``W_down (g sigmoid(alpha g) (u + 1))`` with ``g = min(W_gate x, limit)``, ``u = clamp(W_up x, -limit, limit)``:
    the form a routed expert has (:mod:`gesso_amd.parts.routed_moe`), as a feed-forward of its own for every token."""

    graph_safe = True
    stage, out_stage = "dense_ffn", "ffn_down"

    @staticmethod
    def tensor_specs(spec):
        H, F = spec.hidden, spec.intermediate
        return {"gate.weight": TensorSpec((F, H), MATRIX), "up.weight": TensorSpec((F, H), MATRIX),
                "down.weight": TensorSpec((H, F), MATRIX)}

    def bind(self, tensors):
        g, u = tensors["gate.weight"], tensors["up.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gu = self.rt.prepare(torch.cat([g, u], 0).contiguous(), unit=g.shape[0])
        self.w_down = self.rt.prepare(tensors["down.weight"])

    def forward(self, x, ctx):
        rt, s = self.rt, self.spec
        with rt.stage("ffn_gateup"):
            a = rt.ops.clamped_glu(rt.linear(rt.dense(x), self.w_gu), s.limit, s.alpha, rt.dtype)
        return rt.linear(a, self.w_down)


register("ffn", "gated_mlp", GatedMLP)
register("ffn", "clamped_glu", ClampedGLU)
