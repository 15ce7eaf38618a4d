"""A mixture of gated feed-forwards chosen by a router over the token's features.

    z = W_r x  (float32),  s = softmax(z) over all ``E + I`` router outputs  (``score = "sigmoid"``: s = sigmoid(z))
    chosen: the ``top`` outputs with the largest ``s + correction``;  weights: ``s`` of the chosen / (their sum + 1e-20)
    (``renormalize = False``: ``s`` of the chosen as they are), times ``route_scale``
    expert e < E:   W_down[e] (g sigmoid(alpha g) (u + 1)),  g = min(W_gate[e] x, limit),  u = clamp(W_up[e] x, -limit, limit)
    expert e >= E:  x itself (an identity expert: it has no tensors)
    y = sum over the chosen of weight * expert(x)  +  shared(x)   (an expert of its own width and limit, for every token)

The experts' weights are stacked at load, gate over up: ``(E, 2F, H)`` and ``(E, H, F)``; the shared expert's gate and
up rows are laid side by side, so one product gives both.  Router, softmax, choice and weights are float32.
"""
from __future__ import annotations

import torch

from .base import MATRIX, VECTOR, Part, TensorSpec
from .registry import register


class RoutedMoE(Part):
    graph_safe = True
    stage, out_stage = "moe_ffn", "ffn_down"

    @staticmethod
    def tensor_specs(spec):
        H, F, EA = spec.hidden, spec.expert_ff, spec.n_experts + spec.n_identity
        out = {"router.weight": TensorSpec((EA, H), MATRIX)}
        if spec.correction:
            out["router.correction"] = TensorSpec((EA,), VECTOR)
        for e in range(spec.n_experts):
            out[f"experts.{e}.gate.weight"] = TensorSpec((F, H), MATRIX)
            out[f"experts.{e}.up.weight"] = TensorSpec((F, H), MATRIX)
            out[f"experts.{e}.down.weight"] = TensorSpec((H, F), MATRIX)
        if spec.shared_ff is not None:
            out["shared.gate.weight"] = TensorSpec((spec.shared_ff, H), MATRIX)
            out["shared.up.weight"] = TensorSpec((spec.shared_ff, H), MATRIX)
            out["shared.down.weight"] = TensorSpec((H, spec.shared_ff), MATRIX)
        return out

    def bind(self, tensors):
        s, rt = self.spec, self.rt
        router = self.router = tensors["router.weight"].contiguous()
        self.correction = tensors.get("router.correction")
        E = s.n_experts
        gus = [torch.cat([tensors[f"experts.{e}.gate.weight"], tensors[f"experts.{e}.up.weight"]], 0) for e in range(E)]
        downs = [tensors[f"experts.{e}.down.weight"] for e in range(E)]
        if len({w.dtype for w in gus + downs}) > 1:
            gus, downs = [w.float() for w in gus], [w.float() for w in downs]
        dev, dt = router.device, (gus[0].dtype if E else router.dtype)
        self.gate_up = torch.stack(gus, 0).contiguous() if E else torch.zeros((0, 2 * s.expert_ff, s.hidden), dtype=dt, device=dev)
        self.down = torch.stack(downs, 0).contiguous() if E else torch.zeros((0, s.hidden, s.expert_ff), dtype=dt, device=dev)
        self.w_sgu = self.w_sdown = None
        if s.shared_ff is not None:
            g, u = tensors["shared.gate.weight"], tensors["shared.up.weight"]
            if g.dtype != u.dtype:
                g, u = g.float(), u.float()
            self.w_sgu = rt.prepare(torch.cat([g, u], 0).contiguous(), unit=g.shape[0])
            self.w_sdown = rt.prepare(tensors["shared.down.weight"])

    def forward(self, x, ctx):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        x = rt.dense(x)
        with rt.stage("ffn_router"):
            choice, weight = ops.moe_router(x, self.router, self.correction, s.top, score=getattr(s, "score", "softmax"),
                                            renormalize=getattr(s, "renormalize", True),
                                            scale=getattr(s, "route_scale", 1.0))
        shared = None
        if self.w_sgu is not None:
            with rt.stage("ffn_shared"):
                limit = s.limit if s.shared_limit is None else s.shared_limit
                shared = rt.linear(ops.clamped_glu(rt.linear(x, self.w_sgu), limit, s.alpha, rt.dtype), self.w_sdown)
        # once the pairs outnumber the experts twice over, sorting them by expert reads less: each expert's weights
        # once, instead of once a pair (the option "token" keeps the token-by-token kernels for every step)
        if (x.shape[0] * s.top >= 2 * s.n_experts and rt.options.routed_experts != "token"
                and ops.moe_routed_grouped_ok(x, self.gate_up, self.down)):
            return ops.moe_routed_grouped(x, choice, weight, self.gate_up, self.down, s.limit, s.alpha, shared=shared)
        return ops.moe_routed(x, choice, weight, self.gate_up, self.down, s.limit, s.alpha, shared=shared)


register("ffn", "routed_moe", RoutedMoE)
