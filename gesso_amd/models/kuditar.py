"""Kuditar as a composition of parts: configuration -> model as data.

A decoder of pre-norm blocks with layer norms (weight and bias): ``x += mixer(ln1(x)); x += ff(ln2(x))``.  A block's
mixer is one of three.  ``attention``: grouped-query softmax attention whose q and k are turned over their first
features (every frequency divided by one factor) and then divided by their root mean square, with capped scores, values
blended with the values of the first such layer, and a sigmoid gate on the heads (``AttentionSpec``).  ``parallel``: half
the sum of two branches, each normed over the model width (``MixerPairSpec`` with branch norms): softmax attention with
biases, weighted head norms, a window that keeps the sequence's first positions and a learned sink per head; and the
gated delta rule (``GatedDeltaSpec``).  ``parallel_2``: the same sum of attention over runs of positions, without turn
or cap, and linear attention with a decay per key channel (``GatedLinearSpec``).  The feed-forward is a clamped gated
unit (``ClampedGLUSpec``) or a mixture of such units chosen by sigmoid scores (``RoutedMoESpec``).  The embedding rows
are scaled; the embedding table is the head.

This file holds what is Kuditar's own: the tensor names and the way the typed configuration fills the parts' sizes.
Layers may differ from one another in every size.
"""
from __future__ import annotations

from ..config.kuditar import (ARCHITECTURE, ATTENTION, PARALLEL, DenseFFConfig, KuditarConfig, complete)
from ..config.registry import register_architecture
from ..config.spec import (AttentionSpec, BlockSpec, ClampedGLUSpec, GatedDeltaSpec, GatedLinearSpec, LayerCall,
                           LayerNormSpec, MixerPairSpec, ModelSpec, NoPositionSpec, RMSNormSpec, RopeSpec, RoutedMoESpec)

ACTIVATION_SLOPE = 1.702     # a gated unit's gate is g * sigmoid(1.702 g)
UNIT_EPS = 1e-6              # under the root where the delta rule makes q and k unit vectors


def _position(mx, max_position):
    if getattr(mx, "rot", None) is None:
        return NoPositionSpec()
    return RopeSpec(head_dim=mx.dim, rotary_dim=mx.rot.dims, theta=mx.rot.base, max_position=max_position,
                    frequency_divisor=mx.rot.factor)


def _gated_attention(mx, W, eps, p, max_position):
    spec = AttentionSpec(hidden=W, n_heads=mx.heads, n_kv_heads=mx.kv_heads, head_dim=mx.dim,
                         position=_position(mx, max_position), qk_norm=RMSNormSpec(mx.dim, eps), qk_norm_weight=False,
                         scale=mx.scale, value_dim=mx.vdim, softcap=mx.softcap, out_gate="sigmoid", value_mix=mx.v_mix)
    names = {"q_proj.weight": p + "q", "k_proj.weight": p + "k", "v_proj.weight": p + "v", "gate_proj.weight": p + "g",
             "out_proj.weight": p + "o"}
    if mx.v_mix:
        names["value_mix"] = p + "vmix"
    return spec, names


def _biased_attention(mx, W, eps, p, max_position, windowed: bool):
    """The left side of a pair: biases on q, k and v, weighted head norms; a window with kept first positions and a
    sink of the head's own, or runs of positions."""
    spec = AttentionSpec(hidden=W, n_heads=mx.heads, n_kv_heads=mx.kv_heads, head_dim=mx.dim,
                         position=_position(mx, max_position), qk_norm=RMSNormSpec(mx.dim, eps), bias=True,
                         out_bias=False, scale=mx.scale, value_dim=mx.vdim, softcap=mx.softcap,
                         window=mx.window if windowed else None,
                         keep_first=(mx.keep_first if mx.window is not None else 0) if windowed else 0,
                         head_sinks=windowed, chunk=None if windowed else mx.run)
    names = {"q_proj.weight": p + "q", "k_proj.weight": p + "k", "v_proj.weight": p + "v", "q_proj.bias": p + "q.b",
             "k_proj.bias": p + "k.b", "v_proj.bias": p + "v.b", "q_norm.weight": p + "q.norm",
             "k_norm.weight": p + "k.norm", "out_proj.weight": p + "o"}
    if windowed:
        names["sinks"] = p + "sink"
    return spec, names


def _delta(mx, W, eps, p):
    spec = GatedDeltaSpec(hidden=W, n_heads=mx.heads, qk_heads=mx.kv_heads, key_dim=mx.dim, value_dim=mx.vdim,
                          conv_taps=mx.conv, eps=eps, unit_eps=UNIT_EPS)
    names = {"q_proj.weight": p + "q", "k_proj.weight": p + "k", "v_proj.weight": p + "v", "gate_proj.weight": p + "g",
             "beta_proj.weight": p + "b", "decay_proj.weight": p + "a", "q_conv.weight": p + "q.conv",
             "k_conv.weight": p + "k.conv", "v_conv.weight": p + "v.conv", "A_log": p + "A_log", "dt_bias": p + "dt_bias",
             "out_norm.weight": p + "norm", "out_proj.weight": p + "o"}
    return spec, names


def _channel_decay(mx, W, eps, p):
    spec = GatedLinearSpec(hidden=W, n_heads=mx.heads, key_dim=mx.dim, value_dim=mx.vdim, decay_rank=mx.rank, tau=mx.tau,
                           eps=eps)
    names = {"q_proj.weight": p + "q", "k_proj.weight": p + "k", "v_proj.weight": p + "v", "gate_proj.weight": p + "g",
             "decay_down.weight": p + "a1", "decay_up.weight": p + "a2", "decay_up.bias": p + "a2.b",
             "out_norm.weight": p + "norm", "out_proj.weight": p + "o"}
    return spec, names


def _pair(layer, W, eps, p, max_position):
    windowed = layer.type == PARALLEL
    left, lnames = _biased_attention(layer.mixer.left, W, eps, p + "left.", max_position, windowed)
    right, rnames = (_delta if windowed else _channel_decay)(layer.mixer.right, W, eps, p + "right.")
    spec = MixerPairSpec(left=left, right=right, left_scale=0.5, right_scale=0.5, branch_norm_eps=eps, hidden=W)
    names = {"left." + k: v for k, v in lnames.items()}
    names.update({"right." + k: v for k, v in rnames.items()})
    names.update({"left_norm.weight": p + "left.out", "right_norm.weight": p + "right.out"})
    return spec, names


def _feed_forward(m, W, p):
    if isinstance(m, DenseFFConfig):
        spec = ClampedGLUSpec(hidden=W, intermediate=m.ff, limit=m.limit, alpha=ACTIVATION_SLOPE)
        return spec, {"gate.weight": p + "gate", "up.weight": p + "up", "down.weight": p + "down"}
    spec = RoutedMoESpec(hidden=W, n_experts=m.experts, top=m.top, expert_ff=m.ff, limit=m.limit, alpha=ACTIVATION_SLOPE,
                         correction=True, score="sigmoid", renormalize=False, route_scale=m.scale)
    names = {"router.weight": p + "router", "router.correction": p + "correction"}
    for e in range(m.experts):
        for w in ("gate", "up", "down"):
            names[f"experts.{e}.{w}.weight"] = p + f"e{e}.{w}"
    return spec, names


def kuditar_spec(cfg: KuditarConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    norm = LayerNormSpec(size=W, eps=eps, bias=True)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == ATTENTION:
            mixer, local = _gated_attention(layer.mixer, W, eps, p + "mix.", cfg.max_position)
        else:
            mixer, local = _pair(layer, W, eps, p + "mix.", cfg.max_position)
        names = {"mixer_norm.weight": p + "norm1", "mixer_norm.bias": p + "norm1.b"}
        names.update({"mixer." + k: v for k, v in local.items()})
        ffn = None
        if layer.mlp is not None:
            ffn, local = _feed_forward(layer.mlp, W, p + "mlp.")
            names.update({"ffn." + k: v for k, v in local.items()})
            names.update({"ffn_norm.weight": p + "norm2", "ffn_norm.bias": p + "norm2.b"})
        blocks.append(BlockSpec(mixer=mixer, mixer_norm=norm, ffn=ffn, ffn_norm=norm if ffn is not None else None,
                                names=names))
    names = {"embed": "embed", "final_norm.weight": "final.norm", "final_norm.bias": "final.norm.b"}
    return ModelSpec(architecture=ARCHITECTURE, hidden=W, vocab=cfg.vocab, blocks=tuple(blocks),
                     schedule=tuple(LayerCall(i) for i in range(len(blocks))), final_norm=norm, tie_embeddings=True,
                     max_position=cfg.max_position, names=names, embed_scale=cfg.embedding_scale,
                     # (a file may hold the second norm of a layer without a feed-forward, or the share of a layer
                     # that blends nothing: nobody reads them)
                     ignored_tensors=(".norm2", ".norm2.b", ".vmix"))


register_architecture(ARCHITECTURE, KuditarConfig.from_dict, kuditar_spec, KuditarConfig.to_json, complete=complete)
