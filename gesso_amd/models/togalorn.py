"""Togalorn as a composition of parts: configuration -> model as data.

A decoder whose blocks have one norm (an RMS norm in equal parts of the row, ``GroupRMSNormSpec``) that both sub-layers
read, the mixer through a causal convolution over time laid on its input, and add both results to the stream
(``SharedNormBlockSpec``).  A block's mixer is attention through low-rank latents with a shared rotated key part,
neighbouring rotation pairs and a gate for every output feature (``LatentAttentionSpec``), or a state-space mixer whose
decay and step size depend on the token (``StateSpaceSpec``).  The feed-forward is a mixture of experts chosen by a
softmax router with a correction of the choice, identity experts and a shared expert (``RoutedMoESpec``).  A run of
layers may be passed through several times with the same weights, each pass with its own cache; before every pass the
stream is mixed with the embedding output again (``ReentrySpec``).  The embedding rows are scaled; the head is untied.

This file holds what is Togalorn's own: the tensor names and the way the typed configuration fills the parts' sizes.
Layers may differ from one another in every size.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.spec import (GroupRMSNormSpec, LatentAttentionSpec, LayerCall, ModelSpec, NoPositionSpec, ReentrySpec,
                           RopeSpec, RoutedMoESpec, SharedNormBlockSpec, StateSpaceSpec)
from ..config.togalorn import ARCHITECTURE, LATENT, TogalornConfig

ACTIVATION_SLOPE = 1.702     # an expert's gate is g * sigmoid(1.702 g)


def _latent(mx, W, eps, p, max_position):
    position = NoPositionSpec() if mx.rot_dim == 0 else RopeSpec(
        head_dim=mx.rot_dim, rotary_dim=mx.rot_dim, theta=mx.rot_base, max_position=max_position, layout="interleaved")
    spec = LatentAttentionSpec(hidden=W, n_heads=mx.heads, plain_dim=mx.dim, rot_dim=mx.rot_dim, value_dim=mx.vdim,
                               q_rank=mx.q_rank, kv_rank=mx.kv_rank, scale=mx.scale, eps=eps, position=position,
                               window=None, gated=True, gate_each=True)
    names = {local: p + stored for local, stored in (
        ("q_down.weight", "dq"), ("q_norm.weight", "dq.norm"), ("q_up.weight", "uq"), ("kv_down.weight", "dkv"),
        ("kv_norm.weight", "dkv.norm"), ("k_up.weight", "uk"), ("v_up.weight", "uv"), ("gate.weight", "g"),
        ("out.weight", "o"))}
    return spec, names


def _state_space(mx, W, eps, p):
    spec = StateSpaceSpec(hidden=W, n_heads=mx.heads, head_dim=mx.vdim, state=mx.state, groups=mx.groups,
                          norm_groups=mx.norm_groups, conv_taps=mx.conv, eps=eps)
    names = {local: p + stored for local, stored in (
        ("in_proj.weight", "in"), ("conv.weight", "conv"), ("conv.bias", "conv.b"), ("dt_bias", "dt_bias"),
        ("A_log", "A_log"), ("D", "D"), ("norm.weight", "norm"), ("out_proj.weight", "o"))}
    return spec, names


def _moe(m, W, p):
    ex = m.expert
    spec = RoutedMoESpec(hidden=W, n_experts=m.experts, top=m.top, expert_ff=ex.ff if ex is not None else 1,
                         limit=ex.limit if ex is not None else 1.0, n_identity=m.identity, alpha=ACTIVATION_SLOPE,
                         correction=True, shared_ff=None if m.shared is None else m.shared.ff,
                         shared_limit=None if m.shared is None else m.shared.limit)
    names = {"router.weight": p + "router", "router.correction": p + "correction"}
    for e in range(m.experts):
        for w in ("gate", "up", "down"):
            names[f"experts.{e}.{w}.weight"] = p + f"e{e}.{w}"
    if m.shared is not None:
        for w in ("gate", "up", "down"):
            names[f"shared.{w}.weight"] = p + f"shared.{w}"
    return spec, names


def run_order(cfg: TogalornConfig):
    """``(the layers in the order they run, the places in that order where a pass of the loop begins)``."""
    n = len(cfg.layers)
    if cfg.loop is None:
        return list(range(n)), []
    a, b, times = cfg.loop.start, cfg.loop.stop, cfg.loop.times
    order, starts = list(range(a)), []
    for _ in range(times):
        starts.append(len(order))
        order += list(range(a, b))
    return order + list(range(b, n)), starts


def togalorn_spec(cfg: TogalornConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    norm = GroupRMSNormSpec(size=W, eps=eps, groups=cfg.norm_groups)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == LATENT:
            mixer, local = _latent(layer.mixer, W, eps, p + "mix.", cfg.max_position)
        else:
            mixer, local = _state_space(layer.mixer, W, eps, p + "mix.")
        names = {"norm.weight": p + "norm1"}
        names.update({"mixer." + k: v for k, v in local.items()})
        if cfg.canon_taps is not None:
            names["input_conv.weight"] = p + "canon1"
        ffn = None
        if layer.mlp is not None:
            ffn, local = _moe(layer.mlp, W, p + "mlp.")
            names.update({"ffn." + k: v for k, v in local.items()})
        blocks.append(SharedNormBlockSpec(mixer=mixer, norm=norm, ffn=ffn, input_taps=cfg.canon_taps, names=names))
    order, starts = run_order(cfg)
    names = {"embed": "embed", "final_norm.weight": "final.norm", "head": "head"}
    reentry = None
    if starts:
        reentry = ReentrySpec(at=tuple(starts))
        names.update({"reentry.weight": "loop.in", "reentry.step": "loop.step"})
    return ModelSpec(architecture=ARCHITECTURE, hidden=W, vocab=cfg.vocab, blocks=tuple(blocks),
                     schedule=tuple(LayerCall(i) for i in order), final_norm=norm, tie_embeddings=False,
                     max_position=cfg.max_position, names=names, embed_scale=cfg.embedding_scale, reentry=reentry)


register_architecture(ARCHITECTURE, TogalornConfig.from_dict, togalorn_spec, TogalornConfig.to_json)
