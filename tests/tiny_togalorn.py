"""Tiny Togalorn configurations of the tests.

A: a state-space layer, an attention layer and another state-space layer in a loop of two passes, then a state-space
   layer; norms in three parts; three taps on every mixer's input; identity experts and a shared expert.
B: values that are often equal made different and values that are often one made otherwise: the loop in the middle
   (layers 1 .. 2, two passes, an attention layer inside it, so every pass keeps pages of its own); a layer without a
   feed-forward; one norm part and one group of B and C in one layer, as many groups as heads in another; two, three and
   five taps; one expert used of three, all of four used; no identity experts; no shared expert in one layer; the
   unrotated part narrower and wider than the rotated one; value heads wider than keys; an embedding scale of 1.
C: sizes in whole tiles of the matrix cores (heads of 64, latents of 128 and 256, states of 64 and 128), no loop at all,
   sequences of a few hundred tokens.
D: sizes that are multiples of nothing (width 100, vocabulary 97, heads of 10, 6 and 14, a state of 7, an expert width
   of 12), a head without any unrotated part, a loop of one pass over all layers, one tap, no convolution on the state-space
   mixer beyond its own single tap.

``write_tiny`` draws the weights and then sets the few vectors whose scale matters to values that make the mechanisms
show: state decays from almost none to fast (``A_log`` from -7 to 0.5 over the heads), step-size biases between -3 and 1,
skips around 1, and corrections of the router's scores large enough to change which experts are chosen.
"""
import os

import torch

from gesso_amd.config import (ExpertConfig, LatentMixerConfig, LoopConfig, Mamba2MixerConfig, MoEConfig, TogalornConfig,
                              TogalornLayer)
from gesso_amd.weights import write_model_folder

STD = 0.12


def mamba(heads, vdim, state, groups, norm_groups, conv, mlp):
    return TogalornLayer("mamba2", Mamba2MixerConfig(heads, vdim, state, groups, norm_groups, conv), mlp)


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, mlp):
    return TogalornLayer("latent_attention", LatentMixerConfig(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base), mlp)


def moe(experts, top, identity, ff, limit, shared=None):
    return MoEConfig(experts, top, identity, ExpertConfig(ff, limit) if experts else None,
                     None if shared is None else ExpertConfig(*shared))


TG_A = TogalornConfig(vocab=211, width=96, norm_eps=1e-6, norm_groups=3, embedding_scale=9.8, canon_taps=3,
                      loop=LoopConfig(0, 3, 2), max_position=512, layers=(
    mamba(4, 16, 24, 2, 2, 4, moe(6, 2, 2, 40, 1.0, (48, 2.0))),
    latent(3, 16, 16, 16, 40, 48, 0.18, 5e5, moe(5, 2, 1, 24, 1.5, (32, 1.0))),
    mamba(3, 24, 16, 1, 3, 3, moe(6, 2, 2, 40, 1.0, (48, 2.0))),
    mamba(4, 16, 24, 2, 2, 4, moe(6, 2, 2, 40, 1.0, (48, 2.0)))))

TG_B = TogalornConfig(vocab=150, width=64, norm_eps=1e-5, norm_groups=1, embedding_scale=1.0, canon_taps=2,
                      loop=LoopConfig(1, 3, 2), max_position=512, layers=(
    latent(2, 8, 16, 24, 24, 32, 0.25, 1e4, None),
    latent(1, 24, 8, 16, 16, 36, 0.2, 100.0, moe(3, 1, 0, 16, 0.7, None)),
    mamba(2, 12, 8, 2, 1, 5, moe(4, 4, 0, 24, 3.0, (16, 0.5))),
    mamba(6, 8, 12, 3, 6, 2, moe(2, 3, 2, 8, 1.0, (40, 4.0)))))

TG_C = TogalornConfig(vocab=320, width=128, norm_eps=1e-6, norm_groups=4, embedding_scale=11.3, canon_taps=4, loop=None,
                      max_position=1024, layers=(
    mamba(4, 64, 64, 1, 2, 4, moe(8, 2, 2, 64, 1.0, (64, 2.0))),
    latent(4, 64, 64, 64, 64, 128, 0.09, 5e5, moe(8, 2, 2, 64, 1.0, (64, 2.0))),
    mamba(2, 128, 128, 2, 1, 4, moe(8, 2, 2, 64, 1.0, (64, 2.0))),
    latent(2, 64, 64, 128, 128, 256, 0.09, 1e4, moe(8, 4, 0, 32, 2.0, None))))

TG_D = TogalornConfig(vocab=97, width=100, norm_eps=1e-4, norm_groups=5, embedding_scale=3.0, canon_taps=1,
                      loop=LoopConfig(0, 3, 1), max_position=384, layers=(
    mamba(5, 10, 7, 5, 2, 1, moe(3, 2, 1, 12, 1.0, (20, 1.0))),
    latent(5, 0, 6, 14, 18, 22, 0.3, 3e4, moe(7, 3, 3, 12, 0.5, (36, 2.5))),
    latent(2, 18, 2, 6, 10, 30, 0.2, 1e4, None)))

CONFIGS = {"A": (TG_A, 60), "B": (TG_B, 61), "C": (TG_C, 62), "D": (TG_D, 63)}


def sharpen(tensors: dict, seed: int) -> dict:
    """The drawn tensors with the vectors whose scale matters set (see the module's text); keeps every type."""
    g = torch.Generator().manual_seed(seed)
    out = dict(tensors)
    for name, t in tensors.items():
        n = t.numel()
        if name.endswith(".A_log"):
            v = torch.linspace(-7.0, 0.5, n) if n > 1 else torch.tensor([-3.0])
        elif name.endswith(".dt_bias"):
            v = torch.rand(n, generator=g) * 4.0 - 3.0
        elif name.endswith(".D"):
            v = 1.0 + 0.3 * torch.randn(n, generator=g)
        elif name.endswith(".correction"):
            v = 0.4 * torch.randn(n, generator=g)
        elif name.endswith(".router"):
            v = t.float() * 4.0
        elif name == "loop.step":
            v = t.float() * 5.0
        else:
            continue
        out[name] = v.reshape(t.shape).to(t.dtype)
    return out


def write_folder(out_dir: str, cfg, seed: int, dtype=torch.float32, std: float = STD) -> str:
    """A model folder with drawn and sharpened weights."""
    from safetensors.torch import load_file

    from gesso_amd.weights import write_safetensors
    write_model_folder(out_dir, cfg, seed, dtype, std=std)
    path = os.path.join(out_dir, "model.safetensors")
    write_safetensors(path, sharpen(load_file(path), seed), metadata={"format": "pt", "seed": str(seed)})
    return out_dir


def write_tiny(root: str, name: str, dtype=torch.float32) -> str:
    cfg, seed = CONFIGS[name]
    d = os.path.join(root, f"togalorn_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(d, "model.safetensors")):
        write_folder(d, cfg, seed, dtype)
    return d
