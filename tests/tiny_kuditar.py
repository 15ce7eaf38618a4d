"""Tiny Kuditar configurations of the tests.

A: a pair with a window and kept first positions, an attention layer that shares its values, a pair with runs, a second
   and a third attention layer that blend their values with the first one's; dense and routed feed-forwards.
B: values that are often equal made different and values that are often one made otherwise: the pair with runs first; an
   attention layer that shares nothing, turned over a part of its head only and without a cap; as many key heads as query
   heads in one layer, one key head in another; a window with no kept positions; a window of one page; no turn at all in a
   windowed branch; one, two and five taps; a bottleneck of three features, tau of one; one expert used of three, all of
   four used; a layer without a feed-forward; an embedding scale of one; a frequency divisor of one and of 2.5.
C: sizes in whole tiles of the matrix cores (heads of 64 and 128, values as wide as keys, states of 64 and 128 rows),
   sequences of a few hundred tokens, windows and runs of 64 and 96.
D: sizes that are multiples of nothing (width 100, vocabulary 97, heads of 10, 6 and 14, values of 6 and 22, an expert
   width of 12), a run of one position, a window of one, more kept positions than the window is wide.

``write_tiny`` draws the weights and then sets the few vectors whose scale matters to values that make the mechanisms
show: decays from almost none to fast (``A_log`` from -6 to 1 over the heads), step-size biases between -3 and 1, sinks
between -2 and 3, blending shares between 0.2 and 0.8, decay biases that spread the channels' decays between 0.5 and
almost 1, and corrections of the router's scores large enough to change which experts are chosen.
"""
import os

import torch

from gesso_amd.config import (ChannelDecayConfig, DeltaRuleConfig, DenseFFConfig, GatedAttentionConfig, KuditarConfig,
                              KuditarLayer, PairConfig, RunAttentionConfig, SigmoidMoEConfig, Turn, WindowedAttentionConfig)
from gesso_amd.weights import write_model_folder

STD = 0.12


def attention(heads, kv_heads, dim, vdim, scale, mlp, softcap=None, rot=None, v_mix=False):
    return KuditarLayer("attention", GatedAttentionConfig(heads, kv_heads, dim, vdim, scale, softcap, rot, v_mix), mlp)


def windowed(left, right, mlp):
    """``left``: heads, kv_heads, dim, vdim, scale, softcap, rot, window, keep_first; ``right``: heads, kv_heads, dim, vdim, conv."""
    return KuditarLayer("parallel", PairConfig(WindowedAttentionConfig(*left), DeltaRuleConfig(*right)), mlp)


def runs(left, right, mlp):
    """``left``: heads, kv_heads, dim, vdim, scale, run; ``right``: heads, dim, vdim, tau, rank."""
    h, g, d, vd, scale, run = left
    return KuditarLayer("parallel_2", PairConfig(RunAttentionConfig(h, g, d, vd, scale, None, None, run),
                                                 ChannelDecayConfig(*right)), mlp)


def dense(ff, limit):
    return DenseFFConfig(ff, limit)


def moe(experts, top, scale, ff, limit):
    return SigmoidMoEConfig(experts, top, scale, ff, limit)


KD_A = KuditarConfig(vocab=211, width=96, norm_eps=1e-6, embedding_scale=9.0, max_position=1024, layers=(
    windowed((4, 2, 24, 16, 0.2, 20.0, Turn(1e5, 24), 40, 6), (4, 2, 16, 24, 4), dense(80, 1.5)),
    attention(6, 2, 32, 16, 0.18, moe(6, 2, 2.0, 40, 2.0), 25.0, Turn(2e4, 16, 4.0), True),
    runs((4, 2, 16, 40, 0.25, 28), (3, 16, 24, 8.0, 8), moe(5, 2, 1.5, 24, 1.0)),
    attention(4, 2, 40, 16, 0.15, moe(6, 2, 2.0, 40, 2.0), 25.0, Turn(2e4, 16, 4.0), True),
    attention(2, 2, 16, 16, 0.2, dense(48, 2.0), 30.0, Turn(1e4, 16), True)))

KD_B = KuditarConfig(vocab=150, width=64, norm_eps=1e-5, embedding_scale=1.0, max_position=512, layers=(
    runs((3, 3, 8, 8, 0.3, 19), (2, 24, 8, 1.0, 3), None),
    attention(4, 1, 24, 12, 0.2, moe(3, 1, 1.0, 16, 0.7), None, Turn(100.0, 8), False),
    windowed((2, 2, 16, 24, 0.25, None, None, 16, 0), (6, 1, 8, 12, 1), moe(4, 4, 3.0, 24, 3.0)),
    windowed((4, 1, 12, 8, 0.3, 8.0, Turn(3e4, 6, 2.5), 33, 5), (2, 2, 12, 20, 5), dense(40, 0.8)),
    runs((2, 1, 12, 16, 0.3, None), (4, 8, 16, 3.0, 5), dense(24, 4.0)),
    windowed((2, 1, 8, 8, 0.35, 50.0, Turn(1e4, 8), 500, 3), (3, 3, 8, 8, 2), None)))

KD_C = KuditarConfig(vocab=320, width=128, norm_eps=1e-6, embedding_scale=11.3, max_position=1024, layers=(
    windowed((4, 2, 64, 64, 0.125, 30.0, Turn(5e5, 64), 96, 16), (2, 2, 64, 64, 4), moe(8, 2, 2.5, 64, 2.0)),
    attention(4, 2, 128, 128, 0.09, moe(8, 2, 2.5, 64, 2.0), 30.0, Turn(1e4, 64, 8.0), True),
    runs((4, 1, 64, 64, 0.125, 64), (2, 128, 128, 16.0, 16), dense(256, 1.5)),
    attention(4, 2, 128, 128, 0.09, moe(8, 4, 1.0, 32, 2.0), 30.0, Turn(1e4, 64, 8.0), True)))

KD_D = KuditarConfig(vocab=97, width=100, norm_eps=1e-4, embedding_scale=3.0, max_position=384, layers=(
    attention(5, 5, 10, 6, 0.3, moe(3, 2, 0.5, 12, 1.0), 5.0, Turn(3e4, 6, 1.5), True),
    runs((3, 1, 6, 22, 0.4, 1), (5, 6, 14, 2.0, 7), moe(7, 3, 2.5, 12, 0.5)),
    windowed((2, 1, 14, 10, 0.25, 15.0, Turn(1e4, 14), 1, 0), (5, 1, 10, 6, 3), dense(36, 2.5)),
    attention(5, 5, 6, 6, 0.4, None, None, None, True),
    windowed((3, 3, 10, 10, 0.3, None, Turn(500.0, 2), 7, 11), (2, 2, 14, 22, 4), None)))

CONFIGS = {"A": (KD_A, 80), "B": (KD_B, 81), "C": (KD_C, 82), "D": (KD_D, 83)}


def sharpen(tensors: dict, seed: int) -> dict:
    """The drawn tensors with the vectors whose scale matters set (see the module's text); keeps every type."""
    g = torch.Generator().manual_seed(seed)
    out = dict(tensors)
    for name, t in tensors.items():
        n = t.numel()
        if name.endswith(".A_log"):
            v = torch.linspace(-6.0, 1.0, n) if n > 1 else torch.tensor([-2.0])
        elif name.endswith(".dt_bias"):
            v = torch.rand(n, generator=g) * 4.0 - 3.0
        elif name.endswith(".sink"):
            v = torch.rand(n, generator=g) * 5.0 - 2.0
        elif name.endswith(".vmix"):
            v = torch.rand(n, generator=g) * 0.6 + 0.2
        elif name.endswith(".a2.b"):
            v = torch.rand(n, generator=g) * 6.0
        elif name.endswith(".correction"):
            v = 0.3 * torch.randn(n, generator=g)
        elif name.endswith(".router"):
            v = t.float() * 4.0
        elif name.endswith(".conv"):
            v = t.float() * 4.0
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
    d = os.path.join(root, f"kuditar_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(d, "model.safetensors")):
        write_folder(d, cfg, seed, dtype)
    return d
