"""Position encodings as tables: what the attention kernels need is ``cos``, ``sin``, ``rotary_dim`` and ``layout``.

Rotary; pair ``i`` is ``(i, i + rotary_dim/2)`` (``layout = "half"``) or ``(2i, 2i + 1)`` (``"interleaved"``), its
angle ``pos * theta^(-2i/rotary_dim)`` (reference ``src/Operators/cpu.jl:357-371``; LFM2 has ``interleaved=false``,
``src/Inference/architecture_spec.jl:66``).  A kernel that is written for one layout is not used for the other: the
mixer asks ``layout`` before it takes a fused route.  Angles, cosines and
sines are computed on the host in float64 and stored as float32, one table per distinct spec.
Another encoding (scaled frequencies, another theta per layer) is another class that fills
the same three attributes; ``rotary_dim = 0`` means none.
"""
from __future__ import annotations

import torch

from .base import Part
from .registry import register


def rope_tables(rotary_dim: int, theta: float, max_position: int, divisor: float = 1.0):
    """``divisor``: every frequency is divided by it (positions stretched evenly, "linear scaling")."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    inv_freq = torch.tensor(float(theta), dtype=torch.float64) ** (-2.0 * i / rotary_dim) / float(divisor)
    ang = torch.arange(max_position, dtype=torch.float64)[:, None] * inv_freq[None, :]
    return torch.cos(ang).to(torch.float32), torch.sin(ang).to(torch.float32)


class Rope(Part):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.rotary_dim % 2 or not 0 < spec.rotary_dim <= spec.head_dim:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even and within the head width {spec.head_dim}")
        self.rotary_dim = spec.rotary_dim
        self.layout = getattr(spec, "layout", "half")
        if self.layout not in rt.ops.ROPE_LAYOUTS:
            raise ValueError(f"rotation pairs are laid out 'half' or 'interleaved', not {self.layout!r}")

        def make():
            cos, sin = rope_tables(spec.rotary_dim, spec.theta, spec.max_position, divisor)
            return cos.to(rt.device), sin.to(rt.device)

        divisor = float(getattr(spec, "frequency_divisor", 1.0))
        self.cos, self.sin = rt.shared(("rope", spec.rotary_dim, float(spec.theta), spec.max_position, divisor), make)


def scaled_rope_tables(spec):
    """cos and sin tables of a :class:`~gesso_amd.config.spec.ScaledRopeSpec` (see there for the rule): pairs that turn
    often keep their frequency, slow pairs are slowed by ``factor``, those between are blended, and both tables carry
    the amplitude factor.  float64 on the host, stored as float32."""
    import math
    dims, theta = spec.rotary_dim, float(spec.theta)
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = torch.tensor(theta, dtype=torch.float64) ** (-2.0 * i / dims)
    amplitude = 1.0
    if spec.factor is not None:
        def pair_of(turns):
            return dims * math.log(float(spec.original) / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
        lo = max(math.floor(pair_of(float(spec.fast))), 0)
        hi = min(math.ceil(pair_of(float(spec.slow))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        freq = freq / float(spec.factor) * ramp + freq * (1.0 - ramp)
        amplitude = float(spec.amplitude_slope) * math.log(float(spec.factor)) + 1.0
    ang = torch.arange(spec.max_position, dtype=torch.float64)[:, None] * freq[None, :]
    return (torch.cos(ang) * amplitude).to(torch.float32), (torch.sin(ang) * amplitude).to(torch.float32)


class ScaledRope(Part):
    """Rotation with slowed pairs and an amplitude: the same three attributes as :class:`Rope`, other tables."""

    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.rotary_dim % 2 or not 0 <= spec.rotary_dim <= spec.head_dim:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even and within the head width {spec.head_dim}")
        self.rotary_dim = spec.rotary_dim
        self.layout = spec.layout
        if self.layout not in rt.ops.ROPE_LAYOUTS:
            raise ValueError(f"rotation pairs are laid out 'half' or 'interleaved', not {self.layout!r}")
        self.cos = self.sin = None
        if spec.rotary_dim:
            def make():
                cos, sin = scaled_rope_tables(spec)
                return cos.to(rt.device), sin.to(rt.device)

            key = ("scaled_rope", spec.rotary_dim, float(spec.theta), spec.max_position, spec.factor, float(spec.original),
                   float(spec.fast), float(spec.slow), float(spec.amplitude_slope))
            self.cos, self.sin = rt.shared(key, make)


def stretched_rope_tables(spec):
    """cos and sin tables of a :class:`~gesso_amd.config.spec.StretchedRopeSpec` (see there for the rule): a pair keeps
    its frequency, gets it divided by ``factor``, or a blend of both, by where its wavelength stands against
    ``original / high`` and ``original / low``.  float64 on the host, stored as float32."""
    import math
    dims, theta = spec.rotary_dim, float(spec.theta)
    freq = [theta ** (-2.0 * i / dims) for i in range(dims // 2)]
    if spec.factor is not None:
        factor, low, high, original = float(spec.factor), float(spec.low), float(spec.high), float(spec.original)
        for i, f in enumerate(freq):
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                freq[i] = f / factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                freq[i] = (1.0 - s) * f / factor + s * f
    ang = torch.arange(spec.max_position, dtype=torch.float64)[:, None] * torch.tensor(freq, dtype=torch.float64)[None, :]
    return torch.cos(ang).to(torch.float32), torch.sin(ang).to(torch.float32)


class StretchedRope(Part):
    """Rotation with frequencies stretched by wavelength: the same three attributes as :class:`Rope`, other tables."""

    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if spec.rotary_dim % 2 or not 0 < spec.rotary_dim <= spec.head_dim:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even and within the head width {spec.head_dim}")
        self.rotary_dim = spec.rotary_dim
        self.layout = spec.layout
        if self.layout not in rt.ops.ROPE_LAYOUTS:
            raise ValueError(f"rotation pairs are laid out 'half' or 'interleaved', not {self.layout!r}")

        def make():
            cos, sin = stretched_rope_tables(spec)
            return cos.to(rt.device), sin.to(rt.device)

        key = ("stretched_rope", spec.rotary_dim, float(spec.theta), spec.max_position, spec.factor, float(spec.original),
               float(spec.low), float(spec.high))
        self.cos, self.sin = rt.shared(key, make)


class NoPosition(Part):
    graph_safe = True
    rotary_dim = 0
    layout = "half"
    cos = None
    sin = None


register("position", "rope", Rope)
register("position", "scaled_rope", ScaledRope)
register("position", "stretched_rope", StretchedRope)
register("position", "none", NoPosition)
