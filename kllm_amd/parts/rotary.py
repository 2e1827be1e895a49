"""Rotary position encoding, half-split pairing.

For pair (j, j + head_dim/2) of every head: angle = pos * theta^(-2j/head_dim),
computed in double; a' = a cos - b sin, b' = b cos + a sin
(backend/model.cu:170-184).  Keys are rotated before they are cached
(:1093-1100), so the cache never needs re-encoding.

Parameters: ``head_dim``, ``theta``.  No tensors.  ``prepare`` computes the
step's cos/sin tables once; every mixer that shares this part reads them.
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part


@register_part("position", "rotary")
class RotaryEncoding(Part):
    graph_safe = True
    records_launches = True


    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.head_dim = int(self.param("head_dim"))
        self.theta = float(self.param("theta"))
        if self.head_dim % 2:
            raise ValueError(f"rotary: head_dim {self.head_dim} must be even")

    def prepare(self, ctx):
        half = self.head_dim // 2
        cos = ctx.buf(f"rope.cos.{id(self)}", (ctx.n, half), torch.float32)
        sin = ctx.buf(f"rope.sin.{id(self)}", (ctx.n, half), torch.float32)
        K.rope_tables(cos, sin, ctx.positions[:ctx.n], self.head_dim, self.theta)
        ctx.scratch[("rotary", id(self))] = (cos, sin)

    def tables(self, ctx):
        return ctx.scratch[("rotary", id(self))]


def scaled_frequencies(dims, base, scaling=None):
    """Angle per position of each of the ``dims / 2`` rotated pairs, and the factor on cos and
    sin.  Pair i turns by f_i = base^(-2i/dims) a position.  ``scaling`` = (factor, original,
    fast, slow) stretches the slow pairs (YaRN): with dim(t) = dims ln(original / (2 pi t)) /
    (2 ln base), the pair at which a rotation takes original / t positions, lo = max(floor(dim(fast)),
    0), hi = min(ceil(dim(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    pair i turns by f_i / factor * r_i + f_i (1 - r_i), and cos and sin are multiplied by
    0.1 ln(factor) + 1.  All in double."""
    import math
    half = dims // 2
    freq = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if scaling is None:
        return freq, 1.0
    if scaling[0] == "by_wavelength":
        return wavelength_scaled(freq, *scaling[1:]), 1.0
    factor, original, fast, slow = (float(v) for v in scaling)

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), dims - 1)
    out = []
    for i, f in enumerate(freq):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def wavelength_scaled(freq, factor, low, high, original):
    """Frequencies slowed down by their wavelength l = 2 pi / f: kept where l < original / high,
    divided by ``factor`` where l > original / low, and between the two blended linearly in
    s = (original / l - low) / (high - low): (1 - s) f / factor + s f.  All in double."""
    import math
    factor, low, high, original = float(factor), float(low), float(high), float(original)
    out = []
    for f in freq:
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


@register_part("position", "rotary_scaled")
class ScaledRotaryEncoding(Part):
    """Rotation of the first ``rotary_dim`` elements of a head, neighbours paired ((2j, 2j + 1);
    ``interleaved`` False pairs (j, j + rotary_dim / 2)), with the frequencies of
    ``scaled_frequencies``.  A mixer reads ``rotary_dim`` and ``interleaved`` and applies the
    tables; angles are taken in double and the tables rounded to float32 once.

    Parameters: ``rotary_dim``, ``base``, ``scaling`` (None, (factor, original, fast, slow) for the
    stretch by pair index, or ("by_wavelength", factor, low, high, original) for the one of
    ``wavelength_scaled``), ``interleaved`` (default True).  No tensors of the checkpoint."""
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.rotary_dim = int(self.param("rotary_dim"))
        self.interleaved = bool(self.param("interleaved", True))
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"rotary_scaled: rotary_dim {self.rotary_dim} must be even and positive")
        scaling = self.param("scaling", None)
        freq, self.factor = scaled_frequencies(self.rotary_dim, float(self.param("base")),
                                               tuple(scaling) if scaling is not None else None)
        self._freq_host = freq
        self.freq = None           # float64 [rotary_dim / 2] on the device at the first step

    def prepare(self, ctx):
        if self.freq is None:
            self.freq = torch.tensor(self._freq_host, dtype=torch.float64, device=self.runtime.device)
            self.runtime.tensors_changed()
        half = self.rotary_dim // 2
        cos = ctx.buf(f"rope.cos.{id(self)}", (ctx.n, half), torch.float32)
        sin = ctx.buf(f"rope.sin.{id(self)}", (ctx.n, half), torch.float32)
        K.rope_tables_freq(cos, sin, ctx.positions[:ctx.n], self.freq, self.factor)
        ctx.scratch[("rotary", id(self))] = (cos, sin)

    def tables(self, ctx):
        return ctx.scratch[("rotary", id(self))]
