"""Rotary position encoding (pairs (i, i + rot/2)).

inv_freq[i] = 1 / theta ** (2 i / rot), built exactly as the reference builds it
(engine/model.py:132-135: int64 arange -> float, divided by the size, theta to
that power, in float32); angle = position * inv_freq in float32
(engine/model.py:138-152); out = x * cos + rotate_half(x) * sin (:126-129,155-161).
The reference casts cos and sin to the activation type before the multiply; here
they stay float32 and the result is rounded once.

A position encoding encodes heads in place (`encode`) and knows nothing of caches:
storing keys and values is the mixer's business.  An encoding that is a rotation by a
table of cosines and sines may also hand out that table (`rotary_table`), which lets a
mixer run the rotation inside its own fused kernels.
"""

from __future__ import annotations

import math

import torch

from ..kernels import lib as K
from .base import Part, register_position_encoding


@register_position_encoding("neox_rope")
class NeoxRope(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        rot = spec.rotary_dim
        if rot % 2:
            raise ValueError(f"rotary_dim {rot} must be even")
        exponent = torch.arange(0, rot, 2, dtype=torch.int64).to(torch.float32)
        self.inv_freq = (1.0 / (spec.theta ** (exponent / rot))).to(device)

    def rotary_table(self, ctx):
        """(rotated width, cosines and sines [T, width / 2, 2] of every token's angles): computed by
        the first layer of a step that asks and shared by all layers with the same rotation."""
        rot = self.spec.rotary_dim
        if not rot:
            return 0, None
        key = ("neox_rope", rot, self.spec.theta)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = K.rope_table(ctx.positions, self.inv_freq)
        return rot, table

    def encode(self, ctx, x: torch.Tensor, num_heads: int, head_dim: int) -> None:
        """Rotate the first `num_heads` heads of every row of `x` in place."""
        rot, table = self.rotary_table(ctx)
        if rot:
            K.rotate_heads(x, num_heads, head_dim, rot, table, ctx.positions)


def ramped_frequencies(rot: int, theta: float, ramp) -> "tuple[torch.Tensor, float]":
    """(float32 frequency of every pair, multiplier of cosines and sines) of a rotation whose
    frequencies are stretched by `ramp` (a `FrequencyRamp`, or None for the plain theta ** (-2i / rot)).
    With turns(i) = original * f_i / (2 pi), the number of turns pair i makes over the original context:
    the index at which a pair makes t turns is rot * ln(original / (2 pi t)) / (2 ln theta); pairs up to
    the index of `fast` turns keep f_i, pairs from the index of `slow` turns on get f_i / factor, and
    the pairs between blend the two linearly in the index.  Formed in float64, rounded once."""
    i = torch.arange(rot // 2, dtype=torch.float64)
    freq = theta ** (-2.0 * i / rot)
    if ramp is None:
        return freq.to(torch.float32), 1.0
    if hasattr(ramp, "low"):
        return stretched_by_wavelength(freq, ramp).to(torch.float32), 1.0

    def index_of(turns: float) -> float:
        return rot * math.log(ramp.original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    low = max(math.floor(index_of(ramp.fast)), 0)
    high = min(math.ceil(index_of(ramp.slow)), rot - 1)
    blend = torch.clamp((i - low) / max(high - low, 0.001), 0.0, 1.0)
    freq = freq / ramp.factor * blend + freq * (1.0 - blend)
    return freq.to(torch.float32), 0.1 * math.log(ramp.factor) + 1.0


def stretched_by_wavelength(freq: torch.Tensor, ramp) -> torch.Tensor:
    """The float64 frequencies `freq` stretched by a `WavelengthRamp`: a pair whose wavelength 2 pi / f is below
    original / high keeps f, one above original / low gets f / factor, and between the two f / factor and f are
    blended by s = (original / wavelength - low) / (high - low)."""
    wavelength = 2.0 * math.pi / freq
    share = (ramp.original / wavelength - ramp.low) / (ramp.high - ramp.low) if ramp.high != ramp.low else torch.ones_like(freq)
    blended = (1.0 - share) * freq / ramp.factor + share * freq
    out = torch.where(wavelength > ramp.original / ramp.low, freq / ramp.factor, blended)
    return torch.where(wavelength < ramp.original / ramp.high, freq, out)


@register_position_encoding("interleaved_rope")
class InterleavedRope(Part):
    """Rotation of the pairs (2i, 2i + 1) of each head's first `rotary_dim` features by
    position * f_i, with optionally stretched frequencies (`spec.ramp`) and cosines and sines
    multiplied by `magnitude`.  Angles are float32 products of the position and the float32 frequency."""

    graph_safe = True
    interleaved = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even")
        freq, self.magnitude = ramped_frequencies(spec.rotary_dim, spec.theta, spec.ramp)
        self.inv_freq = freq.to(device)

    def rotary_table(self, ctx):
        rot = self.spec.rotary_dim
        if not rot:
            return 0, None
        key = ("interleaved_rope", rot, self.spec.theta, self.spec.ramp)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = K.rope_table(ctx.positions, self.inv_freq)
        return rot, table

    def encode(self, ctx, x: torch.Tensor, num_heads: int, head_dim: int) -> None:
        rot, table = self.rotary_table(ctx)
        if rot:
            K.qk_norm_rotate_store(x, num_heads, 0, head_dim, head_dim, None, None, 0.0, rot, True, table,
                                   self.magnitude, ctx.positions, None, None, 1, None, None)


@register_position_encoding("none")
class NoPosition(Part):
    """No encoding: queries and keys stay as they are."""

    graph_safe = True

    def rotary_table(self, ctx):
        return 0, None

    def encode(self, ctx, x: torch.Tensor, num_heads: int, head_dim: int) -> None:
        return None
