"""Rotary position encoding, half-split pairing: channel i of a head pairs with channel
i + rotary_dim/2, angle = position * theta^(-2i/rotary_dim); channels past ``rotary_dim``
pass through (native/include/flyweight_v2_native_kernels.hpp:993-1050). ``rotary_interleaved``
pairs channel 2i with channel 2i + 1 instead, by the same angles (``interleaved`` tells the mixer's
kernels which pairing the tables are for). The inverse
frequencies are formed in float64 on the host; the per-step cos/sin tables are float32.
``rotary_dim = 0`` (or kind ``none``) means no position encoding at all. ``scaling_factor`` f
(linear position scaling) divides every frequency by f: position p turns as p / f would.
``wavelength_scaling`` (factor, low, high, original) stretches by wavelength instead: with l = 2 pi / f
a frequency stays where l < original / high, becomes f / factor where l > original / low, and between the
two is the blend (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""

from __future__ import annotations

import math

import torch

from ..config.spec import ConfigError
from ..kernels import ops
from .base import PositionEncoding, register_position_encoding


@register_position_encoding("rotary_neox")
class RotaryNeox(PositionEncoding):
    graph_safe = True
    interleaved = False

    def __init__(self, spec):
        super().__init__(spec)
        self.theta = float(spec["theta"])
        self.head_dim = int(spec["head_dim"])
        self.rotary_dim = int(spec.get("rotary_dim", self.head_dim))
        self.scaling_factor = float(spec.get("scaling_factor", 1.0))
        if not self.scaling_factor > 0.0:
            raise ConfigError(f"the rotation's scaling factor must be positive, found {self.scaling_factor}")
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ConfigError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        stretch = spec.get("wavelength_scaling")
        self.wavelength_scaling = None if stretch is None else tuple(float(number) for number in stretch)
        if self.wavelength_scaling is not None:
            factor, low, high, original = self.wavelength_scaling      # four numbers, or this raises
            if not (factor > 0 and original > 0 and high > low >= 0):
                raise ConfigError(f"the rotation's wavelength scaling needs factor > 0, original > 0 and high > low >= 0, found {stretch}")
        self._inv_freq = None

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        half = self.rotary_dim // 2
        exponents = torch.arange(half, dtype=torch.float64) * 2.0 / max(self.rotary_dim, 1)
        frequencies = self.theta ** (-exponents) / self.scaling_factor
        if self.wavelength_scaling is not None:
            factor, low, high, original = self.wavelength_scaling
            wavelength = 2.0 * math.pi / frequencies
            blend = (original / wavelength - low) / (high - low)
            between = (1.0 - blend) * frequencies / factor + blend * frequencies
            frequencies = torch.where(wavelength < original / high, frequencies,
                                      torch.where(wavelength > original / low, frequencies / factor, between))
        self._inv_freq = frequencies.to(device)

    def tables(self, ctx):
        if self.rotary_dim == 0:
            return None, None
        return ops.rope_table(ctx.encoding_pos, self._inv_freq)


@register_position_encoding("rotary_interleaved")
class RotaryInterleaved(RotaryNeox):
    """The pair (u, v) = (channel 2i, channel 2i + 1) becomes (u cos a - v sin a, v cos a + u sin a),
    a = position * theta^(-2i / rotary_dim)."""
    interleaved = True


@register_position_encoding("query_temperature")
class QueryTemperature(PositionEncoding):
    """No rotation: a factor per row on the finished queries, 1 + coef * ln(floor((p + 1) / every) + 1) at position p
    (1 up to position every - 2, then a step up every ``every`` positions). ``tables`` gives float32 [rows]."""
    graph_safe = True
    rotary_dim = 0

    def __init__(self, spec):
        super().__init__(spec)
        self.coef = float(spec["coef"])
        self.every = int(spec["every"])
        if self.every < 1:
            raise ConfigError(f"a query temperature steps every {self.every} positions (at least 1)")

    def tables(self, ctx):
        return ops.query_temperature(ctx.encoding_pos, self.coef, self.every)


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    rotary_dim = 0

    def tables(self, ctx):
        return None, None
