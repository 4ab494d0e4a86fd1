"""Rotary position encoding, half-split pairing: channel i of a head pairs with channel
i + rotary_dim/2, angle = position * theta^(-2i/rotary_dim); channels past ``rotary_dim``
pass through (native/include/flyweight_v2_native_kernels.hpp:993-1050). ``rotary_interleaved``
pairs channel 2i with channel 2i + 1 instead, by the same angles (``interleaved`` tells the mixer's
kernels which pairing the tables are for). The inverse
frequencies are formed in float64 on the host; the per-step cos/sin tables are float32.
``rotary_dim = 0`` (or kind ``none``) means no position encoding at all. ``scaling_factor`` f
(linear position scaling) divides every frequency by f: position p turns as p / f would."""

from __future__ import annotations

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
        self._inv_freq = None

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        half = self.rotary_dim // 2
        exponents = torch.arange(half, dtype=torch.float64) * 2.0 / max(self.rotary_dim, 1)
        self._inv_freq = (self.theta ** (-exponents) / self.scaling_factor).to(device)

    def tables(self, ctx):
        if self.rotary_dim == 0:
            return None, None
        return ops.rope_table(ctx.encoding_pos, self._inv_freq)


@register_position_encoding("rotary_interleaved")
class RotaryInterleaved(RotaryNeox):
    """The pair (u, v) = (channel 2i, channel 2i + 1) becomes (u cos a - v sin a, v cos a + u sin a),
    a = position * theta^(-2i / rotary_dim)."""
    interleaved = True


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    rotary_dim = 0

    def tables(self, ctx):
        return None, None
