"""Gated linear unit with clamped halves: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
f = W_down (g * sigmoid(alpha * g) * (u + shift)), no biases. Gate and up are one operand of 2I rows,
so h is read once; the activation is formed from the float32 sums and rounded once."""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import FeedForward, register_feed_forward
from .linear import Linear

_DEFAULT_NAMES = {"gate": "gate", "up": "up", "down": "down"}


@register_feed_forward("clamped_glu")
class ClampedGLU(FeedForward):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.intermediate = int(spec["intermediate_size"])
        self.limit = float(spec["limit"])
        self.alpha = float(spec.get("alpha", 1.702))
        self.shift = float(spec.get("shift", 1.0))
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        self.weight_suffix = spec.get("weight_suffix", ".weight")
        if not self.limit > 0:
            raise ConfigError(f"the feed-forward's limit must be positive, found {self.limit}")

    def _name(self, which: str) -> str:
        return f"{self.prefix}{self.names[which]}{self.weight_suffix}"

    def tensors(self) -> Dict[str, TensorDecl]:
        return {
            self._name("gate"): TensorDecl((self.intermediate, self.hidden)),
            self._name("up"): TensorDecl((self.intermediate, self.hidden)),
            self._name("down"): TensorDecl((self.hidden, self.intermediate)),
        }

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        gate, up = tensors[self._name("gate")], tensors[self._name("up")]
        if gate.dtype != up.dtype:
            raise ConfigError(f"{self.prefix}: gate and up projections are stored in different precisions")
        self.gate_up = Linear(torch.cat([gate, up], dim=0))
        self.down = Linear(tensors[self._name("down")])

    def activation(self, h) -> torch.Tensor:
        return self.gate_up.clamped_glu(h, self.limit, self.alpha, self.shift)

    def output_terms(self, h, ctx) -> List[Tuple[torch.Tensor, float]]:
        return [(self.down.forward(self.activation(h), out_dtype=torch.float32), 1.0)]

    def forward(self, h, residual, ctx):
        self.down.accumulate(self.activation(h), residual)
        return None
