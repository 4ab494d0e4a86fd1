"""Mixers side by side: every branch reads the same input and the outputs are mixed with fixed
weights, out = sum_i scale_i * branch_i(h). A branch is any registered mixer that can give its
output as rows of its own (``output(h, ctx, cache)``); each keeps its own cache entry, so the
whole asks the cache manager for a mapping branch name -> that branch's need.
"""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ConfigError
from ..weights.loader import TensorDecl
from .base import Mixer, build_part, register_mixer


@register_mixer("parallel_branches")
class ParallelBranches(Mixer):
    """``branches``: a sequence of (name, PartSpec of a mixer, scale)."""

    def __init__(self, spec):
        super().__init__(spec)
        self.branches: List[Tuple[str, Mixer, float]] = []
        for name, part, scale in spec["branches"]:
            mixer = build_part("mixer", part)
            if not hasattr(mixer, "output"):
                raise ConfigError(f"mixer '{part.kind}' cannot stand in a parallel arrangement: it has no output()")
            self.branches.append((str(name), mixer, float(scale)))
        if not self.branches:
            raise ConfigError("a parallel arrangement needs at least one branch")
        if len({name for name, _, _ in self.branches}) != len(self.branches):
            raise ConfigError("the branches of a parallel arrangement need different names")

    @property
    def graph_safe(self) -> bool:
        return all(mixer.graph_safe and getattr(getattr(mixer, "position", None), "graph_safe", True)
                   for _, mixer, _ in self.branches)

    def tensors(self) -> Dict[str, TensorDecl]:
        declared: Dict[str, TensorDecl] = {}
        for _, mixer, _ in self.branches:
            declared.update(mixer.tensors())
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        for _, mixer, _ in self.branches:
            mixer.bind(tensors, dtype, device)

    def cache_need(self):
        return {name: mixer.cache_need() for name, mixer, _ in self.branches}

    # a branch's index arrays travel with the step as any part's do
    def sub_parts(self):
        return [mixer for _, mixer, _ in self.branches]

    def output_terms(self, h, ctx, cache) -> List[Tuple[torch.Tensor, float]]:
        """[(float32 rows, scale)]: the mixer's output is their weighted sum, which the caller forms
        where it reads them."""
        return [(mixer.output(h, ctx, cache[name]), scale) for name, mixer, scale in self.branches]

    def forward(self, h, residual, ctx, cache):
        for rows, scale in self.output_terms(h, ctx, cache):
            residual.add_(rows, alpha=scale)
        return None
