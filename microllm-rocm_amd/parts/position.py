"""Rotary position encoding in the split-half layout, and in the layout of neighbours.

For pair ``i`` of a head: ``theta = p * base^(-2i/d)``;
``x'[i] = x[i] cos - x[i+d/2] sin``; ``x'[i+d/2] = x[i] sin + x[i+d/2] cos``
(src/ops/ops.cpp:863-878). The part owns the table of inverse frequencies, held
in float64 so that the angle of any position is exact before cos and sin are
rounded to float32. cos and sin of a step's positions are computed once and
shared by the layers whose encoding has the same parameters; the attention
mixer's fused kernels apply the rotation. With ``scaling_factor`` every rate is
divided by that number (positions stretched linearly).

``rope_neighbours`` pairs channel ``2i`` with ``2i + 1`` instead. Moving channel
``2i`` to ``i`` and ``2i + 1`` to ``i + d/2`` makes it the split-half rule, and a
dot product of two vectors does not change when both are reordered alike: a
mixer whose turned queries and keys only ever meet in their dot product reorders
the rows of the weights that produce them once, at load (``split_half_order``),
and runs the split-half kernels.
"""
from __future__ import annotations

import torch

from ..ops import kernels
from .base import PositionEncoding, Runtime
from .registry import register_part
from .spec import PartSpec


class RopeSplitHalf(PositionEncoding):
    graph_safe = True
    fused_split_half = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.theta = float(spec.params["theta"])
        self.head_dim = int(spec.params["head_dim"])
        self.rotary_dim = int(spec.params.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 != 0 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and at most head_dim")
        self.scaling_factor = float(spec.params.get("scaling_factor") or 1.0)
        if self.scaling_factor <= 0.0:
            raise ValueError("scaling_factor must be positive")
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim
        self.inv_freq = ((self.theta ** -exponents) / self.scaling_factor).to(runtime.device)

    def table(self, ctx) -> torch.Tensor:
        """``[tokens, rotary_dim / 2, 2]`` float32: cos and sin for the step's tokens."""
        key = ("rope_split_half", self.theta, self.rotary_dim, self.scaling_factor)
        if key not in ctx.memo:
            ctx.memo[key] = kernels.rope_table(ctx.positions, self.inv_freq)
        return ctx.memo[key]


class RopeNeighbours(RopeSplitHalf):
    """Channel ``2i`` turns with channel ``2i + 1`` by ``p * base^(-2i/d)``. The mixer brings the turned channels into
    ``split_half_order`` at load; from there on this is the split-half encoding with the same rates."""

    def split_half_order(self) -> torch.Tensor:
        """``order[new] = old``: the even channels of the turned part first, then the odd ones."""
        return torch.cat([torch.arange(0, self.rotary_dim, 2), torch.arange(1, self.rotary_dim, 2)])


register_part("position", "rope_split_half", RopeSplitHalf)
register_part("position", "rope_neighbours", RopeNeighbours)
