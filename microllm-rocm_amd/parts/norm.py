"""RMSNorm over the float32 residual stream.

``y = x * (1 / sqrt(mean(x^2) + eps)) * w`` with eps inside the root and the
weight multiplied last (src/ops/ops.cpp:687-698); fused with the residual sum as
the reference's ``add_rms_norm`` is (src/ops/hip/basic_kernels.hip:393-418).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import Norm, Runtime, TensorDecl, VECTOR
from .registry import register_part
from .spec import PartSpec


class NormedDelta:
    """A sublayer's result that is still to be RMS-normed with a weight of its own and multiplied by ``mult`` before
    it joins the residual stream: ``h += mult * values / sqrt(mean(values^2) + eps) * weight``. The norm that reads the
    stream next does both in one kernel. ``values`` is ``[tokens, hidden]`` or float32 partial sums ``[parts, tokens,
    hidden]``, which are added in order first. ``extra``: float32 rows ``[tokens, hidden]`` that join the stream after
    it, unnormed (``with_extra``)."""

    def __init__(self, values: torch.Tensor, weight: torch.Tensor, eps: float, mult: float, extra: Optional[torch.Tensor] = None):
        self.values = values
        self.weight = weight
        self.eps = float(eps)
        self.mult = float(mult)
        self.extra = extra

    def with_extra(self, rows: torch.Tensor) -> "NormedDelta":
        if self.extra is not None:
            raise ValueError("this delta already takes further rows along")
        return NormedDelta(self.values, self.weight, self.eps, self.mult, rows)

    def resolved(self) -> torch.Tensor:
        """What joins the stream, as a float32 tensor ``[tokens, hidden]`` (for observers; a step never needs it)."""
        shape = self.values.shape[-2:]
        joined = torch.zeros(shape, dtype=torch.float32, device=self.values.device)
        kernels.rms_norm_after(joined, self.values, self.weight, self.eps, self.mult, None, 1.0, self.values.dtype, write_h=True,
                               extra=self.extra)
        return joined


class RMSNorm(Norm):
    graph_safe = True
    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        # ``unit_offset``: the file stores the gain's distance from one; the gain ``1 + w`` is formed once, at load,
        # in float32 (the sum a float32 evaluation of ``x * (1 + w)`` forms for every element).
        self.unit_offset = bool(spec.params.get("unit_offset", False))
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name("weight"): TensorDecl((self.size,), VECTOR)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")]
        if self.unit_offset:
            self.weight = (self.weight.to(torch.float32) + 1.0).contiguous()

    def weight_then_factor(self):
        return (self.weight, self.size, self.eps) if self.weight is not None and self.weight.dtype == torch.float32 else None

    def forward(self, h, delta=None, write_h=True, rows=None):
        if isinstance(delta, NormedDelta):
            return kernels.rms_norm_after(h, delta.values, delta.weight, delta.eps, delta.mult, self.weight, self.eps,
                                          self.runtime.dtype, rows=rows, write_h=write_h and rows is None, extra=delta.extra)
        return kernels.rms_norm(h, self.weight, self.eps, self.runtime.dtype, delta=delta, rows=rows,
                                write_h=write_h and delta is not None and rows is None)


register_part("norm", "rms_norm", RMSNorm)
