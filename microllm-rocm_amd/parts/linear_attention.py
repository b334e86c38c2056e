"""Gated linear attention: per head a matrix of state, decayed per key channel, carried from token to token.

``q = Wq x * query_scale`` and ``k = Wk x`` (``heads x key_dim``), ``v = Wv x`` (``heads x value_dim``). The decay of
key channel ``c`` is ``a = sigmoid(z)^(1 / tau)`` with ``z = A2 (A1 x) + b`` through a small inner size. Per head

    S_t = diag(a_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t

(the decay scales the rows of ``S`` that belong to key channels). With ``fixed_decay`` (one number a head) there are no
``A1``, ``A2`` and ``b``: every key channel of head ``h`` decays by ``fixed_decay[h]`` at every token (retention). A
scale on the keys instead of the queries is the same ``query_scale``: ``o`` is linear in both. Each head's ``o`` is divided by its root mean square
over ``value_dim`` and multiplied by a weight ``[value_dim]`` that all heads share (``norm_weight`` false: by none); the heads side by side are
multiplied by ``silu(Wg x)`` and projected by ``Wo``. The state starts at zero, is float32, and lives in the
request's state slot, so a request can be cut into steps anywhere. The five projections that read ``x`` are one
stacked product with a float32 result; decays, the recurrence, the norm and the gate are float32.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import MATRIX, Mixer, Runtime, StateNeed, TensorDecl, VECTOR
from .linear import Weight, linear
from .registry import register_part
from .spec import PartSpec


class GatedLinearAttention(Mixer):
    # A step that is run twice would decay and add to the state twice: the engine, which runs a step once before it
    # captures it, saves the step's state slots before that run and puts them back (``CacheManager.save_slots``).
    graph_safe = True
    LONG_PORTION = 8        # from this many tokens of one request in a step on, the walk stages its operands through LDS

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.fixed_decay = [float(value) for value in p["fixed_decay"]] if p.get("fixed_decay") is not None else None
        if self.fixed_decay is not None and len(self.fixed_decay) != self.heads:
            raise ValueError("one fixed decay a head")
        self.rank = int(p["decay_rank"]) if self.fixed_decay is None else 0
        self.tau = float(p["tau"]) if self.fixed_decay is None else 1.0
        self.has_norm_weight = bool(p.get("norm_weight", True))
        self.eps = float(p.get("eps", 1e-6))
        self.query_scale = float(p.get("query_scale", self.key_dim ** -0.5))
        keys, values = self.heads * self.key_dim, self.heads * self.value_dim
        # columns of the stacked projection's rows
        self.q_at, self.k_at, self.v_at, self.g_at, self.low_at = 0, keys, 2 * keys, 2 * keys + values, 2 * keys + 2 * values
        self.in_weight: Optional[Weight] = None
        self.decay_weight: Optional[torch.Tensor] = None
        self.decay_bias: Optional[torch.Tensor] = None
        self.decay_row: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None
        self.o_tensor: Optional[torch.Tensor] = None
        self.o_weight: Optional[Weight] = None

    @property
    def inner_width(self) -> int:
        return self.heads * self.value_dim

    def tensors(self) -> Dict[str, TensorDecl]:
        keys, values = self.heads * self.key_dim, self.heads * self.value_dim
        decls = {self.name("q"): TensorDecl((keys, self.hidden), MATRIX), self.name("k"): TensorDecl((keys, self.hidden), MATRIX),
                 self.name("v"): TensorDecl((values, self.hidden), MATRIX), self.name("g"): TensorDecl((values, self.hidden), MATRIX),
                 self.name("o"): TensorDecl((self.hidden, values), MATRIX)}
        if self.has_norm_weight:
            decls[self.name("norm")] = TensorDecl((self.value_dim,), VECTOR)
        if self.fixed_decay is None:
            decls.update({self.name("a1"): TensorDecl((self.rank, self.hidden), MATRIX), self.name("a2"): TensorDecl((keys, self.rank), MATRIX),
                          self.name("a2_bias"): TensorDecl((keys,), VECTOR)})
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        weights = [tensors[self.name(role)] for role in ("q", "k", "v", "g") + (("a1",) if self.fixed_decay is None else ())]
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the projections of one layer must share a dtype to be stacked")
        self.in_weight = Weight(torch.cat(weights, dim=0).contiguous(), keep_plain=self.runtime.keep_plain_weights)
        del weights
        self.o_tensor = tensors[self.name("o")]
        if self.fixed_decay is None:
            self.decay_weight = tensors[self.name("a2")].contiguous()
            self.decay_bias = tensors[self.name("a2_bias")]
        else:       # one row of decays for every token: the head's number for each of its key channels
            per_head = torch.tensor(self.fixed_decay, dtype=torch.float32, device=self.o_tensor.device)
            self.decay_row = per_head.repeat_interleave(self.key_dim).contiguous()
        self.norm_weight = tensors[self.name("norm")] if self.has_norm_weight else None

    def take_output_projection(self) -> Optional[torch.Tensor]:
        tensor, self.o_tensor = self.o_tensor, None
        return tensor

    def cache_need(self):
        return StateNeed((self.heads, self.key_dim, self.value_dim), torch.float32)

    def flops(self, tokens: int) -> float:
        keys, values = self.heads * self.key_dim, self.heads * self.value_dim
        outputs = values if self.o_tensor is not None or self.o_weight is not None else 0
        products = 2.0 * tokens * (self.hidden * (2 * keys + 2 * values + outputs + self.rank) + keys * self.rank)
        return products + 5.0 * tokens * self.heads * self.key_dim * self.value_dim

    def forward_inner(self, x, ctx, cache, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        proj = linear(x, self.in_weight, out_dtype=torch.float32)
        if self.fixed_decay is None:
            decay = kernels.gla_decay(proj, self.low_at, self.decay_weight, self.decay_bias, self.tau)
        else:
            decay = self.decay_row
        o = kernels.gla_scan(proj, self.q_at, self.k_at, self.v_at, decay, cache.state, ctx.cu_tokens, ctx.slots, ctx.n_seqs,
                             self.heads, self.key_dim, self.value_dim, self.query_scale,
                             long_portions=ctx.max_count >= self.LONG_PORTION)
        return kernels.gla_gate(o, proj, self.g_at, self.norm_weight, self.eps, self.heads, self.value_dim, out_scale,
                                self.runtime.dtype, out=out)

    def forward(self, x, ctx, cache):
        if self.o_weight is None:
            if self.o_tensor is None:
                raise RuntimeError("this mixer's output projection was taken by the mixer it is a part of")
            self.o_weight = Weight(self.take_output_projection(), keep_plain=self.runtime.keep_plain_weights)
        return linear(self.forward_inner(x, ctx, cache), self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
