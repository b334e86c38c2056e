"""The gated delta rule: per head a matrix of state that forgets by one factor a token and is corrected towards the
token's value along its key.

``q = Wq x`` and ``k = Wk x`` (``key_heads x key_dim``), ``v = Wv x`` (``heads x value_dim``); value head ``h`` reads
query/key head ``h // (heads / key_heads)``. Each passes a causal convolution per channel over the last ``taps`` tokens
(``conv`` weights ``[channels, taps]``, the last column the token's own, zeros before the request's first token) and
SiLU; queries and keys are then made unit vectors per head, ``a / sqrt(sum(a^2) + unit_eps)``, and queries multiplied
by ``query_scale`` (``key_dim^(-1/2)`` unless given). Per head and token ``beta = sigmoid(Wb x)`` and
``g = exp(-exp(A_log) * softplus(Wa x + dt_bias))``, and

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          (S: [key_dim, value_dim])

so the read-out sees the token's own write. Each head's ``o`` is divided by its root mean square over ``value_dim``,
multiplied by a weight ``[value_dim]`` that all heads share and by ``silu(Wg x)``, and projected by ``Wo``. A request
keeps ``S`` and the convolution's last ``taps - 1`` inputs, both float32, in its state slot, so it can be cut into steps
anywhere. The six projections that read ``x`` are one stacked product with a float32 result; the convolution, the unit
vectors, the gates, the recurrence, the norm and the output gate are float32. Steps in which a request brings
``LONG_PORTION`` tokens or more walk the recurrence on the kernel that stages tiles of tokens through LDS; it does the
same operations in the same order as the one that reads a token's operands from memory, so the state's bits do not
depend on how a request was cut.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import CompositeNeed, MATRIX, Mixer, Runtime, StateNeed, TensorDecl, VECTOR
from .linear import Weight, linear
from .registry import register_part
from .spec import PartSpec


class GatedDeltaRule(Mixer):
    # A step that is run twice would change the state twice: the engine, which runs a step once before it captures
    # it, saves the step's state slots before that run and puts them back.
    graph_safe = True
    LONG_PORTION = 8        # from this many tokens of one request in a step on, the walk stages its operands through LDS

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["heads"])
        self.key_heads = int(p["key_heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.taps = int(p["taps"])
        self.eps = float(p.get("eps", 1e-6))
        self.unit_eps = float(p.get("unit_eps", 1e-6))
        self.query_scale = float(p.get("query_scale", self.key_dim ** -0.5))
        if self.heads % self.key_heads != 0 or self.taps < 1:
            raise ValueError("the value heads must divide into the key heads, and the convolution needs a tap")
        keys, values = self.key_heads * self.key_dim, self.heads * self.value_dim
        self.channels = 2 * keys + values       # of the convolution: queries, keys, values
        # columns of the stacked projection's rows
        self.conv_at, self.gate_at, self.beta_at, self.step_at = 0, self.channels, self.channels + values, self.channels + values + self.heads
        self.in_weight: Optional[Weight] = None
        self.o_weight: Optional[Weight] = None
        self.conv = self.a_log = self.dt_bias = self.norm_weight = None

    def tensors(self) -> Dict[str, TensorDecl]:
        keys, values = self.key_heads * self.key_dim, self.heads * self.value_dim
        return {self.name("q"): TensorDecl((keys, self.hidden), MATRIX), self.name("q_conv"): TensorDecl((keys, self.taps), VECTOR),
                self.name("k"): TensorDecl((keys, self.hidden), MATRIX), self.name("k_conv"): TensorDecl((keys, self.taps), VECTOR),
                self.name("v"): TensorDecl((values, self.hidden), MATRIX), self.name("v_conv"): TensorDecl((values, self.taps), VECTOR),
                self.name("g"): TensorDecl((values, self.hidden), MATRIX), self.name("beta"): TensorDecl((self.heads, self.hidden), MATRIX),
                self.name("step"): TensorDecl((self.heads, self.hidden), MATRIX), self.name("dt_bias"): TensorDecl((self.heads,), VECTOR),
                self.name("A_log"): TensorDecl((self.heads,), VECTOR), self.name("norm"): TensorDecl((self.value_dim,), VECTOR),
                self.name("o"): TensorDecl((self.hidden, values), MATRIX)}

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        weights = [tensors[self.name(role)] for role in ("q", "k", "v", "g", "beta", "step")]
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the projections of one layer must share a dtype to be stacked")
        keep = self.runtime.keep_plain_weights
        self.in_weight = Weight(torch.cat(weights, dim=0).contiguous(), keep_plain=keep)
        del weights
        self.o_weight = Weight(tensors[self.name("o")], keep_plain=keep)
        self.conv = torch.cat([tensors[self.name(f"{role}_conv")] for role in ("q", "k", "v")], dim=0).contiguous()
        self.a_log, self.dt_bias = tensors[self.name("A_log")], tensors[self.name("dt_bias")]
        self.norm_weight = tensors[self.name("norm")]

    def cache_need(self):
        return CompositeNeed((StateNeed((self.taps - 1, self.channels), torch.float32),
                              StateNeed((self.heads, self.key_dim, self.value_dim), torch.float32)))

    def flops(self, tokens: int) -> float:
        return super().flops(tokens) + 2.0 * tokens * (self.channels * self.taps + 3 * self.heads * self.key_dim * self.value_dim)

    def forward(self, x, ctx, cache):
        kept, state = cache.parts[0].state, cache.parts[1].state
        proj = linear(x, self.in_weight, out_dtype=torch.float32)
        u, gates = kernels.delta_prepare(proj, self.conv_at, self.conv, kept, ctx.seq_of_token, ctx.cu_tokens, ctx.slots, self.beta_at,
                                         self.step_at, self.a_log, self.dt_bias, self.key_heads, self.heads, self.key_dim,
                                         self.value_dim, self.query_scale, self.unit_eps)
        if self.taps > 1:
            kernels.conv_keep(proj, self.conv_at, kept, ctx.cu_tokens, ctx.slots, ctx.n_seqs)
        o = kernels.delta_scan(u, gates, state, ctx.cu_tokens, ctx.slots, ctx.n_seqs, self.key_heads, self.heads, self.key_dim,
                               self.value_dim, long_portions=ctx.max_count >= self.LONG_PORTION)
        gated = kernels.gla_gate(o, proj, self.gate_at, self.norm_weight, self.eps, self.heads, self.value_dim, 1.0, self.runtime.dtype)
        return linear(gated, self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "gated_delta_rule", GatedDeltaRule)
