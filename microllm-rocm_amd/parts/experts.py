"""A mixture of experts: every token goes through ``top`` of ``experts`` small gated feed-forwards.

Router logits ``z = Wr x`` are a float32 product (the router's weight is kept in float32); scores are ``sigmoid(z)`` or
the softmax over the experts; the ``top`` largest are chosen (ties: the lower index) and their scores are the weights
(``renormalize``: divided by their sum). With ``weight_on`` ``"input"`` the weight multiplies what the expert reads,
``sum_e expert_e(w_e x)``; with ``"output"`` what it returns. An expert is ``Wd (act(Wg x) * (Wu x))`` without
biases, or with ``expert_form`` ``"plain"`` ``Wd act(Wu x)`` (no ``gate`` tensors); ``activation`` is ``silu``,
``gelu_erf`` (the exact gelu) or ``gelu_tanh``. With ``groups`` the experts form that many equal groups of neighbours, a
group counts as much as its best expert, and only experts of the ``keep_groups`` best groups can be chosen. A shared expert of the same form may run for every token; with ``shared_scale`` ``"sigmoid"`` it is
multiplied by ``sigmoid(ws . x)``, one number a token, whose weight rides as one more row of the router's product.

The result is handed on as float32 partial sums ``[top (+ 1), tokens, hidden]``: one part a choice and one for the
shared expert, which the next norm adds in order; a token's sums therefore never depend on the other tokens of the
step. Which expert a (token, choice) pair takes is known on the device only: the experts' kernels read the ids there,
and nothing comes back to the host.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .base import FeedForward, MATRIX, Runtime, TensorDecl, VECTOR
from .linear import Weight, linear
from .registry import register_part
from .spec import PartSpec


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.experts = int(p["experts"])
        self.top = int(p["top"])
        self.expert_size = int(p["expert_size"])
        self.shared_size = int(p["shared_size"]) if p.get("shared_size") else 0
        self.score = p.get("score", "sigmoid")
        self.renormalize = bool(p.get("renormalize", False))
        self.weight_on = p.get("weight_on", "output")
        self.shared_scale = p.get("shared_scale") if self.shared_size else None
        self.gated = p.get("expert_form", "gated") == "gated"
        self.activation = p.get("activation", "silu")
        self.groups = int(p.get("groups") or 0)
        self.keep_groups = int(p.get("keep_groups") or 0)
        if p.get("expert_form", "gated") not in ("gated", "plain") or self.activation not in kernels.ACTIVATIONS:
            raise ValueError("expert_form is gated or plain, activation one of " + ", ".join(kernels.ACTIVATIONS))
        if self.gated and self.shared_size and self.activation != "silu":
            raise ValueError("a gated shared expert takes SiLU: the products' gated epilogue has no other activation")
        if self.groups and (self.experts % self.groups or not 1 <= self.keep_groups <= self.groups
                            or self.keep_groups * (self.experts // self.groups) < self.top):
            raise ValueError("equal groups of experts, of which the kept ones hold at least `top` experts")
        if self.score not in ("sigmoid", "softmax") or self.weight_on not in ("input", "output") or self.shared_scale not in (None, "sigmoid"):
            raise ValueError("score is sigmoid or softmax, weight_on input or output, shared_scale sigmoid or None")
        if not 1 <= self.top <= self.experts:
            raise ValueError("between one and all experts a token")
        self.route_weight: Optional[torch.Tensor] = None
        self.gate_up: Optional[torch.Tensor] = None
        self.down: Optional[torch.Tensor] = None
        self.shared_gate_up: Optional[Weight] = None
        self.shared_down: Optional[Weight] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        decls = {self.name("router"): TensorDecl((self.experts, self.hidden), VECTOR)}
        for expert in range(self.experts):
            if self.gated:
                decls[self.name(f"expert{expert}.gate")] = TensorDecl((self.expert_size, self.hidden), MATRIX)
            decls[self.name(f"expert{expert}.up")] = TensorDecl((self.expert_size, self.hidden), MATRIX)
            decls[self.name(f"expert{expert}.down")] = TensorDecl((self.hidden, self.expert_size), MATRIX)
        if self.shared_size:
            if self.gated:
                decls[self.name("shared.gate")] = TensorDecl((self.shared_size, self.hidden), MATRIX)
            decls[self.name("shared.up")] = TensorDecl((self.shared_size, self.hidden), MATRIX)
            decls[self.name("shared.down")] = TensorDecl((self.hidden, self.shared_size), MATRIX)
            if self.shared_scale is not None:
                decls[self.name("shared.scale")] = TensorDecl((1, self.hidden), VECTOR)
        return decls

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        rows = [tensors[self.name("router")]]
        if self.shared_scale is not None:
            rows.append(tensors[self.name("shared.scale")])
        self.route_weight = torch.cat(rows, dim=0).contiguous()        # float32 [experts (+ 1), hidden]
        gate_up = down = None
        inner_rows = (2 if self.gated else 1) * self.expert_size
        for expert in range(self.experts):      # every tensor is looked up once: the loader lets go of it then
            gate = tensors[self.name(f"expert{expert}.gate" if self.gated else f"expert{expert}.up")]
            if gate_up is None:
                gate_up = torch.empty((self.experts, inner_rows, self.hidden), dtype=gate.dtype, device=gate.device)
                down = torch.empty((self.experts, self.hidden, self.expert_size), dtype=gate.dtype, device=gate.device)
            gate_up[expert, :self.expert_size] = gate
            if self.gated:
                gate_up[expert, self.expert_size:] = tensors[self.name(f"expert{expert}.up")]
            down[expert] = tensors[self.name(f"expert{expert}.down")]
            del gate
        self.gate_up, self.down = gate_up, down
        if self.shared_size:
            keep = self.runtime.keep_plain_weights
            if self.gated:
                gate, up = tensors[self.name("shared.gate")], tensors[self.name("shared.up")]
                self.shared_gate_up = Weight(torch.cat([gate, up], dim=0).contiguous(), gated=True, keep_plain=keep)
                del gate, up
            else:
                self.shared_gate_up = Weight(tensors[self.name("shared.up")], keep_plain=keep)
            self.shared_down = Weight(tensors[self.name("shared.down")], keep_plain=keep)

    def flops(self, tokens: int) -> float:
        routed = (6.0 if self.gated else 4.0) * tokens * self.top * self.hidden * self.expert_size
        return super().flops(tokens) + routed + 2.0 * tokens * self.hidden * self.experts

    def weight_bytes_read(self, rows: int) -> int:
        """Bytes of weights a step of ``rows`` tokens reads at most: the router, the shared expert, and the experts that
        the rows' choices can reach (each once, where the rows are multiplied in tiles; fewer than a reading a pair)."""
        element = self.gate_up.element_size()
        reached = min(self.experts, rows * self.top)
        matrices = 3 if self.gated else 2
        total = 4 * self.route_weight.numel() + reached * matrices * self.expert_size * self.hidden * element
        return total + matrices * self.shared_size * self.hidden * element

    def forward(self, x, ctx):
        n_tokens = x.shape[0]
        z = kernels.router_logits(x, self.route_weight)
        ids, weights, shared_factor = kernels.moe_route(z, self.experts, self.top, softmax_scores=self.score == "softmax",
                                                        renormalize=self.renormalize,
                                                        shared_at=self.experts if self.shared_scale is not None else -1,
                                                        groups=self.groups, keep=self.keep_groups)
        parts = torch.empty((self.top + (1 if self.shared_size else 0), n_tokens, self.hidden), dtype=torch.float32, device=x.device)
        kernels.moe_experts(x, ids, weights, self.gate_up, self.down, self.weight_on == "input", out=parts, gated=self.gated,
                            activation=self.activation)
        if self.shared_size:
            if self.gated:
                inner = linear(x, self.shared_gate_up, gated=True)
            else:       # the activation reads the product's float32 sums and rounds once
                inner = kernels.activation(linear(x, self.shared_gate_up, out_dtype=torch.float32, partials=True), self.activation, x.dtype)
            if shared_factor is not None:
                kernels.scale_rows(linear(inner, self.shared_down, out_dtype=torch.float32, partials=True), shared_factor, parts[self.top])
            else:
                parts[self.top].copy_(linear(inner, self.shared_down, out_dtype=torch.float32))
        return parts


register_part("ffn", "routed_experts", RoutedExperts)
