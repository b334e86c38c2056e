"""Causal softmax attention with the pieces that designs put around it, each a parameter: a norm of queries and keys, a
learned bias by distance bucket or a slope a head times the distance, a rotation of queries and keys, a sink in the
softmax, a query factor that grows with the position, a sliding window or a mask by chunks of positions, a gate a head.

``q = Wq x``, ``k = Wk x``, ``v = Wv x`` (with ``projection_bias`` each and the output projection have a bias, named
as the weight with ``_bias``); query head ``h`` uses kv head ``h // (heads / kv_heads)``; keys
have ``key_dim`` and values ``value_dim`` channels. With ``qk_norm`` queries and keys are divided by their root mean
square over the head (eps inside the root) and, unless ``qk_norm_weight`` is false, multiplied by a weight
``[key_dim]`` that all heads share. Queries
at position ``p`` are multiplied by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``. The score of key ``j``
for a query at ``i >= j`` is ``(q . k) * scale + table[bucket(i - j), h]`` with, for a table of ``B`` rows and a
longest distance ``D``: ``bucket(n) = n`` below ``B / 2``, else ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2))
* (B - B/2)))``. With ``slopes`` (one number a head) ``slopes[h] * (i - j)`` is taken off the score instead. The
softmax's denominator also holds ``exp(sink[h])``, which has no key and no value; ``sink_value`` gives every head
that number instead of a tensor (0: one is added to the denominator). With ``chunk`` a query sees ``j <= i`` with
``floor(j / chunk) = floor(i / chunk)``, positions counted from the sequence's start. With ``position`` (a split-half
rotary encoding, which may turn fewer channels than the head has and stretch positions) queries and keys are turned
after their norm. With ``head_gate`` head ``h``'s result is multiplied by ``sigmoid(Wg x)_h``, ``Wg`` being ``[heads,
hidden]``, one more block of rows of the stacked input product. With ``window`` a query sees
``0 <= i - j < window``. With ``owns_kv`` false the layer has no ``Wk`` and ``Wv``: it reads the keys (as cached, after
their norm) and values of another run entry, with queries, bias and window of its own.

Every distance from ``D`` on falls into the last bucket, so the table is unrolled once, at load, into one row per
distance up to ``D`` and the kernels index it with ``min(i - j, D)``. Slopes under a window become such a table for
the MFMA kernels (a row per distance inside the window); the kernel for plain pages takes the slopes themselves.
Under chunks nothing is given back early: a request keeps its pages until it closes.

In bfloat16, with keys and values of one width that is a multiple of 16, the pages are the paged attention's own
(``PagedKVNeed``) and the attention runs on its MFMA kernels, which take the bias, the sink and the result's factor
as extras; everything else (float32, two widths, other sizes) lies in plain pages (``PagedKeyValueNeed``) and runs on
the kernel that takes a wave per token and head.
"""
from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .attention import QueryTilePlanner
from .base import MATRIX, Mixer, PagedKeyValueNeed, PagedKVNeed, Runtime, TensorDecl, VECTOR
from .linear import Weight, linear
from .registry import build_part, register_part
from .spec import PartSpec


def distance_bucket(distance: int, rows: int, longest: int) -> int:
    """The row of a ``rows``-row bias table for ``distance >= 0``: exact below ``rows // 2``, logarithmic up to
    ``longest``, the last row beyond."""
    half = rows // 2
    if distance < half:
        return distance
    return min(rows - 1, half + int(math.floor(math.log(distance / half) / math.log(longest / half) * (rows - half))))


class BucketBiasAttention(Mixer):
    graph_safe = True

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.scale = float(p.get("scale", 1.0 / math.sqrt(self.key_dim)))
        self.qk_norm = bool(p.get("qk_norm", True))
        self.eps = float(p.get("eps", 1e-6))
        self.temp_coef = float(p.get("temp_coef", 0.0))
        self.temp_every = int(p.get("temp_every", 1))
        self.bias_rows = int(p["bias_rows"]) if p.get("bias_rows") else 0      # 0: no bias
        self.bias_max = int(p.get("bias_max", 0))
        self.has_sink = bool(p.get("sink", True))
        self.projection_bias = bool(p.get("projection_bias", False))
        self.qk_norm_weight = bool(p.get("qk_norm_weight", True)) and self.qk_norm
        self.slope_values = [float(value) for value in p["slopes"]] if p.get("slopes") is not None else None
        self.window = int(p["window"]) if p.get("window") else 0
        self.chunk = int(p["chunk"]) if p.get("chunk") else 0
        self.head_gate = bool(p.get("head_gate", False))
        self.sink_value = float(p["sink_value"]) if p.get("sink_value") is not None else None
        if self.sink_value is not None:
            self.has_sink = False       # no tensor in the files: the number is the sink of every head
        self.position = build_part("position", p["position"], runtime) if p.get("position") is not None else None
        if self.position is not None and (not self.position.fused_split_half or 2 * self.position.inv_freq.shape[0] > self.key_dim):
            raise ValueError("queries and keys turn by a split-half encoding over at most their head's channels")
        if self.window and self.chunk:
            raise ValueError("a window or chunks of positions, not both")
        # how long the keys and values are kept: the widest window of the layers that read them (0: for ever)
        self.kept_window = int(p.get("kept_window") or self.window) if self.window else 0
        self.owns_kv = bool(p.get("owns_kv", True))
        if self.heads % self.kv_heads != 0:
            raise ValueError("heads must divide into kv_heads groups")
        if self.bias_rows and self.bias_max <= self.bias_rows // 2:
            raise ValueError("bias_max must lie beyond the distances that have a bucket of their own")
        if self.slope_values is not None and (len(self.slope_values) != self.heads or self.bias_rows):
            raise ValueError("one slope a head, and either slopes or a table of buckets")
        if self.window and self.kept_window < self.window:
            raise ValueError("the keys and values must be kept at least as long as this layer's window")
        # the paged attention's pages and MFMA kernels, where they fit (the bias column must fit the prefill kernel's LDS;
        # slopes are such a column only under a window that fits)
        # (the widest window among the layers that share the pages decides, so that all of them lay the pages out alike)
        table_rows = self.kept_window if self.slope_values is not None else self.bias_max + 1
        self.tiled = (bool(p.get("mfma", True)) and runtime.dtype == torch.bfloat16 and self.key_dim == self.value_dim
                      and self.key_dim % 16 == 0 and self.key_dim <= 256 and 0 < table_rows <= kernels.MFMA_BIAS_ROWS)
        self.planner = QueryTilePlanner(bool(self.window or self.chunk)) if self.tiled else None
        self.slopes = self.o_bias = self.qkv_bias = None
        self.qkv_weight: Optional[Weight] = None
        self.o_tensor: Optional[torch.Tensor] = None
        self.o_weight: Optional[Weight] = None
        self.q_norm = self.k_norm = self.bias = self.sink = None

    @property
    def inner_width(self) -> int:
        return self.heads * self.value_dim

    def tensors(self) -> Dict[str, TensorDecl]:
        decls = {self.name("q"): TensorDecl((self.heads * self.key_dim, self.hidden), MATRIX),
                 self.name("o"): TensorDecl((self.hidden, self.heads * self.value_dim), MATRIX)}
        if self.owns_kv:
            decls[self.name("k")] = TensorDecl((self.kv_heads * self.key_dim, self.hidden), MATRIX)
            decls[self.name("v")] = TensorDecl((self.kv_heads * self.value_dim, self.hidden), MATRIX)
        if self.projection_bias:
            for role in self._in_roles() + ("o",):
                decls[self.name(f"{role}_bias")] = TensorDecl((decls[self.name(role)].shape[0],), VECTOR)
        if self.qk_norm_weight:
            decls[self.name("q_norm")] = TensorDecl((self.key_dim,), VECTOR)
            if self.owns_kv:
                decls[self.name("k_norm")] = TensorDecl((self.key_dim,), VECTOR)
        if self.bias_rows:
            decls[self.name("bias")] = TensorDecl((self.bias_rows, self.heads), VECTOR)
        if self.has_sink:
            decls[self.name("sink")] = TensorDecl((self.heads,), VECTOR)
        if self.head_gate:
            decls[self.name("g")] = TensorDecl((self.heads, self.hidden), MATRIX)
        return decls

    def _in_roles(self):
        return ("q", "k", "v") if self.owns_kv else ("q",)

    def sub_parts(self):
        return (self.position,) if self.position is not None else ()

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        weights = [tensors[self.name(role)] for role in self._in_roles() + (("g",) if self.head_gate else ())]
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the q, k and v weights of one layer must share a dtype to be stacked")
        self.qkv_weight = Weight(torch.cat(weights, dim=0).contiguous() if len(weights) > 1 else weights[0],
                                 keep_plain=self.runtime.keep_plain_weights)
        del weights
        self.o_tensor = tensors[self.name("o")]
        if self.projection_bias:
            self.qkv_bias = torch.cat([tensors[self.name(f"{role}_bias")] for role in self._in_roles()]).contiguous()
            self.o_bias = tensors[self.name("o_bias")]
        if self.qk_norm_weight:
            self.q_norm = tensors[self.name("q_norm")]
            self.k_norm = tensors[self.name("k_norm")] if self.owns_kv else None
        if self.slope_values is not None:
            device = self.o_tensor.device
            self.slopes = torch.tensor(self.slope_values, dtype=torch.float32, device=device)
            if self.tiled:      # a row per distance inside the window: what lies further is not seen
                distances = torch.arange(self.window, dtype=torch.float32, device=device)
                self.bias = (-(distances[:, None] * self.slopes[None, :])).contiguous()
        if self.bias_rows:
            table = tensors[self.name("bias")]
            rows = [distance_bucket(distance, self.bias_rows, self.bias_max) for distance in range(self.bias_max + 1)]
            self.bias = table[torch.tensor(rows, dtype=torch.int64, device=table.device)].contiguous()   # [bias_max + 1, heads]
        if self.has_sink:
            self.sink = tensors[self.name("sink")]
        elif self.sink_value is not None:
            self.sink = torch.full((self.heads,), self.sink_value, dtype=torch.float32, device=self.o_tensor.device)

    def take_output_projection(self) -> Optional[torch.Tensor]:
        """The output projection ``[hidden, inner_width]`` as loaded, for a mixer that runs this one beside others and
        multiplies all their results with one stacked weight; this part then no longer holds it."""
        tensor, self.o_tensor = self.o_tensor, None
        return tensor

    def step_planner(self):
        return self.planner

    def cache_need(self):
        if not self.owns_kv:
            return None
        window = self.kept_window or None
        if self.tiled:
            return PagedKVNeed(self.kv_heads, self.key_dim, window)
        return PagedKeyValueNeed(self.kv_heads, self.key_dim, self.value_dim, window)

    def flops(self, tokens: int) -> float:
        window = self.window or tokens
        pairs = sum(min(position + 1, window) for position in range(tokens))
        columns = self.heads * self.key_dim + ((self.key_dim + self.value_dim) * self.kv_heads if self.owns_kv else 0)
        if self.o_tensor is not None or self.o_weight is not None:      # else the mixer that took the projection counts it
            columns += self.heads * self.value_dim
        if self.chunk:
            pairs = sum(position % self.chunk + 1 for position in range(tokens))
        columns += self.heads if self.head_gate else 0
        return 2.0 * tokens * self.hidden * columns + 2.0 * self.heads * (self.key_dim + self.value_dim) * pairs

    def forward_inner(self, x, ctx, cache, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
        """The heads' results side by side, ``[tokens, heads * value_dim]`` times ``out_scale``, before the output
        projection; written into ``out`` if given (columns of a wider buffer)."""
        view = ctx.paged[cache.group]
        # rounded once, after norm and factor; the gate's columns, which the attention kernel reads as they are, want whole sums
        qkv = linear(x, self.qkv_weight, out_dtype=torch.float32, partials=not self.head_gate)
        q = kernels.qk_norm_store(qkv, self.q_norm, self.k_norm, self.eps, ctx.positions, view.slot_mapping, self.temp_coef,
                                  self.temp_every, cache.k, cache.v, self.heads, self.kv_heads, self.key_dim, self.value_dim,
                                  self.runtime.dtype, tiled_page_size=view.page_size if self.tiled else 0, bias=self.qkv_bias,
                                  normed=self.qk_norm, queries_only=not self.owns_kv,
                                  cos_sin=self.position.table(ctx) if self.position is not None else None,
                                  further_columns=self.heads if self.head_gate else 0)
        gate = qkv[:, qkv.shape[1] - self.heads:] if self.head_gate else None
        if self.tiled:
            if out is None:
                out = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=self.runtime.dtype, device=x.device)
            extras = kernels.AttentionExtras(self.bias, self.sink, out_scale, chunk=self.chunk, gate=gate)
            return kernels.paged_attention(q, cache.k, cache.v, view, ctx, self.scale, self.window, self.heads, self.kv_heads,
                                           self.key_dim, planner=self.planner, extras=extras, out=out)
        return kernels.bias_attention(q, cache.k, cache.v, view.block_table, ctx.seq_of_token, ctx.positions, self.bias,
                                      self.sink, self.scale, out_scale, self.heads, self.kv_heads, self.key_dim,
                                      self.value_dim, out=out, slopes=self.slopes, window=self.window, chunk=self.chunk, gate=gate)

    def forward(self, x, ctx, cache):
        if self.o_weight is None:
            if self.o_tensor is None:
                raise RuntimeError("this attention's output projection was taken by the mixer it is a part of")
            self.o_weight = Weight(self.take_output_projection(), keep_plain=self.runtime.keep_plain_weights)
        y = linear(self.forward_inner(x, ctx, cache), self.o_weight, out_dtype=torch.float32, partials=True)
        return kernels.add_bias(y, self.o_bias) if self.o_bias is not None else y


register_part("mixer", "bucket_bias_attention", BucketBiasAttention)
