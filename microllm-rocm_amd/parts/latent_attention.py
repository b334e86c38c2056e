"""Attention whose keys and values are projections of one cached latent vector a token.

Queries go through a latent of their own: ``cq = norm(Wdq x)``, ``q = Wuq cq``, laid out head by head as ``[dim
unrotated | rot_dim rotated]``. ``Wdkv x`` gives ``kv_rank + rot_dim`` numbers: the first ``kv_rank``, normed, are the
latent ``c``; the last ``rot_dim``, turned by the token's position, are one key part ``kr`` that all heads share. Both
norms are RMS norms with a plain weight. Head ``h`` has keys ``Wuk_h c`` and values ``Wuv_h c``; a query at ``p`` sees
the keys ``j`` with ``0 <= p - j < window``, scores are ``(q_flat . Wuk_h c_j + q_rot . kr_j) * scale``, the softmax
is the ordinary one, the heads side by side are multiplied by ``sigmoid(Wg x)`` (``output_gate``) and projected by
``Wo``. A layer with ``owns_kv`` False has no ``Wdkv``: it reads the latents another run entry cached. Without a
``q_rank`` the queries have no latent: ``q = Wq x``. With ``gate_a_head`` the gate is one number a head, ``Wg`` being
``[heads, hidden]``. With a position encoding that turns neighbouring channels together (``rope_neighbours``) the rows
of ``Wq`` (or ``Wuq``) and ``Wdkv`` that make the turned parts are brought into split-half order once, at load: the turned
parts of queries and keys only ever meet in their dot product, which does not change when both are reordered alike.

Only ``[c | kr]`` is cached, one row a token. The up projections are folded into the query and into the result:
``q'_h = Wuk_h^T q_flat`` (``kv_rank`` numbers) and ``o_h = Wuv_h sum_j p_j c_j``, so the attention has a single kv
head whose key is the cached row and whose value is its first ``kv_rank`` entries, and every head reads the same
rows. In bfloat16, with rows of a multiple of 16 up to 256 elements, the rows lie in the paged attention's own pages
(``PagedKVNeed`` with one kv head, the row as key and as value) and the attention runs on its MFMA kernels; anything
else (float32, other sizes) lies in plain pages (``PagedLatentNeed``) and runs on the kernel that takes a wave per token
and head. The products per head are a batched library product for bfloat16 steps of many rows and this package's
kernel otherwise.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..ops import kernels
from .attention import QueryTilePlanner
from .base import MATRIX, Mixer, PagedKVNeed, PagedLatentNeed, Runtime, TensorDecl, VECTOR
from .linear import MEDIUM_ROWS, Weight, linear, linear_into_stream, takes_unscaled
from .registry import build_part, register_part
from .spec import PartSpec


class LatentAttention(Mixer):
    graph_safe = True
    fuses_residual = True
    BATCHED_ROWS = MEDIUM_ROWS     # bfloat16 steps of more rows take the library's batched product for the per-head products

    def __init__(self, spec: PartSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["heads"])
        self.dim = int(p["dim"])
        self.rot_dim = int(p["rot_dim"])
        self.vdim = int(p["vdim"])
        self.q_rank = int(p["q_rank"]) if p.get("q_rank") else 0       # 0: queries straight from the input
        self.kv_rank = int(p["kv_rank"])
        self.scale = float(p["scale"])
        self.window = int(p["window"]) if p.get("window") else 0
        # how long the cached rows are kept: the widest window of the layers that read them (0: for ever)
        self.kept_window = int(p.get("kept_window") or 0) if self.window else 0
        self.eps = float(p.get("eps", 1e-6))
        self.owns_kv = bool(p.get("owns_kv", True))
        self.output_gate = bool(p.get("output_gate", False))
        self.gate_a_head = bool(p.get("gate_a_head", False))
        if self.window and self.kept_window < self.window:
            raise ValueError("the cached rows must be kept at least as long as this layer's window")
        self.position = build_part("position", p["position"], runtime)
        if not self.position.fused_split_half or 2 * self.position.inv_freq.shape[0] != self.rot_dim:
            raise ValueError("the rotated part turns whole, by the split-half rule")
        self.row = self.kv_rank + self.rot_dim
        self.tiled = bool(p.get("mfma", True)) and runtime.dtype == torch.bfloat16 and self.row % 16 == 0 and self.row <= 256
        self.planner = QueryTilePlanner(bool(self.window)) if self.tiled else None
        self.q_width = self.heads * (self.dim + self.rot_dim)
        self.gate_width = (self.heads if self.gate_a_head else self.heads * self.vdim) if self.output_gate else 0
        self.q_at = 0
        self.kv_at = self.q_rank or self.q_width
        self.gate_at = self.kv_at + (self.row if self.owns_kv else 0)
        self.in_weight: Optional[Weight] = None
        self.uq_weight: Optional[Weight] = None
        self.o_weight: Optional[Weight] = None
        self.q_norm = self.kv_norm = self.fold_keys = self.unfold_values = None

    def tensors(self) -> Dict[str, TensorDecl]:
        inner = self.heads * self.vdim
        decls = {self.name("uk"): TensorDecl((self.heads * self.dim, self.kv_rank), MATRIX),
                 self.name("uv"): TensorDecl((inner, self.kv_rank), MATRIX),
                 self.name("o"): TensorDecl((self.hidden, inner), MATRIX)}
        if self.q_rank:
            decls[self.name("dq")] = TensorDecl((self.q_rank, self.hidden), MATRIX)
            decls[self.name("dq_norm")] = TensorDecl((self.q_rank,), VECTOR)
            decls[self.name("uq")] = TensorDecl((self.q_width, self.q_rank), MATRIX)
        else:
            decls[self.name("q")] = TensorDecl((self.q_width, self.hidden), MATRIX)
        if self.owns_kv:
            decls[self.name("dkv")] = TensorDecl((self.row, self.hidden), MATRIX)
            decls[self.name("dkv_norm")] = TensorDecl((self.kv_rank,), VECTOR)
        if self.output_gate:
            decls[self.name("g")] = TensorDecl((self.gate_width, self.hidden), MATRIX)
        return decls

    def _turned_rows_reordered(self, weight: torch.Tensor, vectors: int, first: int, stride: int) -> torch.Tensor:
        """``weight``'s rows that make the turned parts (``vectors`` runs of ``rot_dim`` rows, the first at ``first``,
        ``stride`` apart) brought into the order the position encoding turns them in."""
        order = self.position.split_half_order().to(weight.device)
        rows = torch.arange(weight.shape[0], device=weight.device)
        for vector in range(vectors):
            at = first + vector * stride
            rows[at:at + self.rot_dim] = at + order
        return weight[rows].contiguous()

    def bind(self, tensors: Mapping[str, torch.Tensor]) -> None:
        roles = ["dq" if self.q_rank else "q"] + (["dkv"] if self.owns_kv else []) + (["g"] if self.output_gate else [])
        weights = [tensors[self.name(role)] for role in roles]
        reorder = hasattr(self.position, "split_half_order")     # queries' and keys' turned channels, both alike
        if reorder and not self.q_rank:
            weights[0] = self._turned_rows_reordered(weights[0], self.heads, self.dim, self.dim + self.rot_dim)
        if reorder and self.owns_kv:
            weights[1] = self._turned_rows_reordered(weights[1], 1, self.kv_rank, 0)
        if len({w.dtype for w in weights}) != 1:
            raise TypeError("the projections of one layer must share a dtype to be stacked")
        keep = self.runtime.keep_plain_weights
        self.in_weight = Weight(torch.cat(weights, dim=0).contiguous() if len(weights) > 1 else weights[0], keep_plain=keep)
        del weights
        self.o_weight = Weight(tensors[self.name("o")], keep_plain=keep)
        if self.q_rank:
            uq = tensors[self.name("uq")]
            if reorder:
                uq = self._turned_rows_reordered(uq, self.heads, self.dim, self.dim + self.rot_dim)
            self.uq_weight = Weight(uq, keep_plain=keep)
            self.q_norm = tensors[self.name("dq_norm")]
        if self.owns_kv:
            self.kv_norm = tensors[self.name("dkv_norm")]
        # per head [in, out]: Wuk_h as stored maps the latent to the head's dims, so read along its rows it folds a query
        self.fold_keys = tensors[self.name("uk")].view(self.heads, self.dim, self.kv_rank).contiguous()
        self.unfold_values = tensors[self.name("uv")].view(self.heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()

    def sub_parts(self):
        return (self.position,)

    def step_planner(self):
        return self.planner

    def cache_need(self):
        if not self.owns_kv:
            return None
        window = self.kept_window or None
        return PagedKVNeed(1, self.row, window) if self.tiled else PagedLatentNeed(self.row, window)

    def flops(self, tokens: int) -> float:
        window = self.window or tokens
        pairs = sum(min(position + 1, window) for position in range(tokens))
        per_head = 2.0 * tokens * self.heads * self.kv_rank * (self.dim + self.vdim)
        return super().flops(tokens) + per_head + 2.0 * self.heads * (self.row + self.kv_rank) * pairs

    def takes_unscaled(self, rows: int) -> bool:
        return takes_unscaled(self.in_weight, rows)

    def forward(self, x, ctx, cache, residual=None):
        view = ctx.paged[cache.group]
        dtype = self.runtime.dtype
        n_tokens = x.shape[0]
        proj = linear(x, self.in_weight, out_dtype=torch.float32)     # applies the rows' factors where x comes without them
        device = proj.device
        cos_sin = self.position.table(ctx)
        stored = dict(pages=None, k_pages=None, v_pages=None, tiled_page_size=0)
        if self.owns_kv and self.tiled:
            stored = dict(pages=None, k_pages=cache.k, v_pages=cache.v, tiled_page_size=view.page_size)
        elif self.owns_kv:
            stored = dict(pages=cache.rows, k_pages=None, v_pages=None, tiled_page_size=0)
        cq = kernels.latent_prepare(proj, self.q_at, self.q_rank, self.q_norm, self.kv_at, self.kv_rank, self.rot_dim, self.kv_norm,
                                    self.eps, cos_sin, view.slot_mapping if self.owns_kv else None, dtype, **stored)
        # the queries: through their latent, or columns of the stacked product; rounded once, after folding and rotation
        q = linear(cq, self.uq_weight, out_dtype=torch.float32) if self.q_rank else proj[:, :self.q_width]
        q_full = torch.empty((n_tokens, self.heads * self.row), dtype=dtype, device=device)
        batched = dtype == torch.bfloat16 and n_tokens > self.BATCHED_ROWS
        if batched:
            flat = kernels.latent_query(q, self.heads, self.dim, self.rot_dim, self.kv_rank, cos_sin, q_full, want_flat=True)
            folded = torch.bmm(flat, self.fold_keys)
            kernels.latent_query(q, self.heads, self.dim, self.rot_dim, self.kv_rank, cos_sin, q_full, folded=folded)
        else:
            kernels.head_product(q.view(n_tokens, self.heads, self.dim + self.rot_dim)[:, :, :self.dim], self.fold_keys,
                           q_full.view(n_tokens, self.heads, self.row)[:, :, :self.kv_rank])
            kernels.latent_query(q, self.heads, self.dim, self.rot_dim, self.kv_rank, cos_sin, q_full)
        if self.tiled:
            found = kernels.paged_attention(q_full, cache.k, cache.v, view, ctx, self.scale, self.window, self.heads, 1, self.row,
                                            planner=self.planner)
            weighted = found.view(n_tokens, self.heads, self.row)[:, :, :self.kv_rank]
        else:
            weighted = kernels.latent_attention(q_full, cache.rows, view.block_table, ctx.seq_of_token, ctx.positions, self.scale,
                                                self.window, self.heads, self.kv_rank, self.rot_dim)
        gate = proj[:, self.gate_at:self.gate_at + self.gate_width] if self.output_gate else None
        if batched:
            o = kernels.gate_heads(torch.bmm(weighted.transpose(0, 1), self.unfold_values), gate, gate_a_head=self.gate_a_head)
        else:
            o = torch.empty((n_tokens, self.heads * self.vdim), dtype=dtype, device=device)
            kernels.head_product(weighted, self.unfold_values, o.view(n_tokens, self.heads, self.vdim), gate=gate,
                                 gate_a_head=self.gate_a_head)
        if residual is not None:
            begun = linear_into_stream(o, self.o_weight, residual)
            if begun is not None:
                return begun
        return linear(o, self.o_weight, out_dtype=torch.float32, partials=True)


register_part("mixer", "latent_attention", LatentAttention)
