"""Python bindings of the HIP kernels: shape and type checks on the host, then one launch.

Every function takes torch tensors on the GPU, launches on torch's current HIP
stream and returns the output tensor. Checks happen here, before the launch, so
a kernel never sees operands that do not fit what its grid assumes.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, NamedTuple, Optional, Sequence, Tuple

import torch

from . import library
from .library import KernelLibraryError

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def _code(dtype: torch.dtype) -> int:
    if dtype not in _CODES:
        raise KernelLibraryError(f"kernels take float32 or bfloat16, got {dtype}")
    return _CODES[dtype]


def _ptr(tensor: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if tensor is None else tensor.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)


def _stream() -> ctypes.c_void_p:
    """The current stream of the current device (asked on every launch: a few microseconds through the public
    interface, a fraction of one through the call torch's own compiled code uses)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(status: int, lib) -> None:
    if status != 0:
        raise KernelLibraryError(lib.mll_last_error().decode("utf-8", "replace"))


def _need(condition: bool, text: str) -> None:
    if not condition:
        raise KernelLibraryError(text)


def _device_tensor(tensor: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None) -> None:
    if tensor.is_cuda and tensor.is_contiguous() and (dtype is None or tensor.dtype == dtype):
        return
    _need(tensor.is_cuda, f"{name} must live on the GPU")
    _need(tensor.is_contiguous(), f"{name} must be contiguous")
    _need(tensor.dtype == dtype, f"{name} must be {dtype}, got {tensor.dtype}")


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """``table[ids] * scale`` as float32 rows."""
    lib = library.load()
    _device_tensor(table, "embedding table")
    _device_tensor(ids, "token ids", torch.int32)
    _need(table.dim() == 2 and ids.dim() == 1, "embedding takes a [vocab, width] table and [tokens] ids")
    vocab, width = table.shape
    if out is None:
        out = torch.empty((ids.shape[0], width), dtype=torch.float32, device=table.device)
    _device_tensor(out, "embedding output", torch.float32)
    _need(tuple(out.shape) == (ids.shape[0], width), "embedding output has the wrong shape")
    _check(lib.mll_embedding(_ptr(table), _code(table.dtype), _ptr(ids), _ptr(out),
                             ids.shape[0], width, vocab, ctypes.c_float(scale), _stream()), lib)
    return out


def rms_norm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_h: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out = rms_norm(h[rows] + delta[rows]) * weight``; with ``write_h`` the sum replaces ``h``."""
    lib = library.load()
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(weight, "norm weight", torch.float32)
    _need(h.dim() == 2 and weight.dim() == 1 and weight.shape[0] == h.shape[1],
          "rms_norm weight must match the last dimension")
    width = h.shape[1]
    delta_code, n_partials = F32, 1
    if delta is not None:
        _device_tensor(delta, "delta")
        _need(delta.dtype in (torch.float32, out_dtype), "delta must be float32 or have the output's dtype")
        if delta.dim() == 3:   # partial sums [parts, rows, width], added in order
            n_partials = delta.shape[0]
            _need(n_partials >= 1 and tuple(delta.shape[1:]) == tuple(h.shape), "delta parts must have the residual stream's shape")
        else:
            _need(tuple(delta.shape) == tuple(h.shape), "delta must have the residual stream's shape")
        delta_code = _code(delta.dtype)
    if rows is not None:
        _device_tensor(rows, "row selection", torch.int32)
        _need(not write_h, "cannot write h through a row selection")
        n_rows = rows.shape[0]
    else:
        n_rows = h.shape[0]
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=h.device)
    _device_tensor(out, "norm output", out_dtype)
    _need(tuple(out.shape) == (n_rows, width), "norm output has the wrong shape")
    _check(lib.mll_rms_norm(_ptr(h), _ptr(delta), delta_code, n_partials, ctypes.c_int64(h.numel()), _ptr(rows),
                            _ptr(weight), ctypes.c_float(eps), _ptr(out),
                            _code(out_dtype), n_rows, width, int(write_h), _stream()), lib)
    return out


def rms_norm_after(h: torch.Tensor, delta: torch.Tensor, after_weight: torch.Tensor, after_eps: float, mult: float,
                   weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                   write_h: bool = False, extra: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``v = h[rows] + mult * rms_norm(delta[rows]) * after_weight`` (``delta`` may be float32 partial sums ``[parts,
    tokens, width]``, added in order first), plus ``extra[rows]`` (float32 rows like ``h``'s) if given; with ``write_h`` the
    sum replaces ``h``; returns ``rms_norm(v) * weight``, or None without ``weight``."""
    lib = library.load()
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(after_weight, "norm weight of the delta", torch.float32)
    _need(h.dim() == 2 and tuple(after_weight.shape) == (h.shape[1],), "the delta's norm weight must match the stream's width")
    width = h.shape[1]
    _device_tensor(delta, "delta")
    _need(delta.dtype in (torch.float32, out_dtype), "delta must be float32 or have the output's dtype")
    n_partials = 1
    if delta.dim() == 3:
        n_partials = delta.shape[0]
        _need(n_partials >= 1 and tuple(delta.shape[1:]) == tuple(h.shape), "delta parts must have the residual stream's shape")
    else:
        _need(tuple(delta.shape) == tuple(h.shape), "delta must have the residual stream's shape")
    if rows is not None:
        _device_tensor(rows, "row selection", torch.int32)
        _need(not write_h, "cannot write h through a row selection")
        n_rows = rows.shape[0]
    else:
        n_rows = h.shape[0]
    if extra is not None:
        _device_tensor(extra, "further rows for the stream", torch.float32)
        _need(tuple(extra.shape) == tuple(h.shape), "the further rows must have the residual stream's shape")
    out = None
    if weight is not None:
        _device_tensor(weight, "norm weight", torch.float32)
        _need(tuple(weight.shape) == (width,), "the norm weight must match the stream's width")
        out = torch.empty((n_rows, width), dtype=out_dtype, device=h.device)
    _check(lib.mll_rms_norm_after(_ptr(h), _ptr(delta), _code(delta.dtype), n_partials, ctypes.c_int64(h.numel()), _ptr(rows),
                                  _ptr(after_weight), ctypes.c_float(after_eps), ctypes.c_float(mult), _ptr(extra), _ptr(weight),
                                  ctypes.c_float(eps), _ptr(out), _code(out_dtype), n_rows, width, int(write_h), _stream()), lib)
    return out


def add_bias(values: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``values[..., c] += bias[c]`` in place: float32 ``[rows, width]``, or partial sums ``[parts, rows, width]``, whose
    first part takes the bias."""
    lib = library.load()
    _device_tensor(values, "values", torch.float32)
    _device_tensor(bias, "bias", torch.float32)
    _need(values.dim() in (2, 3) and tuple(bias.shape) == (values.shape[-1],), "one bias a column")
    _check(lib.mll_add_bias(_ptr(values), _ptr(bias), ctypes.c_int64(values.shape[-2]), values.shape[-1], _stream()), lib)
    return values


def softcap(values: torch.Tensor, cap: float) -> torch.Tensor:
    """``cap * tanh(values / cap)`` in place (float32)."""
    lib = library.load()
    _device_tensor(values, "values", torch.float32)
    _check(lib.mll_softcap(_ptr(values), ctypes.c_int64(values.numel()), ctypes.c_float(cap), _stream()), lib)
    return values


ACTIVATIONS = {"silu": 0, "gelu_erf": 1, "gelu_tanh": 2}


def activation(values: torch.Tensor, kind: str, out_dtype: torch.dtype) -> torch.Tensor:
    """``act(values)`` element by element in ``out_dtype``; ``values`` is float32 (then it may be partial sums ``[parts,
    rows, width]``, added in order first) or has ``out_dtype``. ``kind``: ``silu``, ``gelu_erf`` (the exact gelu) or
    ``gelu_tanh``."""
    lib = library.load()
    _device_tensor(values, "values")
    _need(kind in ACTIVATIONS, f"unknown activation {kind!r}")
    _need(values.dtype in (torch.float32, out_dtype), "the values are float32 or have the output's dtype")
    n_parts, part_stride = 1, 0
    if values.dim() == 3:
        _need(values.dtype == torch.float32, "partial sums are float32")
        n_parts, part_stride = values.shape[0], values.shape[1] * values.shape[2]
    out = torch.empty(tuple(values.shape[-2:]) if values.dim() == 3 else tuple(values.shape), dtype=out_dtype, device=values.device)
    _check(lib.mll_activation(_ptr(values), _code(values.dtype), n_parts, ctypes.c_int64(part_stride), _ptr(out), _code(out_dtype),
                              ctypes.c_int64(out.numel()), ACTIVATIONS[kind], _stream()), lib)
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(delta, "delta")
    _need(tuple(delta.shape) == tuple(h.shape) and h.dim() == 2, "delta must have the residual stream's shape")
    _check(lib.mll_residual_add(_ptr(h), _ptr(delta), _code(delta.dtype), h.shape[0], h.shape[1], _stream()), lib)
    return h


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """``[tokens, n_freq, 2]`` float32: cos and sin of ``position * inv_freq``, the angle taken in float64."""
    lib = library.load()
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(inv_freq, "inverse frequencies", torch.float64)
    _need(positions.dim() == 1 and inv_freq.dim() == 1 and inv_freq.shape[0] > 0, "rope_table takes [tokens] and [n_freq]")
    out = torch.empty((positions.shape[0], inv_freq.shape[0], 2), dtype=torch.float32, device=positions.device)
    _check(lib.mll_rope_table(_ptr(positions), _ptr(inv_freq), inv_freq.shape[0], positions.shape[0], _ptr(out), _stream()), lib)
    return out


def qkv_rope_store(qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                   slot_mapping: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   heads: int, kv_heads: int, head_dim: int, page_size: int, out_dtype: torch.dtype,
                   q_out: Optional[torch.Tensor] = None, pair_order: bool = False,
                   cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Bias, rotation and page write of fused projections ``[tokens, (heads + 2 kv_heads) * head_dim]``.

    ``qkv`` is float32 or ``out_dtype``; the rotated queries and the pages have ``out_dtype``. The rotation
    takes ``cos_sin`` (``rope_table``'s, for these tokens) or computes the same from ``inv_freq``. With
    ``pair_order`` the query and key heads of ``qkv`` come in ``rotary_pair_order``."""
    lib = library.load()
    _device_tensor(qkv, "qkv")
    _need(qkv.dtype in (torch.float32, out_dtype), "qkv must be float32 or have the output's dtype")
    total = (heads + 2 * kv_heads) * head_dim
    n_partials = 1
    if qkv.dim() == 3:   # partial sums [parts, tokens, total], added in order
        n_partials = qkv.shape[0]
        _need(n_partials >= 1, "qkv needs at least one part")
    n_tokens = qkv.shape[-2]
    _need(qkv.dim() in (2, 3) and qkv.shape[-1] == total, f"qkv must be [tokens, {total}]")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    _device_tensor(positions, "positions", torch.int32)
    _need(tuple(positions.shape) == (n_tokens,), "positions must hold one entry per token")
    n_freq = 0
    if inv_freq is not None:
        _device_tensor(inv_freq, "inverse frequencies", torch.float64)
        n_freq = inv_freq.shape[0]
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == n_tokens and cos_sin.shape[2] == 2, "the cos/sin table must be [tokens, n_freq, 2]")
        _need(inv_freq is None or cos_sin.shape[1] == n_freq, "the cos/sin table and inv_freq differ in size")
        n_freq = cos_sin.shape[1]
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (n_tokens,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, out_dtype, kv_heads, head_dim, page_size)
    if q_out is None:
        q_out = torch.empty((n_tokens, heads * head_dim), dtype=out_dtype, device=qkv.device)
    _device_tensor(q_out, "q output", out_dtype)
    _need(tuple(q_out.shape) == (n_tokens, heads * head_dim), "q output has the wrong shape")
    _check(lib.mll_qkv_rope_store(_ptr(qkv), _code(qkv.dtype), n_partials, ctypes.c_int64(n_tokens * total),
                                  _code(out_dtype), _ptr(bias), _ptr(positions), _ptr(slot_mapping),
                                  _ptr(inv_freq), _ptr(cos_sin), n_freq, _ptr(q_out), _ptr(k_cache), _ptr(v_cache),
                                  n_tokens, heads, kv_heads, head_dim, page_size, int(pair_order), _stream()), lib)
    return q_out


def rotary_pair_order(heads: int, kv_heads: int, head_dim: int, n_freq: int) -> torch.Tensor:
    """Row order of a stacked q/k/v weight that puts the two dims of a rotary pair side by side.

    In every query and key head rows ``2p`` and ``2p + 1`` become dims ``p`` and ``p + n_freq`` for
    ``p < n_freq``; the dims beyond the rotary part and the value heads stay where they are. Returns the
    old row of every new row."""
    _need(0 <= 2 * n_freq <= head_dim, "more rotary pairs than dims")
    within = torch.arange(head_dim)
    pairs = torch.stack([torch.arange(n_freq), torch.arange(n_freq) + n_freq], dim=1).reshape(-1)
    within[: 2 * n_freq] = pairs
    rows = []
    for head in range(heads + 2 * kv_heads):
        rotated = head < heads + kv_heads
        rows.append(head * head_dim + (within if rotated else torch.arange(head_dim)))
    return torch.cat(rows)


class _RowScale(ctypes.Structure):
    _fields_ = [("sumsq", ctypes.c_void_p), ("groups", ctypes.c_int), ("stride", ctypes.c_int), ("width", ctypes.c_int),
                ("eps", ctypes.c_float)]


class _ResidualNorm(ctypes.Structure):
    _fields_ = [("h", ctypes.c_void_p), ("norm_weight", ctypes.c_void_p), ("x_out", ctypes.c_void_p),
                ("sumsq_out", ctypes.c_void_p), ("sumsq_stride", ctypes.c_int)]


class RowScale(NamedTuple):
    """The rows' factors of an RMS norm that a product applies to its result: row ``r`` is multiplied by
    ``1 / sqrt(sumsq[r, :groups].sum() / width + eps)``. ``gemm_skinny_residual`` makes these."""
    sumsq: torch.Tensor     # float32 [rows, stride]; stride is a multiple of 4
    groups: int
    width: int
    eps: float


def _scale_argument(scale: Optional[RowScale], rows: int):
    if scale is None:
        return None
    _device_tensor(scale.sumsq, "sums of squares", torch.float32)
    _need(scale.sumsq.dim() == 2 and scale.sumsq.shape[0] == rows and rows <= 16, "row factors are [rows <= 16, stride]")
    _need(scale.sumsq.shape[1] % 4 == 0 and 0 < scale.groups <= scale.sumsq.shape[1], "rows of sums must be a multiple of 4 long")
    return ctypes.byref(_RowScale(_ptr(scale.sumsq), int(scale.groups), scale.sumsq.shape[1], int(scale.width), float(scale.eps)))


class _QkvStore(ctypes.Structure):
    _fields_ = [("bias", ctypes.c_void_p), ("slot_mapping", ctypes.c_void_p),
                ("cos_sin", ctypes.c_void_p), ("n_freq", ctypes.c_int), ("q_out", ctypes.c_void_p),
                ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p), ("heads", ctypes.c_int),
                ("kv_heads", ctypes.c_int), ("head_dim", ctypes.c_int), ("page_size", ctypes.c_int)]


def gemm_skinny_qkv(x: torch.Tensor, packed: torch.Tensor, bias: Optional[torch.Tensor],
                    slot_mapping: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                    heads: int, kv_heads: int, head_dim: int, page_size: int,
                    scale: Optional[RowScale] = None) -> torch.Tensor:
    """Queries, keys and values of at most 16 bfloat16 rows in one kernel: ``gemm_skinny`` finished by the work
    of ``qkv_rope_store``. ``packed`` is the stacked weight packed in ``rotary_pair_order``; ``cos_sin`` is
    ``rope_table``'s for these rows (none: no rotation). Returns the queries."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2 and x.shape[0] <= 16, "gemm_skinny_qkv takes [m <= 16, k] activations")
    m, k = x.shape
    total = (heads + 2 * kv_heads) * head_dim
    _need(k % 8 == 0 and head_dim % 16 == 0, "gemm_skinny_qkv needs k % 8 == 0 and head_dim % 16 == 0")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == total // 16
          and packed.shape[1] == -(-k // 32), "the packed weight does not fit the heads and k")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    n_freq = 0
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == m and cos_sin.shape[2] == 2, "the cos/sin table must be [rows, n_freq, 2]")
        n_freq = cos_sin.shape[1]
        _need(2 * n_freq <= head_dim, "more rotary pairs than dims")
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (m,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, torch.bfloat16, kv_heads, head_dim, page_size)
    q_out = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    store = _QkvStore(_ptr(bias), _ptr(slot_mapping), _ptr(cos_sin), n_freq, _ptr(q_out),
                      _ptr(k_cache), _ptr(v_cache), heads, kv_heads, head_dim, page_size)
    _check(lib.mll_gemm_skinny_qkv(_ptr(x), _ptr(packed), m, k, ctypes.byref(store), _scale_argument(scale, m), _stream()), lib)
    return q_out


def gemm_skinny_residual(x: torch.Tensor, packed: torch.Tensor, h: torch.Tensor, norm_weight: torch.Tensor,
                         width: int, eps: float, scale: Optional[RowScale] = None) -> Tuple[torch.Tensor, RowScale]:
    """``h += x @ W.T`` for at most 16 bfloat16 rows, and the RMS norm of the sum begun.

    Returns ``(h * norm_weight)`` in bfloat16, the norm's result but for the rows' factors, and those factors as
    a ``RowScale`` for the product that takes it."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _device_tensor(h, "residual stream", torch.float32)
    _device_tensor(norm_weight, "norm weight", torch.float32)
    _need(x.dim() == 2 and x.shape[0] <= 16, "gemm_skinny_residual takes [m <= 16, k] activations")
    m, k = x.shape
    _need(h.dim() == 2 and h.shape[0] == m and h.shape[1] == width, "the residual stream must be [m, n]")
    n = h.shape[1]
    _need(tuple(norm_weight.shape) == (n,), "the norm's weight must be [n]")
    _need(k % 8 == 0, "gemm_skinny_residual needs k to be a multiple of 8")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == -(-n // 16)
          and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    groups = -(-n // 16)
    x_out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, -(-groups // 4) * 4), dtype=torch.float32, device=x.device)
    residual = _ResidualNorm(_ptr(h), _ptr(norm_weight), _ptr(x_out), _ptr(sumsq), sumsq.shape[1])
    _check(lib.mll_gemm_skinny_residual(_ptr(x), _ptr(packed), m, n, k, ctypes.byref(residual), _scale_argument(scale, m),
                                        _stream()), lib)
    return x_out, RowScale(sumsq, groups, width, eps)


def _check_pages(k_cache, v_cache, dtype, kv_heads, head_dim, page_size=None) -> int:
    """Key and value pages must have the tiled shapes of ``cache.layout``; returns the page size."""
    from ..cache.layout import key_page_shape, value_page_shape
    _device_tensor(k_cache, "key pages", dtype)
    _device_tensor(v_cache, "value pages", dtype)
    _need(k_cache.dim() == 6 and v_cache.dim() == 4, "key pages must have 6 dimensions and value pages 4 (tiled layout)")
    found = k_cache.shape[2] * 16
    _need(page_size is None or page_size == found, "the pages do not have the page size given")
    pages = k_cache.shape[0]
    _need(tuple(k_cache.shape) == key_page_shape(pages, kv_heads, found, head_dim), "key pages have the wrong shape")
    _need(tuple(v_cache.shape) == value_page_shape(pages, kv_heads, found, head_dim), "value pages have the wrong shape")
    return found


def _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim) -> int:
    _device_tensor(q, "queries")
    _need(q.dim() == 2 and q.shape[1] == heads * head_dim, "queries must be [tokens, heads * head_dim]")
    page_size = _check_pages(k_cache, v_cache, q.dtype, kv_heads, head_dim)
    _device_tensor(block_table, "block table", torch.int32)
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    return page_size


ROWWISE_SPLIT_BELOW = 2048      # (token, head) rows: with fewer, a row's chunks of keys get a wave each


def rowwise_heads_a_wave(count: int) -> int:
    """Forces how many query heads of a kv head one wave of the float32 row-wise attention takes (1 to 8; 0 gives
    the choice back to the launch, which goes by the waves the step then has); returns the value before. Every
    count gives the same bits."""
    return int(library.load().mll_rowwise_heads_a_wave(int(count)))


def rowwise_chunks(longest: int, window: int) -> int:
    """The most chunks of keys (at absolute positions) that a row's visible keys can span, for rows that see at
    most ``longest`` keys' positions (position < longest)."""
    chunk = library.load().mll_paged_attention_rowwise_chunk()
    if window > 0:
        return min(-(-longest // chunk), (window + chunk - 2) // chunk + 1)
    return max(1, -(-longest // chunk))


def paged_attention_rowwise(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
                            out: Optional[torch.Tensor] = None, longest: Optional[int] = None,
                            split: Optional[bool] = None, usual: Optional[int] = None) -> torch.Tensor:
    """The plain attention kernel (any dtype, any head size). ``longest``: no position of the step reaches it
    (default: what the block table can hold). ``split``: a wave per chunk of keys and a merge, or a wave per row;
    by default by the number of rows. Both give the same bits. ``usual``: how far the step's rows reach now
    (default ``longest``, which may leave room for later steps of the same shape): how many query heads a wave
    of the float32 kernel takes goes by it, nothing else."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    n_tokens = q.shape[0]
    _device_tensor(seq_of_token, "request of token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(seq_of_token.shape[0] == n_tokens and positions.shape[0] == n_tokens,
          "request-of-token and positions must hold one entry per token")
    if out is None:
        out = torch.empty_like(q)
    _device_tensor(out, "attention output", q.dtype)
    _need(out.shape == q.shape, "attention output must have the queries' shape")
    capacity = block_table.shape[1] * page_size
    longest = capacity if longest is None else min(int(longest), capacity)
    if split is None:
        split = n_tokens * heads < ROWWISE_SPLIT_BELOW
    chunks = rowwise_chunks(max(longest, 1), window) if split else 0
    usual_chunks = rowwise_chunks(max(min(int(usual), longest), 1), window) if split and usual is not None else 0
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((n_tokens, heads, chunks, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_tokens, heads, chunks, 2), dtype=torch.float32, device=q.device)
    else:
        chunks = 0      # one chunk a row: the wave per row is the wave per chunk
    _check(lib.mll_paged_attention_rowwise(_ptr(q), _code(q.dtype), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                           block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out),
                                           _ptr(part_o), _ptr(part_ml), chunks, usual_chunks, ctypes.c_float(scale), int(window),
                                           n_tokens, heads, kv_heads, head_dim, page_size, _stream()), lib)
    return out


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of fused rows ``[tokens, 2 * width]`` (gate first)."""
    lib = library.load()
    _device_tensor(gate_up, "gate/up")
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gate/up must be [tokens, 2 * width]")
    n_tokens, double = gate_up.shape
    width = double // 2
    if out is None:
        out = torch.empty((n_tokens, width), dtype=gate_up.dtype, device=gate_up.device)
    _device_tensor(out, "silu_mul output", gate_up.dtype)
    _need(tuple(out.shape) == (n_tokens, width), "silu_mul output has the wrong shape")
    element = gate_up.element_size()
    for start in range(0, n_tokens, 65535):
        count = min(65535, n_tokens - start)
        gate_ptr = gate_up.data_ptr() + start * double * element
        _check(lib.mll_silu_mul(ctypes.c_void_p(gate_ptr), ctypes.c_void_p(gate_ptr + width * element),
                                ctypes.c_int64(double), ctypes.c_void_p(out.data_ptr() + start * width * element),
                                _code(gate_up.dtype), count, width, _stream()), lib)
    return out


def f32_small_variant(variant: int) -> int:
    """For measurements and tests: which kernel ``gemm_f32`` takes for at most 16 rows: 1 (an element a thread), 2
    (2 x 2 elements) or 4 (1 x 4; at most 8 rows); 0 gives the choice back. Returns the value before. The same
    bits whichever."""
    return int(library.load().mll_gemm_f32_small_variant(int(variant)))


def f32_splits(n: int, k: int) -> int:
    """Into how many parts ``gemm_f32`` may cut the reduction of a weight ``[n, k]``: the weight's shape decides,
    never the rows of a call, so that a row's bits are the same in every batch."""
    return int(library.load().mll_gemm_f32_splits(int(n), int(k)))


def gemm_f32(a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None, partials: bool = False) -> torch.Tensor:
    """``a @ weight.T (+ bias)`` in true float32 with a fixed order of additions per element. With ``partials``
    the result may come as ``[parts, m, n]`` (``f32_splits`` parts): sums over consecutive ranges of k, which the
    caller adds in order."""
    lib = library.load()
    _device_tensor(a, "gemm input", torch.float32)
    _device_tensor(weight, "gemm weight", torch.float32)
    _need(a.dim() == 2 and weight.dim() == 2 and a.shape[1] == weight.shape[1],
          "gemm takes [m, k] and [n, k]")
    m, k = a.shape
    n = weight.shape[0]
    if bias is not None:
        _device_tensor(bias, "gemm bias", torch.float32)
        _need(tuple(bias.shape) == (n,), "gemm bias has the wrong size")
    step = 65535 * 16
    splits = f32_splits(n, k) if partials and m <= step else 1
    shape = (m, n) if splits == 1 else (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=a.device)
    _device_tensor(out, "gemm output", torch.float32)
    _need(tuple(out.shape) == shape, "gemm output has the wrong shape")
    for start in range(0, max(m, 1), step):
        count = min(step, m - start)
        _check(lib.mll_gemm_f32(ctypes.c_void_p(a.data_ptr() + start * k * 4), _ptr(weight), _ptr(bias),
                                ctypes.c_void_p(out.data_ptr() + start * n * 4), count, n, k, splits, _stream()), lib)
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(logits, "logits", torch.float32)
    _need(logits.dim() == 2, "logits must be [rows, vocab]")
    rows, vocab = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    parts = torch.empty((rows, lib.mll_argmax_slices(vocab), 4), dtype=torch.int32, device=logits.device)
    _check(lib.mll_argmax(_ptr(logits), _ptr(out), _ptr(parts), rows, vocab, _stream()), lib)
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: Optional[torch.Tensor],
           uniform: torch.Tensor) -> torch.Tensor:
    lib = library.load()
    _device_tensor(logits, "logits", torch.float32)
    _need(logits.dim() == 2, "logits must be [rows, vocab]")
    rows = logits.shape[0]
    _device_tensor(temperature, "temperature", torch.float32)
    _device_tensor(uniform, "uniform", torch.float32)
    _need(temperature.shape[0] == rows and uniform.shape[0] == rows, "one temperature and uniform per row")
    if top_k is not None:
        _device_tensor(top_k, "top_k", torch.int32)
        _need(top_k.shape[0] == rows, "one top_k per row")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    workspace = torch.empty((lib.mll_sample_workspace(rows, logits.shape[1]) // 4,), dtype=torch.int32, device=logits.device)
    _check(lib.mll_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(uniform), _ptr(out), _ptr(workspace),
                          rows, logits.shape[1], _stream()), lib)
    return out


LIBRARY_TUNE_ROWS = 1024     # with library tuning on, bfloat16 products of this many rows or more are tuned,
LIBRARY_TUNE_DECODE_ROWS = 64     # and those of up to this many (the gate/up product of large decode batches); between
                                  # the two a serving engine meets too many shapes, and short tuning runs mislead
_library_tuning = {"on": False, "seen": set(), "plain": set()}


def set_library_tuning(on: bool, results_file: Optional[str] = None) -> None:
    """Let the library choose the algorithm of a large product by timing its candidates instead of by its
    heuristic (the reference has --bf16-algorithm-index for that, apps/hf_infer.cpp:73). This is PyTorch's
    TunableOp, and the switch is global to the process: the first bfloat16-result product of a new shape with
    ``LIBRARY_TUNE_ROWS`` rows or more (gate/up of a prompt), or with at most ``LIBRARY_TUNE_DECODE_ROWS``, then
    takes seconds; later ones of the shape run the fastest candidate (7B sizes, 2048 rows: 0.45 instead of
    0.52 ms), or the heuristic's choice where that proves faster when the two are timed by turns. Results are
    kept in ``results_file`` (default: a file of this user in the temporary folder) and found again by later
    processes."""
    import torch.cuda.tunable as tunable
    if on:
        if results_file is None:
            results_file = os.path.join(library.private_temporary_folder(), "tunableop_results.csv")
        tunable.set_filename(results_file)
        tunable.set_max_tuning_duration(30)
        tunable.set_max_tuning_iterations(10)
    tunable.enable(on)
    tunable.tuning_enable(False)     # switched on around the first product of a shape only
    _library_tuning["on"] = on


def library_tuning() -> bool:
    return _library_tuning["on"]


def _tune_product(x: torch.Tensor, transposed_weight: torch.Tensor, shape: Tuple[int, int, int]) -> None:
    """Tune one shape, then time the tuned choice and the heuristic's by turns: the tuner's own runs are short."""
    import torch.cuda.tunable as tunable
    _library_tuning["seen"].add(shape)
    tunable.tuning_enable(True)
    try:
        torch.mm(x, transposed_weight)
    finally:
        tunable.tuning_enable(False)
    times = {True: 0.0, False: 0.0}
    try:
        for _ in range(3):
            for tuned in (True, False):
                tunable.enable(tuned)
                torch.mm(x, transposed_weight)
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(10):
                    torch.mm(x, transposed_weight)
                stop.record()
                stop.synchronize()
                times[tuned] += start.elapsed_time(stop)
    finally:
        tunable.enable(True)
    if times[False] < times[True]:
        _library_tuning["plain"].add(shape)


def gemm_bf16(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``x @ weight.T`` for bfloat16 operands with float32 accumulation.

    The product itself is the library's (hipBLASLt through ``torch.mm``), as the
    reference uses the library for its large linears (src/ops/optimized.cpp:94-450).
    """
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(weight, "gemm weight", torch.bfloat16)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "gemm takes [m, k] and [n, k]")
    if out_dtype != torch.bfloat16:
        return torch.mm(x, weight.t(), out_dtype=out_dtype)
    if _library_tuning["on"]:
        shape = (x.shape[0], weight.shape[0], x.shape[1])
        tuned_rows = shape[0] >= LIBRARY_TUNE_ROWS or 0 < shape[0] <= LIBRARY_TUNE_DECODE_ROWS
        if tuned_rows and shape not in _library_tuning["seen"] and not torch.cuda.is_current_stream_capturing():
            _tune_product(x, weight.t(), shape)
        if shape in _library_tuning["plain"]:
            import torch.cuda.tunable as tunable
            tunable.enable(False)
            try:
                return torch.mm(x, weight.t())
            finally:
                tunable.enable(True)
    return torch.mm(x, weight.t())


LIBRARY_TILE = 256          # the library's products of many rows work in tiles of about 256 x 256
LIBRARY_WORKGROUPS = 224    # splitting the reduction pays while tiles x parts stay at or under this (of 256 compute units)
LIBRARY_SPLIT_LENGTH = 2048  # and every part of the reduction keeps at least this many terms


def library_splits(m: int, n: int, k: int) -> int:
    """Into how many ranges of the reduction ``gemm_bf16_split`` cuts a float32 product of ``m`` rows.

    The library takes one workgroup per tile of the result: a long reduction into a narrow result (a
    feed-forward's down projection) leaves most compute units idle. Measured on MI355X (m = 2048, n = 3584,
    k = 18944): 348 us whole, 205 us in two parts. Parts are powers of two up to 8; where the result's tiles do not
    fill their last round over the compute units to 90 % and the reduction has 16384 terms or more, four parts
    still gain (m = 4096 and 8192 at the sizes above)."""
    tiles = -(-m // LIBRARY_TILE) * -(-n // LIBRARY_TILE)
    best = 1
    for parts in (2, 4, 8):
        if k % (32 * parts) == 0 and k // parts >= LIBRARY_SPLIT_LENGTH and tiles * parts <= LIBRARY_WORKGROUPS:
            best = parts
    if best == 1 and k >= 16384 and k % 128 == 0:
        rounds = -(-tiles // 256)
        if tiles > LIBRARY_WORKGROUPS // 2 and tiles < 0.9 * 256 * rounds:
            best = 4
    return best


def gemm_bf16_split(x: torch.Tensor, weight: torch.Tensor, parts: int) -> torch.Tensor:
    """``x @ weight.T`` as ``[parts, m, n]`` float32 sums over ``parts`` equal ranges of the reduction, for the
    caller to add in order: one batched library product over strided views of both operands (no copies)."""
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(weight, "gemm weight", torch.bfloat16)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "gemm takes [m, k] and [n, k]")
    m, k = x.shape
    _need(parts >= 1 and k % parts == 0, f"{parts} parts do not divide a reduction of {k}")
    if parts == 1:
        return torch.mm(x, weight.t(), out_dtype=torch.float32).unsqueeze(0)
    length = k // parts
    a = x.view(m, parts, length).transpose(0, 1)                          # [parts, m, length]
    b = weight.view(weight.shape[0], parts, length).permute(1, 2, 0)      # [parts, length, n]
    return torch.bmm(a, b, out_dtype=torch.float32)


class _AttentionExtras(ctypes.Structure):
    _fields_ = [("bias", ctypes.c_void_p), ("longest", ctypes.c_int), ("sink", ctypes.c_void_p),
                ("out_scale", ctypes.c_float), ("out_stride", ctypes.c_int64), ("chunk", ctypes.c_int), ("gate", ctypes.c_void_p),
                ("gate_stride", ctypes.c_int64)]


class AttentionExtras(NamedTuple):
    """What the MFMA attention kernels take beyond scale and window: ``bias`` float32 ``[distances, heads]`` added to
    the scaled scores by ``min(distance, last row)``; ``sink`` float32 ``[heads]``, one more term ``exp(sink)`` of the
    softmax's denominator; a factor on the result; ``chunk``: a query at ``p`` sees the keys from ``floor(p / chunk) *
    chunk`` on (no window then); ``gate`` float32 ``[tokens, heads]`` (columns of a wider buffer allowed): a head's result
    is multiplied by ``sigmoid(gate)``."""
    bias: Optional[torch.Tensor] = None
    sink: Optional[torch.Tensor] = None
    out_scale: float = 1.0
    chunk: int = 0
    gate: Optional[torch.Tensor] = None


def prefill_bias_rows() -> int:
    """The most rows of a bias table that the prefill kernel takes."""
    return int(library.load().mll_paged_attention_prefill_bias_rows())


def _extras_argument(extras: Optional[AttentionExtras], heads: int, head_dim: int, out: torch.Tensor):
    if extras is None:
        _need(out.is_contiguous(), "the attention output must be contiguous")
        return None
    longest = 0
    if extras.bias is not None:
        _device_tensor(extras.bias, "bias by distance", torch.float32)
        _need(extras.bias.dim() == 2 and extras.bias.shape[1] == heads and extras.bias.shape[0] >= 1, "the bias is [distances, heads]")
        longest = extras.bias.shape[0] - 1
    if extras.sink is not None:
        _device_tensor(extras.sink, "sink", torch.float32)
        _need(tuple(extras.sink.shape) == (heads,), "one sink a head")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == heads * head_dim, "the output is [tokens, heads * head_dim] with unit column stride")
    stride = max(out.stride(0), heads * head_dim)
    gate_stride = 0
    if extras.gate is not None:
        gate = extras.gate
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and tuple(gate.shape) == (out.shape[0], heads)
              and gate.stride(1) == 1, "the gate is float32 [tokens, heads] with unit column stride")
        gate_stride = max(gate.stride(0), heads)
    _need(extras.chunk >= 0, "chunks of positions are positive, or 0 for none")
    return ctypes.byref(_AttentionExtras(extras.bias.data_ptr() if extras.bias is not None else None, longest,
                                         extras.sink.data_ptr() if extras.sink is not None else None,
                                         float(extras.out_scale), stride, int(extras.chunk),
                                         extras.gate.data_ptr() if extras.gate is not None else None, gate_stride))


def decode_splits(n_tokens: int, kv_heads: int, longest: int) -> int:
    """How many splits of the keys: about one workgroup per compute unit, at least 512 keys each, and 1024 where
    that alone fills the GPU (measured on MI355X: a wave keeps two pairs of key tiles on their way, so few long
    splits do as well as many short ones, and joining costs more the more there are)."""
    rows = max(1, n_tokens * kv_heads)
    splits = max(1, min(-(-256 // rows), longest // 512, 256))
    if splits > 1 and rows * splits >= 256 and longest // splits < 1024:
        splits //= 2
    return splits


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                           seq_of_token: torch.Tensor, positions: torch.Tensor, scale: float, window: int,
                           heads: int, kv_heads: int, head_dim: int, n_splits: int,
                           out: Optional[torch.Tensor] = None, token_ids: Optional[torch.Tensor] = None,
                           extras: Optional[AttentionExtras] = None) -> torch.Tensor:
    """The MFMA kernel for bfloat16 queries that each attend alone (one token per request).

    ``token_ids`` restricts the work to those rows of ``q`` (the other rows of ``out`` are left alone)."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    _need(q.dtype == torch.bfloat16, "the decode kernel takes bfloat16")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "the decode kernel takes head sizes in steps of 16 up to 256")
    _need(page_size % 16 == 0, "the decode kernel takes page sizes in steps of 16")
    n_rows = q.shape[0]
    _device_tensor(seq_of_token, "request of token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(seq_of_token.shape[0] == n_rows and positions.shape[0] == n_rows,
          "request-of-token and positions must hold one entry per token")
    n_tokens = n_rows
    if token_ids is not None:
        _device_tensor(token_ids, "token ids", torch.int32)
        _need(token_ids.dim() == 1 and token_ids.shape[0] <= n_rows, "token ids must list rows of q")
        n_tokens = token_ids.shape[0]
    if out is None:
        out = torch.empty_like(q)
    _need(out.is_cuda and out.dtype == q.dtype and out.shape == q.shape, "attention output must have the queries' shape and dtype")
    extra = _extras_argument(extras, heads, head_dim, out)
    part_o = part_ml = None
    if n_splits > 1:
        part_o = torch.empty((n_tokens, heads, n_splits, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_tokens, heads, n_splits, 2), dtype=torch.float32, device=q.device)
    _check(lib.mll_paged_attention_decode_extra(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                                _ptr(seq_of_token), _ptr(positions), _ptr(token_ids), ctypes.c_void_p(out.data_ptr()),
                                                _ptr(part_o), _ptr(part_ml), ctypes.c_float(scale), int(window), n_tokens, heads,
                                                kv_heads, head_dim, page_size, n_splits, extra, _stream()), lib)
    return out


QUERY_TILE = 128   # tokens of one request in one tile of the prefill attention kernel; a workgroup takes two tiles


def pair_query_tiles(tiles: Sequence[Tuple[int, int, int, int]], adjacent: bool = False) -> List[Tuple[int, int, int, int, int]]:
    """The prefill attention's workgroups from its tiles. ``tiles``: (request, first token in the flat list,
    tokens, position of the first token). Returns (request, first token, tokens, first token, tokens) rows, the
    workgroups with the most keys to walk first, so that the longest start first.

    A tile's work grows with its position (it sees every earlier key), so of one request's tiles the last goes
    with the first, the last but one with the second and so on: every workgroup of a request then walks about as
    many keys. With ``adjacent`` neighbours go together instead: under a window every tile sees about as many keys,
    and neighbours see nearly the same ones. A request's odd tile goes alone."""
    by_request: dict = {}
    for tile in tiles:
        by_request.setdefault(tile[0], []).append(tile)
    pairs = []
    for request, own in by_request.items():
        own.sort(key=lambda tile: tile[3])
        count = len(own)
        if adjacent:
            couples = [(own[i], own[i + 1] if i + 1 < count else None) for i in range(0, count, 2)]
        else:
            couples = [(own[count - 1 - i], own[i] if i != count - 1 - i else None) for i in range((count + 1) // 2)]
        for first, second in couples:
            weight = first[3] + first[2] + (second[3] + second[2] if second else 0)
            pairs.append((weight, (request, first[1], first[2], second[1] if second else 0, second[2] if second else 0)))
    pairs.sort(key=lambda pair: -pair[0])
    return [pair[1] for pair in pairs]


def paged_attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                            query_tiles: torch.Tensor, positions: torch.Tensor, scale: float, window: int,
                            heads: int, kv_heads: int, head_dim: int, out: Optional[torch.Tensor] = None,
                            extras: Optional[AttentionExtras] = None) -> torch.Tensor:
    """The MFMA kernel for bfloat16 portions of prompts; ``query_tiles`` rows are (request, first token, tokens,
    first token, tokens): two tiles of up to ``QUERY_TILE`` tokens of the request (``pair_query_tiles``)."""
    lib = library.load()
    page_size = _check_paged(q, k_cache, v_cache, block_table, heads, kv_heads, head_dim)
    _need(q.dtype == torch.bfloat16, "the prefill kernel takes bfloat16")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "the prefill kernel takes head sizes in steps of 16 up to 256")
    _device_tensor(query_tiles, "query tiles", torch.int32)
    _need(query_tiles.dim() == 2 and query_tiles.shape[1] == 5, "query tiles must be [workgroups, 5]")
    _device_tensor(positions, "positions", torch.int32)
    _need(positions.shape[0] == q.shape[0], "positions must hold one entry per token")
    if out is None:
        out = torch.empty_like(q)
    _need(out.is_cuda and out.dtype == q.dtype and out.shape == q.shape, "attention output must have the queries' shape and dtype")
    extra = _extras_argument(extras, heads, head_dim, out)
    _need(extras is None or extras.bias is None or extras.bias.shape[0] <= prefill_bias_rows(), "the bias table has too many rows for the prefill kernel")
    _check(lib.mll_paged_attention_prefill_extra(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                                 _ptr(query_tiles), query_tiles.shape[0], _ptr(positions), ctypes.c_void_p(out.data_ptr()),
                                                 ctypes.c_float(scale), int(window), heads, kv_heads, head_dim, page_size,
                                                 extra, _stream()), lib)
    return out


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, view, ctx,
                    scale: float, window: int, heads: int, kv_heads: int, head_dim: int, planner=None,
                    extras: Optional[AttentionExtras] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the step's queries over their requests' pages; chooses the kernel for the batch's shape.

    bfloat16 with a head size in steps of 16: the MFMA kernels, split over the keys when every request brings
    one token, tiled over the queries otherwise (``planner``: the attention part's, whose plan for the step
    holds the tiles). Everything else (float32, other head sizes): the plain kernel.
    """
    mfma_fits = q.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
    _need(mfma_fits or (extras is None and out is None), "a bias, a sink or an output of its own need the MFMA kernels")
    _need(extras is None or not (extras.chunk and window), "a window or chunks of positions, not both")
    if mfma_fits and ctx.max_count == 1:
        longest = max(ctx.planned_total, ctx.max_total)
        reach = window if window > 0 else (extras.chunk if extras is not None else 0)      # the most keys a query sees, 0: all
        visible = min(longest, reach) if reach > 0 else longest
        splits = decode_splits(ctx.n_tokens, kv_heads, visible)
        return paged_attention_decode(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                      scale, window, heads, kv_heads, head_dim, splits, out=out, extras=extras)
    if mfma_fits:
        # Portions go to the tiled kernel; requests that bring one token, if any, to the split kernel.
        _need(planner is not None, "portions of prompts need the attention part's planner for their tiles")
        plan = ctx.plan_of(planner)
        if out is None:
            out = torch.empty_like(q)
        if plan.tiles.shape[0] > 0:
            paged_attention_prefill(q, k_cache, v_cache, view.block_table, plan.tiles, ctx.positions,
                                    scale, window, heads, kv_heads, head_dim, out=out, extras=extras)
        if plan.single_tokens.shape[0] > 0:
            longest = max(plan.max_single_total, ctx.planned_total) if ctx.fixed else plan.max_single_total
            reach = window if window > 0 else (extras.chunk if extras is not None else 0)
            visible = min(longest, reach) if reach > 0 else longest
            splits = decode_splits(plan.single_tokens.shape[0], kv_heads, visible)
            paged_attention_decode(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                   scale, window, heads, kv_heads, head_dim, splits, out=out, token_ids=plan.single_tokens,
                                   extras=extras)
        return out
    return paged_attention_rowwise(q, k_cache, v_cache, view.block_table, ctx.seq_of_token, ctx.positions,
                                   scale, window, heads, kv_heads, head_dim, longest=max(ctx.planned_total, ctx.max_total),
                                   usual=ctx.max_total)


def pack_weight(weight: torch.Tensor, interleave_halves: bool = False,
                row_order: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The weight ``[n, k]`` in the order ``gemm_skinny`` streams it: ``[n/16, k/32, 4, 16, 8]``, zero padded.

    With ``interleave_halves`` rows ``i`` and ``n/2 + i`` become neighbours first (gate and up of a gated
    feed-forward), which is what the gated epilogue expects. With ``row_order`` new row ``i`` is old row
    ``row_order[i]``.
    """
    _need(weight.dim() == 2 and weight.dtype == torch.bfloat16, "pack_weight takes a bfloat16 matrix")
    n, k = weight.shape
    if row_order is not None:
        _need(not interleave_halves and tuple(row_order.shape) == (n,), "row_order must name every row once")
        weight = weight[row_order.to(weight.device)]
    if interleave_halves:
        _need(n % 2 == 0, "interleaving needs an even number of rows")
        weight = torch.stack([weight[: n // 2], weight[n // 2:]], dim=1).reshape(n, k)
    n_padded, k_padded = -(-n // 16) * 16, -(-k // 32) * 32
    if (n_padded, k_padded) != (n, k):
        padded = torch.zeros((n_padded, k_padded), dtype=weight.dtype, device=weight.device)
        padded[:n, :k] = weight
        weight = padded
    packed = weight.view(n_padded // 16, 16, k_padded // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return packed


SKINNY_MAX_ROWS = 64


def gemm_skinny(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32",
                scale: Optional[RowScale] = None) -> torch.Tensor:
    """``x @ W.T`` for at most 64 bfloat16 rows and a packed weight.

    ``f32``: float32 ``[m, n]``; ``bf16``: bfloat16 ``[m, n]``; ``gated``: bfloat16 ``[m, n / 2]`` of
    silu(gate) * up for interleaved rows. With ``scale`` (at most 16 rows) the rows of the product are
    multiplied by its factors first.
    """
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_skinny takes a packed weight")
    _need(x.dim() == 2, "gemm_skinny takes [m, k] activations")
    m, k = x.shape
    _need(m <= SKINNY_MAX_ROWS, "gemm_skinny takes at most 64 rows")
    _need(k % 8 == 0, "gemm_skinny needs k to be a multiple of 8")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    if epilogue == "f32":
        code, out = 0, torch.empty((m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_skinny(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, _scale_argument(scale, m), _stream()), lib)
    return out


MEDIUM_WORKGROUPS = 224     # workgroups of 8 waves that gemm_medium wants at least (MI355X has 256 compute units)
MEDIUM_WHOLE_WORKGROUPS = 128     # where the reduction cannot be split, two tiles a wave from this many workgroups on


def medium_plan(n: int, k: int, may_split: bool = True) -> Tuple[int, int, int]:
    """(tiles of W a wave takes, waves a workgroup, splits of k) for ``gemm_medium``.

    A function of the weight's shape alone, so that a row's sum does not depend on the other rows. Two tiles a
    wave halve the reads of the activations; they are taken where splitting k (at most 16 times, a stage of 256
    at least per split) still gives enough workgroups.
    """
    n_tiles = -(-n // 16)
    stages = -(-k // 256)
    most = 1
    while may_split and most * 2 <= min(16, stages):
        most *= 2
    tiles_per_wave = 2 if -(-n_tiles // 16) * most >= (MEDIUM_WORKGROUPS if may_split else MEDIUM_WHOLE_WORKGROUPS) else 1
    groups = -(-n_tiles // (8 * tiles_per_wave))
    splits = 1
    while splits < most and groups * splits < MEDIUM_WORKGROUPS:
        splits *= 2
    return tiles_per_wave, 8, splits


def gemm_medium(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32",
                plan: Optional[Tuple[int, int, int]] = None) -> torch.Tensor:
    """``x @ W.T`` for at most 64 bfloat16 rows ``[m, k]`` and a packed weight, activations shared through LDS.

    ``plan`` is ``medium_plan``'s by default; pass ``medium_plan(n, k, may_split=False)`` for a plain ``[m, n]``.

    ``f32``: float32 ``[m, n]``, or ``[splits, m, n]`` partial sums to be added in order when the plan splits k;
    ``bf16`` and ``gated`` as in ``gemm_skinny`` (they never split).
    """
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_medium takes a packed weight")
    _need(x.dim() == 2, "gemm_medium takes [m, k] activations")
    m, k = x.shape
    _need(m <= SKINNY_MAX_ROWS, "gemm_medium takes at most 64 rows")
    _need(k % 8 == 0, "gemm_medium needs k to be a multiple of 8")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == -(-k // 32), "the packed weight does not fit n and k")
    tiles_per_wave, waves, splits = plan if plan is not None else medium_plan(n, k, may_split=epilogue == "f32")
    _need(epilogue == "f32" or splits == 1, "only float32 partial sums can be split over k")
    if epilogue == "f32":
        code = 0
        out = torch.empty((splits, m, n) if splits > 1 else (m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_medium(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, tiles_per_wave, waves, splits, _stream()), lib)
    return out


TILED_TILE = 256            # gemm_tiled works in tiles of up to 256 x 256, stages of 64 of the reduction
COMPUTE_UNITS = 256         # of an MI355X: a workgroup of gemm_tiled has one to itself
TILED_SPLIT_STAGES = 8      # a part of the reduction keeps at least this many stages


def tiled_splits(m: int, n: int, k: int) -> int:
    """Into how many parts ``gemm_tiled`` cuts the reduction of a float32 product: while the result's tiles leave
    compute units idle (a workgroup a tile: 28 workgroups for 512 rows by 3584 columns), up to 8."""
    tiles = -(-m // TILED_TILE) * -(-n // TILED_TILE)
    stages = -(-k // 64)
    splits = 1
    while splits < 8 and tiles * splits * 2 <= LIBRARY_WORKGROUPS and stages // (splits * 2) >= TILED_SPLIT_STAGES:
        splits *= 2
    return splits


def tiled_tile_rows(m: int, n: int, splits: int = 1) -> int:
    """The rows of a workgroup's tile that ``gemm_tiled`` chooses for this product: 256, or fewer where that fills
    the compute units better. The result's bits do not depend on it."""
    return int(library.load().mll_tiled_tile_rows(m, n, splits))


def tiled_fill(m: int, n: int, splits: int = 1) -> float:
    """How much of the compute units' time ``gemm_tiled``'s workgroups fill for this product: workgroups over the
    places of the rounds of ``COMPUTE_UNITS`` they take (0.91 for 2048 x 4608 in tiles of 160 rows, 0.56 in tiles
    of 256)."""
    blocks = -(-m // tiled_tile_rows(m, n, splits)) * -(-n // TILED_TILE) * splits
    return blocks / (-(-blocks // COMPUTE_UNITS) * COMPUTE_UNITS)


def gemm_tiled(x: torch.Tensor, packed: torch.Tensor, n: int, epilogue: str = "f32", splits: int = 1,
               tile_rows: int = 0) -> torch.Tensor:
    """``x @ W.T`` for many bfloat16 rows and a packed weight, on this package's tiled MFMA kernel (0.9 to 1.1 of
    the library's untuned rate at 2048 rows and more, 1.1 to 1.4 PFLOP/s: for weights that are kept in the packed
    order alone). ``k`` must be
    a multiple of 32. With ``splits`` > 1 (float32 only) the result is ``[splits, m, n]`` sums over parts of the
    reduction for the caller to add in order."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2 and packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8), "gemm_tiled takes [m, k] and a packed weight")
    m, k = x.shape
    _need(k % 32 == 0, "gemm_tiled needs k to be a multiple of 32")
    _need(packed.shape[0] == -(-n // 16) and packed.shape[1] == k // 32, "the packed weight does not fit n and k")
    _need(splits >= 1 and (splits == 1 or epilogue == "f32"), "only the float32 epilogue takes the reduction in parts")
    if epilogue == "f32":
        code, out = 0, torch.empty((m, n) if splits == 1 else (splits, m, n), dtype=torch.float32, device=x.device)
    elif epilogue == "bf16":
        code, out = 1, torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    elif epilogue == "gated":
        _need(n % 2 == 0, "the gated epilogue needs an even number of weight rows")
        code, out = 2, torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    else:
        raise KernelLibraryError(f"unknown epilogue {epilogue!r}")
    _check(lib.mll_gemm_tiled(_ptr(x), _ptr(packed), _ptr(out), code, m, n, k, splits, tile_rows, _stream()), lib)
    return out


def gemm_tiled_qkv(x: torch.Tensor, packed: torch.Tensor, bias: Optional[torch.Tensor],
                   slot_mapping: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   heads: int, kv_heads: int, head_dim: int, page_size: int, tile_rows: int = 0) -> torch.Tensor:
    """Queries, keys and values of many bfloat16 rows in one kernel: ``gemm_tiled`` finished by the work of
    ``qkv_rope_store`` (arguments as ``gemm_skinny_qkv``'s; ``k`` a multiple of 32 and an even number of rotary
    pairs). The reduction is not taken in parts, so this pays where ``tiled_splits`` is 1. Returns the queries."""
    lib = library.load()
    _device_tensor(x, "gemm input", torch.bfloat16)
    _device_tensor(packed, "packed weight", torch.bfloat16)
    _need(x.dim() == 2, "gemm_tiled_qkv takes [m, k] activations")
    m, k = x.shape
    total = (heads + 2 * kv_heads) * head_dim
    _need(k % 32 == 0 and head_dim % 16 == 0, "gemm_tiled_qkv needs k % 32 == 0 and head_dim % 16 == 0")
    _need(packed.dim() == 5 and tuple(packed.shape[2:]) == (4, 16, 8) and packed.shape[0] == total // 16
          and packed.shape[1] == k // 32, "the packed weight does not fit the heads and k")
    if bias is not None:
        _device_tensor(bias, "qkv bias", torch.float32)
        _need(tuple(bias.shape) == (total,), "qkv bias has the wrong size")
    n_freq = 0
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] == m and cos_sin.shape[2] == 2, "the cos/sin table must be [rows, n_freq, 2]")
        n_freq = cos_sin.shape[1]
        _need(2 * n_freq <= head_dim and n_freq % 2 == 0, "gemm_tiled_qkv takes an even number of rotary pairs, at most head_dim / 2")
    if slot_mapping is not None:
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _need(tuple(slot_mapping.shape) == (m,), "slot mapping must hold one entry per token")
        _need(k_cache is not None and v_cache is not None, "slot mapping needs both caches")
        _check_pages(k_cache, v_cache, torch.bfloat16, kv_heads, head_dim, page_size)
    q_out = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    store = _QkvStore(_ptr(bias), _ptr(slot_mapping), _ptr(cos_sin), n_freq, _ptr(q_out),
                      _ptr(k_cache), _ptr(v_cache), heads, kv_heads, head_dim, page_size)
    _check(lib.mll_gemm_tiled_qkv(_ptr(x), _ptr(packed), m, k, ctypes.byref(store), tile_rows, _stream()), lib)
    return q_out


def measured_peaks(device: Optional[torch.device] = None, read_bytes: int = 4 << 30) -> dict:
    """What this GPU reaches on a kernel that only reads memory once and on one that only issues bfloat16 MFMAs:
    ``{"hbm_read_GBps": ..., "mfma_bf16_TFLOPs": ...}`` (the best of a few launches each; well under a second)."""
    lib = library.load()
    device = device or torch.device("cuda", torch.cuda.current_device())
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    data = torch.empty(read_bytes // 4, dtype=torch.int32, device=device).random_()
    units = torch.cuda.get_device_properties(device).multi_processor_count

    def best(launch, repeats: int = 5) -> float:
        launch()
        torch.cuda.synchronize(device)
        times = []
        for _ in range(repeats):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            launch()
            stop.record()
            stop.synchronize()
            times.append(start.elapsed_time(stop) * 1e-3)
        return min(times)

    # The rate depends on how many workgroups share the reading (measured on MI355X, 256 units: 6.9 TB/s with two
    # workgroups a unit, 5.5 with eight): the best of a few counts is what the GPU reaches.
    read_time = min(best(lambda: _check(lib.mll_measure_read(_ptr(data), ctypes.c_int64(data.numel() * 4), _ptr(sink),
                                                             units * per_unit, _stream()), lib), repeats=3)
                    for per_unit in (1, 2, 4, 8))
    iterations, blocks = 4096, units * 4       # four waves a SIMD: one wave alone issues at two thirds of this rate
    mfma_time = best(lambda: _check(lib.mll_measure_mfma(iterations, _ptr(sink), blocks, _stream()), lib))
    flops = blocks * 4 * iterations * 16 * 16384.0
    del data
    return {"hbm_read_GBps": round(read_bytes / read_time / 1e9, 1), "mfma_bf16_TFLOPs": round(flops / mfma_time / 1e12, 1)}


# ---- several copies of the residual stream; a norm with a mean; a sinusoidal position vector --------------------
def embedding_sinusoid(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, rates: torch.Tensor) -> torch.Tensor:
    """``table[ids] + wave(positions)`` in float32; entry 2i of the wave is ``sin(p * rates[i])``, entry 2i + 1 the
    cosine of the same angle (``rates``: float64, one per pair of columns)."""
    lib = library.load()
    _device_tensor(table, "embedding table")
    _device_tensor(ids, "token ids", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(rates, "rates of the position waves", torch.float64)
    _need(table.dim() == 2 and ids.dim() == 1 and positions.shape == ids.shape,
          "embedding_sinusoid takes a [vocab, width] table and [tokens] ids and positions")
    vocab, width = table.shape
    _need(tuple(rates.shape) == ((width + 1) // 2,), "one rate per pair of columns")
    out = torch.empty((ids.shape[0], width), dtype=torch.float32, device=table.device)
    _check(lib.mll_embedding_sinusoid(_ptr(table), _code(table.dtype), _ptr(ids), _ptr(positions), _ptr(rates), _ptr(out),
                                      ids.shape[0], width, vocab, _stream()), lib)
    return out


def stream_copies(h: torch.Tensor, copies: int) -> torch.Tensor:
    """``[tokens, width]`` -> ``[tokens, copies, width]``, every copy equal to the row."""
    lib = library.load()
    _device_tensor(h, "stream", torch.float32)
    _need(h.dim() == 2 and copies >= 1, "stream_copies takes [tokens, width] and a positive number of copies")
    out = torch.empty((h.shape[0], copies, h.shape[1]), dtype=torch.float32, device=h.device)
    _check(lib.mll_stream_copies(_ptr(h), _ptr(out), h.shape[0], h.shape[1], copies, _stream()), lib)
    return out


MAX_STREAMS = 8
MFMA_BIAS_ROWS = 4096     # rows of a bias table that the MFMA prefill kernel keeps in LDS (csrc/attention_prefill.hip)


def stream_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, rms: bool = False,
                delta: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                give: Optional[torch.Tensor] = None, take: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None, write_x: bool = False, want_out: bool = True) -> Optional[torch.Tensor]:
    """The write of one sublayer's result into the streams, the read for the next and the norm between them.

    ``x``: float32 ``[tokens, streams, width]`` (or ``[tokens, width]``: one stream). With ``delta`` (float32
    ``[tokens, width]`` or parts ``[parts, tokens, width]``, added in order): ``x'_t = sum_s mix[s, t] x_s + give[t]
    delta`` (``mix`` None: the identity, ``give`` None: ones), written back with ``write_x``. Then
    ``u = sum_t take[t] x'_t`` (None: ones) and the result ``(u - mean) / sqrt(var + eps) * weight`` (``rms``:
    ``u / sqrt(mean(u^2) + eps) * weight``) for the rows asked for; ``want_out`` False only writes the streams."""
    lib = library.load()
    _device_tensor(x, "streams", torch.float32)
    _need(x.dim() in (2, 3), "streams are [tokens, streams, width] or [tokens, width]")
    streams = x.shape[1] if x.dim() == 3 else 1
    width = x.shape[-1]
    _need(1 <= streams <= MAX_STREAMS, f"between 1 and {MAX_STREAMS} streams")
    n_parts, part_stride = 1, 0
    if delta is not None:
        _device_tensor(delta, "delta", torch.float32)
        if delta.dim() == 3:
            n_parts, part_stride = delta.shape[0], delta.shape[1] * delta.shape[2]
            _need(n_parts >= 1 and tuple(delta.shape[1:]) == (x.shape[0], width), "delta parts must be [parts, tokens, width]")
        else:
            _need(tuple(delta.shape) == (x.shape[0], width), "delta must be [tokens, width]")
    else:
        _need(mix is None and give is None and not write_x, "without a delta there is nothing to write")
    for name, tensor, shape in (("mix", mix, (streams, streams)), ("give", give, (streams,)), ("take", take, (streams,))):
        if tensor is not None:
            _device_tensor(tensor, name, torch.float32)
            _need(tuple(tensor.shape) == shape, f"{name} must have shape {shape}")
    if rows is not None:
        _device_tensor(rows, "row selection", torch.int32)
        _need(not write_x, "cannot write the streams through a row selection")
        n_rows = rows.shape[0]
    else:
        n_rows = x.shape[0]
    out = None
    if want_out:
        _need(weight is not None, "a norm needs its weight")
        _device_tensor(weight, "norm weight", torch.float32)
        _need(tuple(weight.shape) == (width,), "the norm weight must match the width")
        out = torch.empty((n_rows, width), dtype=out_dtype, device=x.device)
    _check(lib.mll_stream_norm(_ptr(x), _ptr(delta), n_parts, ctypes.c_int64(part_stride), _ptr(mix), _ptr(give), _ptr(take),
                               _ptr(rows), _ptr(weight), ctypes.c_float(eps), int(rms), _ptr(out), _code(out_dtype),
                               n_rows, streams, width, int(write_x), _stream()), lib)
    return out


def clamped_glu(gate_up: torch.Tensor, limit: float, slope: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``g * sigmoid(slope * g) * (u + 1)`` with ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)`` of float32
    rows ``[tokens, 2 * width]`` (gate first)."""
    lib = library.load()
    _device_tensor(gate_up, "gate/up", torch.float32)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gate/up must be [tokens, 2 * width]")
    n_tokens, width = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((n_tokens, width), dtype=out_dtype, device=gate_up.device)
    for start in range(0, n_tokens, 65535):
        count = min(65535, n_tokens - start)
        _check(lib.mll_clamped_glu(ctypes.c_void_p(gate_up.data_ptr() + start * 2 * width * 4),
                                   ctypes.c_void_p(out.data_ptr() + start * width * out.element_size()), _code(out_dtype),
                                   count, width, ctypes.c_float(limit), ctypes.c_float(slope), _stream()), lib)
    return out


# ---- attention with a bias by distance and a sink ----------------------------------------------------------------
def _parts_of(tensor: torch.Tensor, name: str) -> Tuple[int, int]:
    _device_tensor(tensor, name, torch.float32)
    _need(tensor.dim() in (2, 3), f"{name} must be [tokens, columns] or [parts, tokens, columns]")
    if tensor.dim() == 3:
        return tensor.shape[0], tensor.shape[1] * tensor.shape[2]
    return 1, 0


def qk_norm_store(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                  positions: torch.Tensor, slot_mapping: torch.Tensor, temp_coef: float, temp_every: int,
                  k_pages: torch.Tensor, v_pages: torch.Tensor, heads: int, kv_heads: int, key_dim: int, value_dim: int,
                  out_dtype: torch.dtype, tiled_page_size: int = 0, bias: Optional[torch.Tensor] = None,
                  normed: Optional[bool] = None, queries_only: bool = False, cos_sin: Optional[torch.Tensor] = None,
                  further_columns: int = 0) -> torch.Tensor:
    """Norm of queries and keys over their head, the queries' factor by position, keys and values into their pages
    (``[page, position, kv_head, dim]``, or with ``tiled_page_size`` the pages of ``cache.layout`` with that many
    positions each); returns the queries ``[tokens, heads * key_dim]``. ``bias`` (one number a column of a row) is
    added first. ``normed`` (by default: where weights are given) divides queries and keys by their root mean square
    also without weights. With ``queries_only`` the rows hold queries alone and nothing is stored (a layer that
    reads another's keys and values). With ``cos_sin`` (``rope_table``'s ``[tokens, n, 2]``) queries and keys are turned
    after their norm in their first ``2 n`` channels, channel ``i`` with ``i + n``. The rows may hold
    ``further_columns`` after the values (what another kernel reads from the same product)."""
    lib = library.load()
    n_parts, part_stride = _parts_of(qkv, "q/k/v")
    n_tokens = qkv.shape[-2]
    row_width = heads * key_dim if queries_only else (heads + kv_heads) * key_dim + kv_heads * value_dim
    _need(qkv.shape[-1] == row_width + further_columns, "q/k/v rows have the wrong width")
    row_stride = ctypes.c_int64(qkv.shape[-1])
    rot_dims = 0
    if cos_sin is not None:
        _device_tensor(cos_sin, "cos and sin of the positions", torch.float32)
        _need(cos_sin.dim() == 3 and cos_sin.shape[0] >= n_tokens and cos_sin.shape[2] == 2 and 2 * cos_sin.shape[1] <= key_dim,
              "cos and sin are [tokens, pairs, 2] with at most key_dim / 2 pairs")
        rot_dims = 2 * cos_sin.shape[1]
    _device_tensor(positions, "positions", torch.int32)
    _need(positions.shape[0] >= n_tokens, "a position for every token")
    if normed is None:
        normed = q_weight is not None
    if bias is not None:
        _device_tensor(bias, "projection bias", torch.float32)
        _need(tuple(bias.shape) == (row_width,), "one bias a column of a row")
    q_out = torch.empty((n_tokens, heads * key_dim), dtype=out_dtype, device=qkv.device)
    if queries_only:
        _need(q_weight is None or (q_weight.is_cuda and q_weight.dtype == torch.float32 and tuple(q_weight.shape) == (key_dim,)),
              "the query norm weight must be float32 of the head's size")
        _check(lib.mll_qk_norm_store(_ptr(qkv), n_parts, ctypes.c_int64(part_stride), _ptr(q_weight), _ptr(q_weight),
                                     ctypes.c_float(eps), _ptr(positions), None, ctypes.c_float(temp_coef),
                                     int(temp_every), _ptr(q_out), None, None, _code(out_dtype), n_tokens,
                                     heads, kv_heads, key_dim, value_dim, 0, _ptr(bias), int(normed), 1, row_stride, _ptr(cos_sin),
                                     rot_dims, _stream()), lib)
        return q_out
    _device_tensor(slot_mapping, "slot mapping", torch.int32)
    _need(slot_mapping.shape[0] >= n_tokens, "a slot for every token")
    for name, weight in (("query norm weight", q_weight), ("key norm weight", k_weight)):
        if weight is not None:
            _device_tensor(weight, name, torch.float32)
            _need(tuple(weight.shape) == (key_dim,), f"{name} must have the head's size")
    _device_tensor(k_pages, "key pages", out_dtype)
    _device_tensor(v_pages, "value pages", out_dtype)
    if tiled_page_size:
        _need(key_dim == value_dim, "tiled pages hold keys and values of one width")
        _check_pages(k_pages, v_pages, out_dtype, kv_heads, key_dim, tiled_page_size)
    else:
        _need(k_pages.dim() == 4 and tuple(k_pages.shape[2:]) == (kv_heads, key_dim), "key pages are [page, position, kv_head, key_dim]")
        _need(v_pages.dim() == 4 and tuple(v_pages.shape[2:]) == (kv_heads, value_dim) and v_pages.shape[:2] == k_pages.shape[:2],
              "value pages are [page, position, kv_head, value_dim]")
    _check(lib.mll_qk_norm_store(_ptr(qkv), n_parts, ctypes.c_int64(part_stride), _ptr(q_weight), _ptr(k_weight),
                                 ctypes.c_float(eps), _ptr(positions), _ptr(slot_mapping), ctypes.c_float(temp_coef),
                                 int(temp_every), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _code(out_dtype), n_tokens,
                                 heads, kv_heads, key_dim, value_dim, int(tiled_page_size), _ptr(bias), int(normed), 0,
                                 row_stride, _ptr(cos_sin), rot_dims, _stream()), lib)
    return q_out


def bias_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                   seq_of_token: torch.Tensor, positions: torch.Tensor, bias: Optional[torch.Tensor],
                   sink: Optional[torch.Tensor], scale: float, out_scale: float, heads: int, kv_heads: int, key_dim: int,
                   value_dim: int, out: Optional[torch.Tensor] = None, slopes: Optional[torch.Tensor] = None,
                   window: int = 0, chunk: int = 0, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention with ``bias[min(distance, last row), head]`` added to the scaled scores, ``slopes[head] *
    distance`` taken off them, and ``exp(sink[head])`` in the softmax's denominator; with ``window`` a query sees
    itself and the ``window - 1`` keys before it; with ``chunk`` the keys from ``floor(p / chunk) * chunk`` on; with ``gate``
    (float32 ``[tokens, heads]``, columns of a wider buffer allowed) a head's result is multiplied by ``sigmoid(gate)``;
    ``out`` may be columns of a wider buffer (its row stride is taken)."""
    lib = library.load()
    _device_tensor(q, "queries")
    n_tokens = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == heads * key_dim, "queries are [tokens, heads * key_dim]")
    _device_tensor(k_pages, "key pages", q.dtype)
    _device_tensor(v_pages, "value pages", q.dtype)
    _need(k_pages.dim() == 4 and tuple(k_pages.shape[2:]) == (kv_heads, key_dim), "key pages are [page, position, kv_head, key_dim]")
    _need(v_pages.dim() == 4 and tuple(v_pages.shape[2:]) == (kv_heads, value_dim) and v_pages.shape[:2] == k_pages.shape[:2],
          "value pages are [page, position, kv_head, value_dim]")
    page_size = k_pages.shape[1]
    _device_tensor(block_table, "block table", torch.int32)
    _device_tensor(seq_of_token, "request of every token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(block_table.dim() == 2 and seq_of_token.shape[0] >= n_tokens and positions.shape[0] >= n_tokens,
          "a block table [requests, width] and a request and a position for every token")
    longest = 0
    if bias is not None:
        _device_tensor(bias, "bias by distance", torch.float32)
        _need(bias.dim() == 2 and bias.shape[1] == heads and bias.shape[0] >= 1, "the bias is [distances, heads]")
        longest = bias.shape[0] - 1
    if sink is not None:
        _device_tensor(sink, "sink", torch.float32)
        _need(tuple(sink.shape) == (heads,), "one sink a head")
    if slopes is not None:
        _device_tensor(slopes, "slopes", torch.float32)
        _need(tuple(slopes.shape) == (heads,), "one slope a head")
    _need(window >= 0 and chunk >= 0 and not (window and chunk), "a window or chunks of positions (0 for none), not both")
    gate_stride = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and tuple(gate.shape) == (n_tokens, heads)
              and gate.stride(1) == 1, "the gate is float32 [tokens, heads] with unit column stride")
        gate_stride = max(gate.stride(0), heads)
    if out is None:
        out = torch.empty((n_tokens, heads * value_dim), dtype=q.dtype, device=q.device)
    _need(out.is_cuda and out.dtype == q.dtype and out.dim() == 2 and tuple(out.shape) == (n_tokens, heads * value_dim)
          and out.stride(1) == 1, "the output is [tokens, heads * value_dim] with unit column stride")
    _check(lib.mll_bias_attention(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), block_table.shape[1],
                                  _ptr(seq_of_token), _ptr(positions), _ptr(bias), longest, _ptr(sink),
                                  ctypes.c_void_p(out.data_ptr()), ctypes.c_int64(out.stride(0) if n_tokens > 1 else max(out.stride(0), heads * value_dim)),
                                  _code(q.dtype), n_tokens, heads, kv_heads, key_dim, value_dim, page_size,
                                  ctypes.c_float(scale), ctypes.c_float(out_scale), _ptr(slopes), int(window), int(chunk),
                                  ctypes.c_void_p(gate.data_ptr()) if gate is not None else None, ctypes.c_int64(gate_stride), _stream()), lib)
    return out


# ---- gated linear attention -----------------------------------------------------------------------------------
def gla_decay(proj: torch.Tensor, low_offset: int, a2: torch.Tensor, bias: Optional[torch.Tensor], tau: float) -> torch.Tensor:
    """``sigmoid(a2 @ low + bias)^(1 / tau)`` per token and key channel, ``low`` being columns of ``proj``'s rows."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(a2, "decay weight")
    _need(proj.dim() == 2 and a2.dim() == 2, "projections [tokens, columns] and a decay weight [channels, rank]")
    channels, rank = a2.shape
    if bias is not None:
        _device_tensor(bias, "decay bias", torch.float32)
        _need(tuple(bias.shape) == (channels,), "one bias a channel")
    n_tokens = proj.shape[0]
    decay = torch.empty((n_tokens, channels), dtype=torch.float32, device=proj.device)
    for start in range(0, n_tokens, 65535):
        count = min(65535, n_tokens - start)
        _check(lib.mll_gla_decay(ctypes.c_void_p(proj.data_ptr() + start * proj.shape[1] * 4), ctypes.c_int64(proj.shape[1]),
                                 low_offset, rank, _ptr(a2), _code(a2.dtype), _ptr(bias), ctypes.c_float(tau),
                                 ctypes.c_void_p(decay.data_ptr() + start * channels * 4), count, channels, _stream()), lib)
    return decay


def gla_scan(proj: torch.Tensor, q_offset: int, k_offset: int, v_offset: int, decay: torch.Tensor, state: torch.Tensor,
             cu_tokens: torch.Tensor, slots: torch.Tensor, n_seqs: int, heads: int, key_dim: int, value_dim: int,
             q_scale: float, long_portions: bool = False) -> torch.Tensor:
    """The recurrence over every request's tokens of the step; ``state`` is ``[slots, heads, key_dim, value_dim]``
    float32, read and written at ``slots``. Returns ``[tokens, heads * value_dim]`` float32. ``long_portions``: the
    kernel that stages tiles of tokens through LDS, for steps whose requests bring many tokens (the same bits)."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(decay, "decays", torch.float32)
    _device_tensor(state, "state", torch.float32)
    _device_tensor(cu_tokens, "token offsets", torch.int32)
    _device_tensor(slots, "state slots", torch.int32)
    n_tokens = proj.shape[0]
    _need(proj.dim() == 2 and tuple(decay.shape) in ((n_tokens, heads * key_dim), (heads * key_dim,)),
          "decays are [tokens, heads * key_dim], or [heads * key_dim] for every token alike")
    decay_stride = heads * key_dim if decay.dim() == 2 else 0
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (heads, key_dim, value_dim), "state is [slots, heads, key_dim, value_dim]")
    _need(cu_tokens.shape[0] >= n_seqs + 1 and slots.shape[0] >= n_seqs, "offsets and slots for every request")
    out = torch.empty((n_tokens, heads * value_dim), dtype=torch.float32, device=proj.device)
    _check(lib.mll_gla_scan(_ptr(proj), ctypes.c_int64(proj.shape[1]), q_offset, k_offset, v_offset, _ptr(decay), _ptr(state),
                            _ptr(cu_tokens), _ptr(slots), _ptr(out), n_seqs, heads, key_dim, value_dim,
                            ctypes.c_float(q_scale), int(long_portions), ctypes.c_int64(decay_stride), _stream()), lib)
    return out


def gla_gate(o: torch.Tensor, proj: torch.Tensor, gate_offset: int, weight: Optional[torch.Tensor], eps: float, heads: int,
             value_dim: int, out_scale: float, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per head: ``o / rms(o) * weight * silu(gate) * out_scale`` (``weight`` None: none); ``out`` may be columns of a wider buffer."""
    lib = library.load()
    _device_tensor(o, "recurrence output", torch.float32)
    _device_tensor(proj, "projections", torch.float32)
    if weight is not None:
        _device_tensor(weight, "norm weight", torch.float32)
    n_tokens = o.shape[0]
    _need(tuple(o.shape) == (n_tokens, heads * value_dim) and proj.shape[0] == n_tokens and (weight is None or tuple(weight.shape) == (value_dim,)),
          "gla_gate takes [tokens, heads * value_dim], the projections of the same tokens and a weight [value_dim]")
    if out is None:
        out = torch.empty((n_tokens, heads * value_dim), dtype=out_dtype, device=o.device)
    _need(out.is_cuda and out.dtype == out_dtype and tuple(out.shape) == (n_tokens, heads * value_dim) and out.stride(1) == 1,
          "the output is [tokens, heads * value_dim] with unit column stride")
    _check(lib.mll_gla_gate(_ptr(o), _ptr(proj), ctypes.c_int64(proj.shape[1]), gate_offset, _ptr(weight), ctypes.c_float(eps),
                            ctypes.c_void_p(out.data_ptr()), ctypes.c_int64(max(out.stride(0), heads * value_dim)), _code(out_dtype),
                            n_tokens, heads, value_dim, ctypes.c_float(out_scale), _stream()), lib)
    return out


# ---- the gated delta rule ----------------------------------------------------------------------------------------
def delta_prepare(proj: torch.Tensor, conv_at: int, taps: torch.Tensor, kept: Optional[torch.Tensor], seq_of_token: torch.Tensor,
                  cu_tokens: torch.Tensor, slots: torch.Tensor, beta_at: int, step_at: int, a_log: torch.Tensor,
                  dt_bias: torch.Tensor, key_heads: int, heads: int, key_dim: int, value_dim: int, q_factor: float,
                  unit_eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Queries, keys and values of a step's tokens from the float32 projections ``proj``: a causal convolution per
    channel over ``proj[:, conv_at:conv_at + channels]`` (``taps`` ``[channels, n_taps]``, the last column the token's
    own; before the step's first token the request's ``kept`` inputs ``[slots, n_taps - 1, channels]``), SiLU, unit
    vectors per query and key head, the queries times ``q_factor``; and per head ``beta = sigmoid(proj[:, beta_at +
    h])`` and ``g = exp(-exp(a_log[h]) * softplus(proj[:, step_at + h] + dt_bias[h]))``. Returns ``u`` ``[tokens,
    channels]`` (queries, keys, values) and ``gates`` ``[tokens, heads, 2]``, float32."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(taps, "convolution taps", torch.float32)
    channels = 2 * key_heads * key_dim + heads * value_dim
    _need(proj.dim() == 2 and taps.dim() == 2 and taps.shape[0] == channels, "taps are [channels, n_taps]")
    n_taps = taps.shape[1]
    n_tokens = proj.shape[0]
    _need(0 <= conv_at and conv_at + channels <= proj.shape[1] and 0 <= beta_at and beta_at + heads <= proj.shape[1]
          and 0 <= step_at and step_at + heads <= proj.shape[1], "the columns lie outside the projections' rows")
    if n_taps > 1:
        _device_tensor(kept, "kept inputs", torch.float32)
        _need(kept.dim() == 3 and tuple(kept.shape[1:]) == (n_taps - 1, channels), "kept inputs are [slots, n_taps - 1, channels]")
    for name, tensor in (("A_log", a_log), ("dt_bias", dt_bias)):
        _device_tensor(tensor, name, torch.float32)
        _need(tuple(tensor.shape) == (heads,), f"{name} holds one number a head")
    _device_tensor(seq_of_token, "request of every token", torch.int32)
    _device_tensor(cu_tokens, "token offsets", torch.int32)
    _device_tensor(slots, "state slots", torch.int32)
    _need(seq_of_token.shape[0] >= n_tokens, "a request for every token")
    u = torch.empty((n_tokens, channels), dtype=torch.float32, device=proj.device)
    gates = torch.empty((n_tokens, heads, 2), dtype=torch.float32, device=proj.device)
    _check(lib.mll_delta_prepare(_ptr(proj), ctypes.c_int64(proj.shape[1]), conv_at, _ptr(taps), _ptr(kept if n_taps > 1 else None),
                                 _ptr(seq_of_token), _ptr(cu_tokens), _ptr(slots), beta_at, step_at, _ptr(a_log), _ptr(dt_bias),
                                 _ptr(u), _ptr(gates), n_tokens, key_heads, heads, key_dim, value_dim, n_taps,
                                 ctypes.c_float(q_factor), ctypes.c_float(unit_eps), _stream()), lib)
    return u, gates


def conv_keep(proj: torch.Tensor, conv_at: int, kept: torch.Tensor, cu_tokens: torch.Tensor, slots: torch.Tensor, n_seqs: int) -> None:
    """``kept`` ``[slots, n_taps - 1, channels]`` receives every request's newest inputs ``proj[:, conv_at:conv_at +
    channels]`` of the step, older kept ones before them where the step brought fewer than ``n_taps - 1``."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(kept, "kept inputs", torch.float32)
    _need(proj.dim() == 2 and kept.dim() == 3, "projections [tokens, columns] and kept inputs [slots, n_taps - 1, channels]")
    channels, n_taps = kept.shape[2], kept.shape[1] + 1
    _need(0 <= conv_at and conv_at + channels <= proj.shape[1], "the convolution's columns lie outside the projections' rows")
    _device_tensor(cu_tokens, "token offsets", torch.int32)
    _device_tensor(slots, "state slots", torch.int32)
    _need(cu_tokens.shape[0] >= n_seqs + 1 and slots.shape[0] >= n_seqs, "offsets and slots for every request")
    _check(lib.mll_conv_keep(_ptr(proj), ctypes.c_int64(proj.shape[1]), conv_at, _ptr(kept), _ptr(cu_tokens), _ptr(slots), n_seqs,
                             channels, n_taps, _stream()), lib)


def delta_scan(u: torch.Tensor, gates: torch.Tensor, state: torch.Tensor, cu_tokens: torch.Tensor, slots: torch.Tensor,
               n_seqs: int, key_heads: int, heads: int, key_dim: int, value_dim: int, long_portions: bool = False) -> torch.Tensor:
    """The delta rule over every request's tokens of the step, in order: ``S *= g; c = beta (v - S^T k); S += k c^T;
    o = S^T q`` with ``S = state[slot, head]`` (``[slots, heads, key_dim, value_dim]`` float32, read first and written
    last). ``u`` and ``gates`` as ``delta_prepare`` returns them. Returns ``[tokens, heads * value_dim]`` float32.
    ``long_portions``: the kernel that stages tiles of tokens through LDS, for steps whose requests bring many tokens
    (the same bits)."""
    lib = library.load()
    _device_tensor(u, "queries, keys and values", torch.float32)
    _device_tensor(gates, "gates", torch.float32)
    _device_tensor(state, "state", torch.float32)
    _device_tensor(cu_tokens, "token offsets", torch.int32)
    _device_tensor(slots, "state slots", torch.int32)
    n_tokens = u.shape[0]
    _need(u.dim() == 2 and u.shape[1] == 2 * key_heads * key_dim + heads * value_dim, "u is [tokens, queries | keys | values]")
    _need(tuple(gates.shape) == (n_tokens, heads, 2), "gates are [tokens, heads, 2]")
    _need(state.dim() == 4 and tuple(state.shape[1:]) == (heads, key_dim, value_dim), "state is [slots, heads, key_dim, value_dim]")
    _need(cu_tokens.shape[0] >= n_seqs + 1 and slots.shape[0] >= n_seqs, "offsets and slots for every request")
    out = torch.empty((n_tokens, heads * value_dim), dtype=torch.float32, device=u.device)
    _need(u.is_contiguous() and gates.is_contiguous(), "u and gates are contiguous")
    _check(lib.mll_delta_scan(_ptr(u), _ptr(gates), _ptr(state), _ptr(cu_tokens), _ptr(slots), _ptr(out), n_seqs, key_heads, heads,
                              key_dim, value_dim, int(long_portions), _stream()), lib)
    return out


# ---- attention through latents -----------------------------------------------------------------------------------
def latent_prepare(proj: torch.Tensor, q_at: int, q_rank: int, q_weight: Optional[torch.Tensor], kv_at: int, kv_rank: int, rot_dim: int,
                   kv_weight: Optional[torch.Tensor], eps: float, cos_sin: Optional[torch.Tensor],
                   slot_mapping: Optional[torch.Tensor], out_dtype: torch.dtype, pages: Optional[torch.Tensor] = None,
                   k_pages: Optional[torch.Tensor] = None, v_pages: Optional[torch.Tensor] = None,
                   tiled_page_size: int = 0) -> Optional[torch.Tensor]:
    """The norms of a token's two latents from its float32 down projections ``proj`` ``[tokens, columns]``; returns the
    queries' normed latent ``[tokens, q_rank]`` (``q_rank`` 0: the queries have no latent, and None comes back). With ``slot_mapping`` the keys' normed latent and the turned key
    part go into ``pages`` ``[page, position, kv_rank + rot_dim]`` or, with ``tiled_page_size``, into key and value
    pages of ``cache.layout`` (one kv head of ``kv_rank + rot_dim`` dims, the same row in both)."""
    lib = library.load()
    _device_tensor(proj, "down projections", torch.float32)
    _need(proj.dim() == 2 and 0 <= q_at and q_at + q_rank <= proj.shape[1], "the queries' latent lies outside the projections' rows")
    if q_rank:
        _device_tensor(q_weight, "query latent norm weight", torch.float32)
        _need(tuple(q_weight.shape) == (q_rank,), "the queries' norm weight must match their latent")
    n_tokens = proj.shape[0]
    if slot_mapping is not None:
        _need(0 <= kv_at and kv_at + kv_rank + rot_dim <= proj.shape[1], "the keys' latent lies outside the projections' rows")
        _device_tensor(slot_mapping, "slot mapping", torch.int32)
        _device_tensor(kv_weight, "latent norm weight", torch.float32)
        _device_tensor(cos_sin, "cos/sin table", torch.float32)
        _need(slot_mapping.shape[0] >= n_tokens and tuple(kv_weight.shape) == (kv_rank,), "a slot a token and a weight a latent channel")
        _need(tuple(cos_sin.shape) == (n_tokens, rot_dim // 2, 2) and rot_dim % 2 == 0, "the cos/sin table must be [tokens, rot_dim / 2, 2]")
        if tiled_page_size:
            _check_pages(k_pages, v_pages, out_dtype, 1, kv_rank + rot_dim, tiled_page_size)
        else:
            _device_tensor(pages, "latent pages", out_dtype)
            _need(pages.dim() == 3 and pages.shape[2] == kv_rank + rot_dim, "latent pages are [page, position, kv_rank + rot_dim]")
    q_latent = torch.empty((n_tokens, q_rank), dtype=out_dtype, device=proj.device) if q_rank else None
    _check(lib.mll_latent_prepare(_ptr(proj), ctypes.c_int64(proj.shape[1]), q_at, q_rank, _ptr(q_weight if q_rank else None), kv_at, kv_rank, rot_dim,
                                  _ptr(kv_weight), ctypes.c_float(eps), _ptr(cos_sin), _ptr(slot_mapping), _ptr(q_latent),
                                  _ptr(pages), _ptr(k_pages), _ptr(v_pages), int(tiled_page_size), _code(out_dtype), n_tokens,
                                  _stream()), lib)
    return q_latent


def latent_query(q: torch.Tensor, heads: int, dim: int, rot_dim: int, kv_rank: int, cos_sin: torch.Tensor, q_full: torch.Tensor,
                 folded: Optional[torch.Tensor] = None, want_flat: bool = False) -> Optional[torch.Tensor]:
    """``q`` float32 ``[tokens, heads * (dim + rot_dim)]`` (may be columns of wider rows): the turned rotated parts go behind the folded parts in
    ``q_full`` ``[tokens, heads * (kv_rank + rot_dim)]``; ``folded`` ``[heads, tokens, kv_rank]`` is copied in front;
    with ``want_flat`` the unrotated parts are returned as ``[heads, tokens, dim]`` in ``q_full``'s dtype."""
    lib = library.load()
    _need(q.is_cuda and q.dtype == torch.float32 and q.dim() == 2 and q.stride(1) == 1, "queries are float32 rows with unit column stride")
    n_tokens = q.shape[0]
    _need(q.shape[1] == heads * (dim + rot_dim), "queries are [tokens, heads * (dim + rot_dim)]")
    q_stride = max(q.stride(0), q.shape[1])
    _device_tensor(cos_sin, "cos/sin table", torch.float32)
    _need(tuple(cos_sin.shape) == (n_tokens, rot_dim // 2, 2) and rot_dim % 2 == 0, "the cos/sin table must be [tokens, rot_dim / 2, 2]")
    _device_tensor(q_full, "folded queries")
    _need(tuple(q_full.shape) == (n_tokens, heads * (kv_rank + rot_dim)), "folded queries are [tokens, heads * (kv_rank + rot_dim)]")
    if folded is not None:
        _device_tensor(folded, "folded parts", q_full.dtype)
        _need(tuple(folded.shape) == (heads, n_tokens, kv_rank), "folded parts are [heads, tokens, kv_rank]")
    flat = torch.empty((heads, n_tokens, dim), dtype=q_full.dtype, device=q.device) if want_flat else None
    _check(lib.mll_latent_query(_ptr(q), ctypes.c_int64(q_stride), n_tokens, heads, dim, rot_dim, kv_rank, _ptr(cos_sin), _ptr(folded), _ptr(flat), _ptr(q_full),
                                _code(q_full.dtype), _stream()), lib)
    return flat


HEAD_PRODUCT_TYPES = {(torch.float32, torch.float32, torch.float32), (torch.float32, torch.bfloat16, torch.bfloat16),
                      (torch.bfloat16, torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16, torch.float32)}


def head_product(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None,
                 gate_a_head: bool = False) -> torch.Tensor:
    """``out[t, h, o] = sum_i x[t, h, i] * weight[h, i, o]``, times ``sigmoid(gate[t, h * n_out + o])`` with ``gate``
    (float32 rows), or times ``sigmoid(gate[t, h])`` with ``gate_a_head``. ``x`` ``[tokens, heads, n_in]`` and ``out`` ``[tokens, heads, n_out]`` may be views with strides of
    their own over tokens and heads (unit stride along the last axis); the weight is contiguous."""
    lib = library.load()
    _device_tensor(weight, "per-head weight")
    _need(weight.dim() == 3, "the weight is [heads, n_in, n_out]")
    heads, n_in, n_out = weight.shape
    _need(x.is_cuda and x.dim() == 3 and x.shape[1:] == (heads, n_in) and x.stride(2) == 1, "x is [tokens, heads, n_in] with unit stride along n_in")
    n_tokens = x.shape[0]
    _need(out.is_cuda and tuple(out.shape) == (n_tokens, heads, n_out) and out.stride(2) == 1, "out is [tokens, heads, n_out] with unit stride along n_out")
    _need((x.dtype, weight.dtype, out.dtype) in HEAD_PRODUCT_TYPES, f"head_product is not built for {x.dtype}, {weight.dtype}, {out.dtype}")
    gate_stride = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and gate.stride(1) == 1
              and gate.shape == (n_tokens, heads if gate_a_head else heads * n_out),
              "the gate is float32 [tokens, heads * n_out] (or [tokens, heads]) with unit column stride")
        gate_stride = gate.stride(0)
    _check(lib.mll_head_product(ctypes.c_void_p(x.data_ptr()), _code(x.dtype), ctypes.c_int64(x.stride(0)), ctypes.c_int64(x.stride(1)),
                                _ptr(weight), _code(weight.dtype), ctypes.c_void_p(out.data_ptr()), _code(out.dtype),
                                ctypes.c_int64(out.stride(0)), ctypes.c_int64(out.stride(1)),
                                ctypes.c_void_p(gate.data_ptr() if gate is not None else 0), ctypes.c_int64(gate_stride),
                                int(gate_a_head), n_tokens, heads, n_in, n_out, _stream()), lib)
    return out


def gate_heads(values: torch.Tensor, gate: Optional[torch.Tensor], gate_a_head: bool = False) -> torch.Tensor:
    """``[heads, tokens, n]`` (a batched product's result) -> ``[tokens, heads * n]``, times ``sigmoid(gate)`` (float32
    ``[tokens, heads * n]``, or ``[tokens, heads]`` with ``gate_a_head``; unit column stride) if given."""
    lib = library.load()
    _device_tensor(values, "values per head")
    _need(values.dim() == 3, "values are [heads, tokens, n]")
    heads, n_tokens, n = values.shape
    gate_stride = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and tuple(gate.shape) == (n_tokens, heads if gate_a_head else heads * n)
              and gate.stride(1) == 1, "the gate is float32 [tokens, heads * n] (or [tokens, heads]) with unit column stride")
        gate_stride = gate.stride(0)
    out = torch.empty((n_tokens, heads * n), dtype=values.dtype, device=values.device)
    _check(lib.mll_gate_heads(_ptr(values), ctypes.c_void_p(gate.data_ptr() if gate is not None else 0), ctypes.c_int64(gate_stride),
                              int(gate_a_head), _ptr(out), _code(values.dtype), n_tokens, heads, n, _stream()), lib)
    return out


def latent_attention(q_full: torch.Tensor, pages: torch.Tensor, block_table: torch.Tensor, seq_of_token: torch.Tensor,
                     positions: torch.Tensor, scale: float, window: int, heads: int, kv_rank: int, rot_dim: int) -> torch.Tensor:
    """Attention of folded queries ``[tokens, heads * (kv_rank + rot_dim)]`` over latent pages ``[page, position, kv_rank
    + rot_dim]``; returns the weighted latents ``[tokens, heads, kv_rank]``."""
    lib = library.load()
    _device_tensor(q_full, "folded queries")
    n_tokens = q_full.shape[0]
    width = kv_rank + rot_dim
    _need(q_full.dim() == 2 and q_full.shape[1] == heads * width, "folded queries are [tokens, heads * (kv_rank + rot_dim)]")
    _device_tensor(pages, "latent pages", q_full.dtype)
    _need(pages.dim() == 3 and pages.shape[2] == width, "latent pages are [page, position, kv_rank + rot_dim]")
    _device_tensor(block_table, "block table", torch.int32)
    _device_tensor(seq_of_token, "request of every token", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    _need(block_table.dim() == 2 and seq_of_token.shape[0] >= n_tokens and positions.shape[0] >= n_tokens,
          "a block table [requests, width] and a request and a position for every token")
    out = torch.empty((n_tokens, heads, kv_rank), dtype=q_full.dtype, device=q_full.device)
    _check(lib.mll_latent_attention(_ptr(q_full), _ptr(pages), _ptr(block_table), block_table.shape[1], _ptr(seq_of_token),
                                    _ptr(positions), _ptr(out), ctypes.c_int64(heads * kv_rank), ctypes.c_int64(kv_rank),
                                    _code(q_full.dtype), n_tokens, heads, kv_rank, rot_dim, pages.shape[1], int(window),
                                    ctypes.c_float(scale), _stream()), lib)
    return out


# ---- a recurrent block with a gated linear recurrence -----------------------------------------------------------------
def rglru_conv(proj: torch.Tensor, x_at: int, x_bias: Optional[torch.Tensor], taps: torch.Tensor, conv_bias: Optional[torch.Tensor],
               kept: torch.Tensor, seq_of_token: torch.Tensor, cu_tokens: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """The causal convolution per channel over ``proj[:, x_at : x_at + width] + x_bias``, continued from the inputs
    each request kept (``kept``: float32 ``[slots, taps - 1, width]``); float32 ``[tokens, width]``."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(taps, "taps")
    _need(proj.dim() == 2 and taps.dim() == 2, "projections [tokens, columns] and taps [width, taps]")
    width, n_taps = taps.shape
    _need(0 <= x_at and x_at + width <= proj.shape[1], "the convolution's input lies outside the projections' rows")
    for name, bias in (("input bias", x_bias), ("convolution bias", conv_bias)):
        if bias is not None:
            _device_tensor(bias, name, torch.float32)
            _need(tuple(bias.shape) == (width,), f"one {name} a channel")
    _device_tensor(kept, "kept inputs", torch.float32)
    _need(kept.dim() == 3 and tuple(kept.shape[1:]) == (n_taps - 1, width), "kept inputs are [slots, taps - 1, width]")
    n_tokens = proj.shape[0]
    for name, tensor in (("request of every token", seq_of_token), ("token offsets", cu_tokens), ("state slots", slots)):
        _device_tensor(tensor, name, torch.int32)
    _need(seq_of_token.shape[0] >= n_tokens, "a request for every token")
    u = torch.empty((n_tokens, width), dtype=torch.float32, device=proj.device)
    _check(lib.mll_rglru_conv(_ptr(proj), ctypes.c_int64(proj.shape[1]), x_at, _ptr(x_bias), _ptr(taps), _code(taps.dtype),
                              _ptr(conv_bias), _ptr(kept), _ptr(seq_of_token), _ptr(cu_tokens), _ptr(slots), _ptr(u), n_tokens, width,
                              n_taps, _stream()), lib)
    return u


def rglru_scan(proj: torch.Tensor, x_at: int, x_bias: Optional[torch.Tensor], y_at: int, y_bias: Optional[torch.Tensor],
               u: torch.Tensor, gates: torch.Tensor, r_bias: Optional[torch.Tensor], i_bias: Optional[torch.Tensor],
               lam: torch.Tensor, decay_scale: float, state: torch.Tensor, kept: torch.Tensor, cu_tokens: torch.Tensor,
               slots: torch.Tensor, n_seqs: int, blocks: int, n_taps: int, out_dtype: torch.dtype,
               chunked: bool = False) -> torch.Tensor:
    """The gated linear recurrence over every request's tokens of the step, times the gated branch; ``state`` float32
    ``[slots, width]`` and ``kept`` ``[slots, taps - 1, width]`` are read and written at ``slots``. Returns
    ``[tokens, width]`` in ``out_dtype``. ``chunked``: the recurrence in chunks of tokens that are walked side by
    side (for steps with long portions; the same result but for the rounding of the chunks' products)."""
    lib = library.load()
    _device_tensor(proj, "projections", torch.float32)
    _device_tensor(u, "convolution output", torch.float32)
    _device_tensor(gates, "gates", torch.float32)
    _device_tensor(lam, "decay parameter", torch.float32)
    _device_tensor(state, "state", torch.float32)
    _device_tensor(kept, "kept inputs", torch.float32)
    n_tokens, width = u.shape
    _need(proj.shape[0] == n_tokens and max(x_at, y_at) + width <= proj.shape[1], "the branches lie outside the projections' rows")
    _need(tuple(gates.shape) == (n_tokens, 2 * width) and tuple(lam.shape) == (width,) and width % blocks == 0, "gates are [tokens, 2 * width]")
    _need(state.dim() == 2 and state.shape[1] == width and kept.dim() == 3 and tuple(kept.shape[1:]) == (n_taps - 1, width)
          and kept.shape[0] == state.shape[0], "state is [slots, width], kept inputs [slots, taps - 1, width]")
    for name, bias in (("input bias", x_bias), ("branch bias", y_bias), ("gate bias", r_bias), ("gate bias", i_bias)):
        if bias is not None:
            _device_tensor(bias, name, torch.float32)
            _need(bias.numel() == width, f"one {name} a channel")
    _device_tensor(cu_tokens, "token offsets", torch.int32)
    _device_tensor(slots, "state slots", torch.int32)
    _need(cu_tokens.shape[0] >= n_seqs + 1 and slots.shape[0] >= n_seqs, "offsets and slots for every request")
    out = torch.empty((n_tokens, width), dtype=out_dtype, device=u.device)
    if chunked:
        scratch = torch.empty((int(lib.mll_rglru_scan_scratch(n_tokens, n_seqs, width)),), dtype=torch.float32, device=u.device)
        _check(lib.mll_rglru_scan_chunked(_ptr(proj), ctypes.c_int64(proj.shape[1]), x_at, _ptr(x_bias), y_at, _ptr(y_bias), _ptr(u),
                                          _ptr(gates), _ptr(r_bias), _ptr(i_bias), _ptr(lam), ctypes.c_float(decay_scale), _ptr(state),
                                          _ptr(kept), _ptr(cu_tokens), _ptr(slots), _ptr(out), _ptr(scratch), _code(out_dtype), n_tokens,
                                          n_seqs, width, blocks, n_taps, _stream()), lib)
        return out
    _check(lib.mll_rglru_scan(_ptr(proj), ctypes.c_int64(proj.shape[1]), x_at, _ptr(x_bias), y_at, _ptr(y_bias), _ptr(u), _ptr(gates),
                              _ptr(r_bias), _ptr(i_bias), _ptr(lam), ctypes.c_float(decay_scale), _ptr(state), _ptr(kept),
                              _ptr(cu_tokens), _ptr(slots), _ptr(out), _code(out_dtype), n_seqs, width, blocks, n_taps, _stream()), lib)
    return out


# ---- a mixture of experts ------------------------------------------------------------------------------------------
def router_logits(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ weight.T`` with float32 sums: ``x`` in its own dtype, ``weight`` float32 ``[rows, width]`` with few rows
    (a router's, and what rides with it)."""
    lib = library.load()
    _device_tensor(x, "router input")
    _device_tensor(weight, "router weight", torch.float32)
    _need(x.dim() == 2 and weight.dim() == 2 and weight.shape[1] == x.shape[1], "router_logits takes [tokens, width] and [rows, width]")
    z = torch.empty((x.shape[0], weight.shape[0]), dtype=torch.float32, device=x.device)
    _check(lib.mll_router_logits(_ptr(x), _code(x.dtype), _ptr(weight), _ptr(z), x.shape[0], weight.shape[0], x.shape[1], _stream()), lib)
    return z


def moe_route(z: torch.Tensor, experts: int, top: int, softmax_scores: bool = False, renormalize: bool = False,
              shared_at: int = -1, groups: int = 0, keep: int = 0):
    """The ``top`` experts of every token from router logits ``z`` float32 ``[tokens, columns]`` (experts first):
    ``(ids int32 [tokens, top], weights float32 [tokens, top], sigmoid(z[:, shared_at]) or None)``. With ``groups``
    the experts form that many equal groups of neighbours, a group counts as its best expert, and only experts of the
    ``keep`` best groups are chosen."""
    lib = library.load()
    _device_tensor(z, "router logits", torch.float32)
    _need(z.dim() == 2 and z.shape[1] >= experts and shared_at < z.shape[1], "router logits are [tokens, experts (+ gate)]")
    n_tokens = z.shape[0]
    ids = torch.empty((n_tokens, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((n_tokens, top), dtype=torch.float32, device=z.device)
    shared = torch.empty((n_tokens,), dtype=torch.float32, device=z.device) if shared_at >= 0 else None
    _check(lib.mll_moe_route(_ptr(z), ctypes.c_int64(z.shape[1]), n_tokens, experts, top, int(softmax_scores), int(renormalize),
                             int(shared_at), _ptr(ids), _ptr(weights), _ptr(shared), int(groups), int(keep), _stream()), lib)
    return ids, weights, shared


MOE_PAIRS_A_LAUNCH = 65535


MOE_GROUPED_PAIRS = 64      # from this many (token, choice) pairs on, bfloat16 experts multiply their rows in tiles


def moe_experts(x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor,
                weight_on_input: bool, out: Optional[torch.Tensor] = None, grouped: Optional[bool] = None, gated: bool = True,
                activation: str = "silu") -> torch.Tensor:
    """Every (token, choice) pair through its expert's gated feed-forward: ``gate_up`` ``[experts, 2 * ff, width]``
    (gate rows first), ``down`` ``[experts, width, ff]``. Returns float32 ``[top, tokens, width]``, a part per choice,
    for the reader to add in order (``out``: at least that many leading parts of a larger buffer). ``grouped``: the
    pairs sorted by expert and multiplied in tiles on the matrix units (bfloat16, widths in steps of 8) instead of
    one reading of the expert's weights a pair; by default by the number of pairs. With ``gated`` false an expert is
    ``down act(up x)`` and ``gate_up`` holds ``[experts, ff, width]``; ``activation`` is one of ``ACTIVATIONS``."""
    lib = library.load()
    _device_tensor(x, "expert input")
    _device_tensor(gate_up, "experts' gate and up weights", x.dtype)
    _device_tensor(down, "experts' down weights", x.dtype)
    _device_tensor(ids, "expert ids", torch.int32)
    _device_tensor(weights, "expert weights", torch.float32)
    n_tokens, width = x.shape
    top = ids.shape[1]
    experts, inner_rows, _ = gate_up.shape
    ff = inner_rows // 2 if gated else inner_rows
    _need(activation in ACTIVATIONS, f"unknown activation {activation!r}")
    act_code = ACTIVATIONS[activation]
    _need(gate_up.shape[2] == width and tuple(down.shape) == (experts, width, ff) and tuple(ids.shape) == (n_tokens, top)
          and tuple(weights.shape) == (n_tokens, top), "the experts' weights, ids and weights do not fit the input")
    if out is None:
        out = torch.empty((top, n_tokens, width), dtype=torch.float32, device=x.device)
    _device_tensor(out, "experts' output", torch.float32)
    _need(out.dim() == 3 and out.shape[0] >= top and tuple(out.shape[1:]) == (n_tokens, width), "the output is [parts >= top, tokens, width]")
    act = torch.empty((n_tokens * top, ff), dtype=x.dtype, device=x.device)
    if grouped is None:
        grouped = x.dtype == torch.bfloat16 and n_tokens * top >= MOE_GROUPED_PAIRS and width % 8 == 0 and ff % 8 == 0
    if grouped:
        _need(x.dtype == torch.bfloat16 and width % 8 == 0 and ff % 8 == 0, "the tiled experts take bfloat16 and widths in steps of 8")
        scratch = torch.empty((2 * experts + 1 + n_tokens * top,), dtype=torch.int32, device=x.device)
        counts, offsets, order = scratch[:experts], scratch[experts:2 * experts + 1], scratch[2 * experts + 1:]
        in_order = torch.empty((n_tokens * top, width), dtype=x.dtype, device=x.device)
        _check(lib.mll_moe_grouped(_ptr(x), _ptr(ids), _ptr(weights), top, _ptr(gate_up), _ptr(down), ctypes.c_void_p(counts.data_ptr()),
                                   ctypes.c_void_p(offsets.data_ptr()), ctypes.c_void_p(order.data_ptr()), _ptr(in_order), _ptr(act),
                                   _ptr(out), n_tokens, experts, width, ff, int(weight_on_input), int(gated), act_code, _stream()), lib)
        return out
    step = max(1, MOE_PAIRS_A_LAUNCH // top)       # tokens a launch: its grid has a row of workgroups a pair
    element = x.element_size()
    for first in range(0, n_tokens, step):
        count = min(step, n_tokens - first)
        here = dict(x=ctypes.c_void_p(x.data_ptr() + first * width * element), ids=ctypes.c_void_p(ids.data_ptr() + first * top * 4),
                    weights=ctypes.c_void_p(weights.data_ptr() + first * top * 4), act=ctypes.c_void_p(act.data_ptr() + first * top * ff * element))
        _check(lib.mll_moe_gate_up(here["x"], here["ids"], here["weights"], top, _ptr(gate_up), here["act"], _code(x.dtype), count, width, ff,
                                   int(weight_on_input), int(gated), act_code, _stream()), lib)
        # the output keeps its rows n_tokens apart in every part: the launch writes its tokens' rows of each
        _check(lib.mll_moe_down_rows(here["act"], here["ids"], here["weights"], top, _ptr(down), ctypes.c_void_p(out.data_ptr() + first * width * 4),
                                     _code(x.dtype), count, n_tokens, width, ff, int(weight_on_input), _stream()), lib)
    return out


def scale_rows(values: torch.Tensor, factor: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[t] = factor[t] * values[t]`` in float32; ``values`` may be parts ``[parts, tokens, width]``, added in order first."""
    lib = library.load()
    n_parts, part_stride = _parts_of(values, "values")
    _device_tensor(factor, "row factors", torch.float32)
    _device_tensor(out, "scaled rows", torch.float32)
    n_tokens, width = values.shape[-2], values.shape[-1]
    _need(tuple(out.shape) == (n_tokens, width) and factor.shape[0] >= n_tokens, "out is [tokens, width], one factor a token")
    _check(lib.mll_scale_rows(_ptr(values), n_parts, ctypes.c_int64(part_stride), _ptr(factor), _ptr(out), n_tokens, width, _stream()), lib)
    return out
