"""A plain, slow implementation of the Zabozen decoder on the CPU, one function per mechanism.

It shares no code with the engine: it takes the configuration as the dictionary that config.json holds and the
tensors by their file names, and computes every sequence whole, position by position where the mechanism is a
recurrence, in float64.

Notation. ``x`` is the residual stream ``[T, width]``; ``rms(a) = a / sqrt(mean(a^2) + eps)`` over the last axis.
A layer is ``x += m * (rms(M(rms(x) * w1)) * w1b)`` and then the same around the feed-forward with ``w2`` and ``w2b``;
``m`` is ``residual_mult``. The mixers:

* ``latent_attention``: ``q = Wq a`` head by head as ``[dim | rot_dim]``; ``Wdkv a`` gives the latent ``c``
  (``kv_rank`` numbers, RMS norm with a weight) and one key part ``r`` (``rot_dim`` numbers) for all heads; head
  ``h`` has keys ``[Wuk_h c | turn(r)]`` and values ``Wuv_h c``; causal softmax of ``scale * q . k``; the head's
  result times ``sigmoid(Wg a)_h``; ``Wo``. ``turn`` pairs dimension ``i`` with ``i + n/2`` of the ``n`` turned ones
  and turns the pair by ``p * base^(-2i/n)``.
* ``attention``: ``q, k, v`` with biases; ``q`` and ``k`` divided by their root mean square per head; query head
  ``h`` reads key/value head ``h // (H / G)``; ``score = scale * q . k - 2^(-8 (h + 1) / H) * (i - j)`` for
  ``0 <= i - j < window``; softmax; ``Wo`` with a bias. With ``kv_from`` the keys and values are those of another layer.
* ``delta``: ``q, k, v`` through a causal convolution per channel and SiLU; ``q`` and ``k`` unit vectors per head
  (``a / sqrt(sum(a^2) + 1e-6)``), ``q`` times ``dim^(-1/2)``; ``beta = sigmoid(Wb a)``, ``g = exp(-exp(A_log)
  softplus(Wa a + dt_bias))`` per head; ``S <- g S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``;
  ``rms(o) * w * silu(Wg a)``; ``Wo``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Tuple

import torch

F = torch.float64


def t64(tensors: Mapping[str, torch.Tensor], name: str) -> torch.Tensor:
    return tensors[name].to(F)


def rms(a: torch.Tensor, eps: float) -> torch.Tensor:
    return a / torch.sqrt((a * a).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def turn(a: torch.Tensor, positions: torch.Tensor, base: float, n: int) -> torch.Tensor:
    """``a`` is ``[T, ..., D]``; its first ``n`` dims are turned by the position, the rest pass."""
    half = n // 2
    rates = torch.tensor([base ** (-2.0 * i / n) for i in range(half)], dtype=F)
    angle = positions.to(F)[:, None] * rates[None, :]
    shape = [a.shape[0]] + [1] * (a.dim() - 2) + [half]
    cos, sin = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    u, v = a[..., :half], a[..., half:n]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, a[..., n:]], dim=-1)


def softmax_rows(scores: torch.Tensor, visible: torch.Tensor) -> torch.Tensor:
    scores = scores.masked_fill(~visible, float("-inf"))
    return torch.softmax(scores, dim=-1)


def latent_attention(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    T = a.shape[0]
    H, dim, rot, vdim, rank = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    positions = torch.arange(T)
    q = (a @ t64(tensors, f"{prefix}.q").T).view(T, H, dim + rot)
    down = a @ t64(tensors, f"{prefix}.dkv").T
    c = rms(down[:, :rank], eps) * t64(tensors, f"{prefix}.dkv.norm")
    r = turn(down[:, rank:], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    q_rot = turn(q[:, :, dim:], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    keys = (c @ t64(tensors, f"{prefix}.uk").T).view(T, H, dim)
    values = (c @ t64(tensors, f"{prefix}.uv").T).view(T, H, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q[:, :, :dim], keys) + torch.einsum("ihd,jd->hij", q_rot, r)) * mixer["scale"]
    visible = positions[:, None] >= positions[None, :]
    p = softmax_rows(scores, visible[None])
    o = torch.einsum("hij,jhd->ihd", p, values)
    gate = torch.sigmoid(a @ t64(tensors, f"{prefix}.g").T)       # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * vdim) @ t64(tensors, f"{prefix}.o").T


def attention_keys_values(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    T = a.shape[0]
    G, dim, vdim = mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    k = (a @ t64(tensors, f"{prefix}.k").T + t64(tensors, f"{prefix}.k.b")).view(T, G, dim)
    v = (a @ t64(tensors, f"{prefix}.v").T + t64(tensors, f"{prefix}.v.b")).view(T, G, vdim)
    return rms(k, eps), v


def head_slopes(heads: int) -> List[float]:
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def window_attention(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scale: float, window: int,
                     slopes: Optional[List[float]]) -> torch.Tensor:
    """``q [T, H, dim]``, ``keys [T, G, dim]``, ``values [T, G, vdim]`` -> ``[T, H, vdim]``: query ``i`` sees the keys
    ``j`` with ``0 <= i - j < window`` (``window`` 0: all ``j <= i``); ``slopes[h] * (i - j)`` is taken off the score."""
    T, H, G = q.shape[0], q.shape[1], keys.shape[1]
    positions = torch.arange(T)
    distance = positions[:, None] - positions[None, :]
    visible = (distance >= 0) & ((distance < window) if window else (distance >= 0))
    out = torch.zeros((T, H, values.shape[2]), dtype=F)
    for h in range(H):
        g = h // (H // G)
        scores = (q[:, h] @ keys[:, g].T) * scale
        if slopes is not None:
            scores = scores - slopes[h] * distance.to(F)
        out[:, h] = softmax_rows(scores, visible) @ values[:, g]
    return out


def attention(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float,
              keys: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    T = a.shape[0]
    H, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = rms((a @ t64(tensors, f"{prefix}.q").T + t64(tensors, f"{prefix}.q.b")).view(T, H, dim), eps)
    out = window_attention(q, keys, values, mixer["scale"], mixer["mask"]["size"], head_slopes(H))
    return out.reshape(T, H * vdim) @ t64(tensors, f"{prefix}.o").T + t64(tensors, f"{prefix}.o.b")


def short_convolution(a: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """``a`` is ``[T, C]``, ``taps`` ``[C, n]`` whose last column weighs the current token; zeros before the start."""
    T, n = a.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((n - 1, a.shape[1]), dtype=a.dtype), a], dim=0)
    out = torch.zeros_like(a)
    for s in range(n):
        out += padded[s:s + T] * taps[:, s]
    return out


def unit(a: torch.Tensor) -> torch.Tensor:
    return a / torch.sqrt((a * a).sum(-1, keepdim=True) + 1e-6)


def delta_walk(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor,
               state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``q, k [T, G, dim]``, ``v [T, H, vdim]``, ``beta, decay [T, H]``; ``state [H, dim, vdim]`` (zeros if None).
    Returns the read-outs ``[T, H, vdim]`` and the state after the last token."""
    T, G, dim = q.shape
    H, vdim = v.shape[1], v.shape[2]
    state = torch.zeros((H, dim, vdim), dtype=F) if state is None else state.clone()
    out = torch.zeros((T, H, vdim), dtype=F)
    for h in range(H):
        g = h // (H // G)
        S = state[h]
        for t in range(T):
            S = decay[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.T @ q[t, g]
        state[h] = S
    return out, state


def delta_rule(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    T = a.shape[0]
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = silu(short_convolution(a @ t64(tensors, f"{prefix}.q").T, t64(tensors, f"{prefix}.q.conv"))).view(T, G, dim)
    k = silu(short_convolution(a @ t64(tensors, f"{prefix}.k").T, t64(tensors, f"{prefix}.k.conv"))).view(T, G, dim)
    v = silu(short_convolution(a @ t64(tensors, f"{prefix}.v").T, t64(tensors, f"{prefix}.v.conv"))).view(T, H, vdim)
    q, k = unit(q) * dim ** -0.5, unit(k)
    beta = torch.sigmoid(a @ t64(tensors, f"{prefix}.b").T)                                     # [T, H]
    step = torch.nn.functional.softplus(a @ t64(tensors, f"{prefix}.a").T + t64(tensors, f"{prefix}.dt_bias"))
    decay = torch.exp(-torch.exp(t64(tensors, f"{prefix}.A_log")) * step)                       # [T, H]
    out, _ = delta_walk(q, k, v, beta, decay)
    gate = silu(a @ t64(tensors, f"{prefix}.g").T).view(T, H, vdim)
    out = rms(out, eps) * t64(tensors, f"{prefix}.norm") * gate
    return out.reshape(T, H * vdim) @ t64(tensors, f"{prefix}.o").T


def dense_feed_forward(a: torch.Tensor, tensors, prefix: str) -> torch.Tensor:
    hidden = silu(a @ t64(tensors, f"{prefix}.gate").T) * (a @ t64(tensors, f"{prefix}.up").T)
    return hidden @ t64(tensors, f"{prefix}.down").T


def forward(config: Mapping, tensors: Mapping[str, torch.Tensor], tokens: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Logits ``[T, vocab]`` and the stream after every layer ``[layers, T, width]``, float64."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = t64(tensors, "embed")[torch.tensor(tokens, dtype=torch.int64)]
    kept: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    streams = []
    for index, layer in enumerate(config["layers"]):
        name, mixer = f"l{index}", layer["mixer"]
        a = rms(x, eps) * t64(tensors, f"{name}.norm1")
        if layer["type"] == "latent_attention":
            y = latent_attention(a, tensors, f"{name}.mix", mixer, eps)
        elif layer["type"] == "attention":
            source = mixer.get("kv_from")
            if source is None:
                kept[index] = attention_keys_values(a, tensors, f"{name}.mix", mixer, eps)
                source = index
            y = attention(a, tensors, f"{name}.mix", mixer, eps, *kept[source])
        elif layer["type"] == "delta":
            y = delta_rule(a, tensors, f"{name}.mix", mixer, eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + m * (rms(y, eps) * t64(tensors, f"{name}.norm1b"))
        if layer.get("mlp") is not None:
            a = rms(x, eps) * t64(tensors, f"{name}.norm2")
            y = dense_feed_forward(a, tensors, f"{name}.mlp")
            x = x + m * (rms(y, eps) * t64(tensors, f"{name}.norm2b"))
        streams.append(x.clone())
    logits = (rms(x, eps) * t64(tensors, "final.norm")) @ t64(tensors, "head").T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(streams)


def read_config(folder: str) -> dict:
    import json
    import os
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        return json.load(handle)


def read_tensors(folder: str) -> Dict[str, torch.Tensor]:
    import os
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def generate_greedy(config: Mapping, tensors: Mapping[str, torch.Tensor], prompt: List[int], count: int) -> List[int]:
    """``count`` tokens after ``prompt``, each the first maximum of the last position's logits; every step runs the
    whole sequence again."""
    tokens = list(prompt)
    for _ in range(count):
        logits, _ = forward(config, tensors, tokens)
        tokens.append(int(torch.argmax(logits[-1])))
    return tokens[len(prompt):]
