"""A plain, slow implementation of the Kalevik decoder on the CPU, one function per mechanism.

It shares no code with the engine: it takes the configuration as the dictionary that config.json holds and the
tensors by their file names, and computes every sequence whole, position by position where the mechanism is a
recurrence, in float64.

Notation. ``x`` is the residual stream ``[T, width]``; ``rms(a) = a / sqrt(mean(a^2) + eps)`` over the last axis.
The embedding's output is ``e = E[ids] * embedding.scale``. A layer is ``x += rms(M(rms(x) * w1)) * w1b`` and then the
same around the feed-forward with ``w2`` and ``w2b``. The layers ``loop.start .. loop.stop - 1`` run ``loop.times``
times in a row; before every pass but the first ``x += e``. The mixers:

* ``latent_attention``: ``q = Wq a`` head by head as ``[dim | rot_dim]``; ``Wdkv a`` gives the latent ``c``
  (``kv_rank`` numbers, RMS norm with a weight) and one key part ``r`` (``rot_dim`` numbers) for all heads; head
  ``h`` has keys ``[Wuk_h c | turn(r)]`` and values ``Wuv_h c``; causal softmax of ``scale * q . k``; ``Wo``.
  ``turn`` here pairs dimension ``2i`` with ``2i + 1`` and turns the pair by ``p * base^(-2i/n)``.
* ``parallel``: ``left_scale * left(a) + right_scale * right(a)``.
  left: grouped heads; ``q`` and ``k`` RMS-normed per head with a weight all heads share; the first ``rot.dims``
  dimensions of each head turned with dimension ``i`` paired with ``i + n/2`` by ``p * base^(-2i/n) / factor``;
  ``score = scale * q . k`` for ``j <= i`` in the same chunk (``i // size == j // size``); weights
  ``exp(s_j) / (1 + sum exp(s))``; head ``h`` times ``sigmoid(Wg a)_h``; ``Wo``.
  right: ``k *= dim^(-1/2)``; per head ``S <- decay_h S + k v^T``, ``o = S^T q``; ``o / sqrt(mean(o^2) + eps)`` per
  head; times ``silu(Wg a)``; ``Wo``.

The feed-forwards: ``dense`` is ``Wd (silu(Wg a) * (Wu a))``; ``moe`` sends every token through the ``top`` experts
with the largest softmax scores among the experts of the ``groups.keep`` best groups (a group's score is its largest),
each expert ``Wd gelu(Wu a)`` with the exact gelu, weighted by its score, plus a shared expert of the same form times
``sigmoid(wsg . a)``.
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


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def _angles(positions: torch.Tensor, base: float, n: int, divide: float) -> Tuple[torch.Tensor, torch.Tensor]:
    rates = torch.tensor([base ** (-2.0 * i / n) / divide for i in range(n // 2)], dtype=F)
    angle = positions.to(F)[:, None] * rates[None, :]
    return torch.cos(angle), torch.sin(angle)


def turn_neighbours(a: torch.Tensor, positions: torch.Tensor, base: float, n: int) -> torch.Tensor:
    """``a`` is ``[T, ..., D]``; of its first ``n`` dims, ``2i`` and ``2i + 1`` are turned together; the rest pass."""
    cos, sin = _angles(positions, base, n, 1.0)
    shape = [a.shape[0]] + [1] * (a.dim() - 2) + [n // 2]
    cos, sin = cos.view(shape), sin.view(shape)
    u, v = a[..., 0:n:2], a[..., 1:n:2]
    out = a.clone()
    out[..., 0:n:2] = u * cos - v * sin
    out[..., 1:n:2] = v * cos + u * sin
    return out


def turn_halves(a: torch.Tensor, positions: torch.Tensor, base: float, n: int, divide: float = 1.0) -> torch.Tensor:
    """Of the first ``n`` dims, ``i`` and ``i + n/2`` are turned together; every rate is divided by ``divide``."""
    cos, sin = _angles(positions, base, n, divide)
    half = n // 2
    shape = [a.shape[0]] + [1] * (a.dim() - 2) + [half]
    cos, sin = cos.view(shape), sin.view(shape)
    u, v = a[..., :half], a[..., half:n]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, a[..., n:]], dim=-1)


def latent_attention(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    T = a.shape[0]
    H, dim, rot, vdim, rank = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    positions = torch.arange(T)
    q = (a @ t64(tensors, f"{prefix}.q").T).view(T, H, dim + rot)
    down = a @ t64(tensors, f"{prefix}.dkv").T
    c = rms(down[:, :rank], eps) * t64(tensors, f"{prefix}.dkv.norm")
    r = turn_neighbours(down[:, rank:], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    q_rot = turn_neighbours(q[:, :, dim:], positions, mixer["rot"]["base"], mixer["rot"]["dims"])
    keys = (c @ t64(tensors, f"{prefix}.uk").T).view(T, H, dim)
    values = (c @ t64(tensors, f"{prefix}.uv").T).view(T, H, vdim)
    out = torch.zeros(T, H, vdim, dtype=F)
    for i in range(T):
        s = (torch.einsum("hd,jhd->hj", q[i, :, :dim], keys[: i + 1]) + q_rot[i] @ r[: i + 1].T) * mixer["scale"]
        p = torch.softmax(s, dim=-1)
        out[i] = torch.einsum("hj,jhd->hd", p, values[: i + 1])
    return out.reshape(T, H * vdim) @ t64(tensors, f"{prefix}.o").T


def attend_in_chunks(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, size: int) -> torch.Tensor:
    """``q`` ``[T, H, d]``, ``k`` ``[T, G, d]``, ``v`` ``[T, G, dv]`` as they enter the scores. Position ``i`` sees ``j <= i``
    of its own chunk of ``size`` positions; the weights are ``exp(s_j) / (1 + sum exp(s))``."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for i in range(T):
        first = (i // size) * size
        for h in range(H):
            g = h // (H // G)
            s = (k[first: i + 1, g] @ q[i, h]) * scale
            w = torch.exp(s)
            out[i, h] = ((w / (1.0 + w.sum()))[:, None] * v[first: i + 1, g]).sum(0)
    return out


def chunked_sink_attention(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    T = a.shape[0]
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    rot = mixer["rot"]
    divide = rot["scaling"]["factor"] if rot.get("scaling") else 1.0
    positions = torch.arange(T)
    q = (a @ t64(tensors, f"{prefix}.q").T).view(T, H, dim)
    k = (a @ t64(tensors, f"{prefix}.k").T).view(T, G, dim)
    v = (a @ t64(tensors, f"{prefix}.v").T).view(T, G, vdim)
    q = turn_halves(rms(q, eps) * t64(tensors, f"{prefix}.q.norm"), positions, rot["base"], rot["dims"], divide)
    k = turn_halves(rms(k, eps) * t64(tensors, f"{prefix}.k.norm"), positions, rot["base"], rot["dims"], divide)
    out = attend_in_chunks(q, k, v, mixer["scale"], mixer["mask"]["size"])
    out = out * torch.sigmoid(a @ t64(tensors, f"{prefix}.g").T)[:, :, None]       # one gate a head
    return out.reshape(T, H * vdim) @ t64(tensors, f"{prefix}.o").T


def retain(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay, state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``S <- decay_h S + k v^T``, ``o = S^T q`` token by token; ``q``, ``k`` ``[T, H, d]``, ``v`` ``[T, H, dv]``."""
    T, H, dim = q.shape
    decay = torch.as_tensor(decay, dtype=F)
    state = torch.zeros(H, dim, v.shape[2], dtype=F) if state is None else state.clone()
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        state = decay[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", state, q[t])
    return out


def retention(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    T = a.shape[0]
    H, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = (a @ t64(tensors, f"{prefix}.q").T).view(T, H, dim)
    k = (a @ t64(tensors, f"{prefix}.k").T).view(T, H, dim) * dim ** -0.5
    v = (a @ t64(tensors, f"{prefix}.v").T).view(T, H, vdim)
    out = rms(retain(q, k, v, mixer["decay"]), eps).reshape(T, H * vdim) * silu(a @ t64(tensors, f"{prefix}.g").T)
    return out @ t64(tensors, f"{prefix}.o").T


def parallel(a: torch.Tensor, tensors, prefix: str, mixer: Mapping, eps: float) -> torch.Tensor:
    left = chunked_sink_attention(a, tensors, f"{prefix}.left", mixer["left"], eps)
    right = retention(a, tensors, f"{prefix}.right", mixer["right"], eps)
    return mixer["left_scale"] * left + mixer["right_scale"] * right


def dense(a: torch.Tensor, tensors, prefix: str) -> torch.Tensor:
    inner = silu(a @ t64(tensors, f"{prefix}.gate").T) * (a @ t64(tensors, f"{prefix}.up").T)
    return inner @ t64(tensors, f"{prefix}.down").T


def small_expert(a: torch.Tensor, tensors, prefix: str) -> torch.Tensor:
    return gelu_erf(a @ t64(tensors, f"{prefix}.up").T) @ t64(tensors, f"{prefix}.down").T


def route(scores: torch.Tensor, top: int, groups: int, keep: int) -> List[int]:
    """The experts one token takes: the ``top`` largest scores among the experts of the ``keep`` groups whose largest
    score is largest (ties to the lower index)."""
    experts = scores.shape[0]
    size = experts // groups
    best = [max(scores[g * size:(g + 1) * size].tolist()) for g in range(groups)]
    kept = sorted(range(groups), key=lambda g: (-best[g], g))[:keep]
    allowed = [e for e in range(experts) if e // size in kept]
    return sorted(allowed, key=lambda e: (-float(scores[e]), e))[:top]


def moe(a: torch.Tensor, tensors, prefix: str, mlp: Mapping, margins: Optional[list] = None) -> torch.Tensor:
    router = mlp["router"]
    experts, top = router["experts"], router["top"]
    group = router.get("groups") or {"count": 1, "keep": 1}
    z = a.to(torch.float32).to(F) @ t64(tensors, f"{prefix}.router").T
    scores = torch.softmax(z, dim=-1)
    out = torch.zeros_like(a)
    for t in range(a.shape[0]):
        chosen = route(scores[t], top, group["count"], group["keep"])
        if margins is not None:
            margins.append(_margin(scores[t], chosen, group["count"], group["keep"]))
        for e in chosen:
            out[t] += scores[t, e] * small_expert(a[t:t + 1], tensors, f"{prefix}.e{e}")[0]
    if mlp.get("shared"):
        gate = torch.sigmoid(a @ t64(tensors, f"{prefix}.shared.sg").T)      # [T, 1]
        out = out + gate * small_expert(a, tensors, f"{prefix}.shared")
    return out


def _margin(scores: torch.Tensor, chosen: List[int], groups: int, keep: int) -> float:
    """How far the token is from another choice: the smallest gap between a score that decided something and the
    best one that lost (over experts within the kept groups, and over groups)."""
    experts = scores.shape[0]
    size = experts // groups
    best = sorted((max(scores[g * size:(g + 1) * size].tolist()) for g in range(groups)), reverse=True)
    gap = best[keep - 1] - best[keep] if keep < groups else float("inf")
    kept = sorted(range(groups), key=lambda g: (-max(scores[g * size:(g + 1) * size].tolist()), g))[:keep]
    losers = [float(scores[e]) for e in range(experts) if e // size in kept and e not in chosen]
    if losers:
        gap = min(gap, min(float(scores[e]) for e in chosen) - max(losers))
    return gap


def run_order(config: Mapping) -> List[Tuple[int, bool]]:
    """(layer, whether the embedding's output joins the stream right before it), run by run."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(count)]
    order = [(i, False) for i in range(loop["start"])]
    for n in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            order.append((i, n > 0 and i == loop["start"]))
    return order + [(i, False) for i in range(loop["stop"], count)]


def forward(config: Mapping, tensors: Mapping[str, torch.Tensor], ids, layers_out: Optional[list] = None,
            margins: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` (float64) of one sequence run whole."""
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(ids, dtype=torch.int64)
    e = t64(tensors, "embed")[ids] * (config.get("embedding") or {}).get("scale", 1.0)
    x = e.clone()
    for index, again in run_order(config):
        layer = config["layers"][index]
        prefix = f"l{index}"
        if again:
            x = x + e
        a = rms(x, eps) * t64(tensors, f"{prefix}.norm1")
        if layer["type"] == "latent_attention":
            mixed = latent_attention(a, tensors, f"{prefix}.mix", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            mixed = parallel(a, tensors, f"{prefix}.mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms(mixed, eps) * t64(tensors, f"{prefix}.norm1b")
        mlp = layer.get("mlp")
        if mlp is not None:
            a = rms(x, eps) * t64(tensors, f"{prefix}.norm2")
            if mlp["kind"] == "dense":
                fed = dense(a, tensors, f"{prefix}.mlp")
            elif mlp["kind"] == "moe":
                fed = moe(a, tensors, f"{prefix}.mlp", mlp, margins)
            else:
                raise ValueError(mlp["kind"])
            x = x + rms(fed, eps) * t64(tensors, f"{prefix}.norm2b")
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms(x, eps) * t64(tensors, "final.norm")
    return x @ t64(tensors, "head").T


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
        tokens.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
    return tokens[len(prompt):]
