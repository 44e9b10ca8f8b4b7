"""Plain, slow Sisisun forward pass: whole sequences, no cache, no paging, one function per part.

The oracle of the Sisisun tests.  It shares no code with ``turboserve_amd``: it reads a raw
``config.json`` mapping and a ``{tensor name: tensor}`` mapping and computes with ordinary torch
arithmetic on the CPU, everything in 32-bit (or 64-bit where ``dtype`` says so).

The design in this file's notation.  ``W`` width, ``T`` tokens of ONE sequence at positions
``0..T-1``.

* start: ``x_p = E[token_p] + s_p`` with ``s_p[2i] = sin(p w_i)``, ``s_p[2i+1] = cos(p w_i)``,
  ``w_i = 10000^(-2i/W)``; ``x`` here is kept as ``x0``.
* layers ``l0 .. l(n-1)``; the slice ``[a, b)`` runs ``r`` times in a row with the same weights,
  then the rest.  Entering pass ``t``: ``x += x0`` (only for ``t > 0``), then ``x += S[t]``
  (``S`` is ``loop.step``, ``[r, W]``).
* a layer: ``x += mix(norm1(x))``; ``x += ff(norm2(x))`` where it has a feed-forward.
  ``norm(x) = x / sqrt(mean(x^2) + eps) * (1 + g)``.
* attention mixer: ``q, k, v`` by three matrices; per head ``q`` and ``k`` are divided by their
  root mean square (``eps`` inside the root) and multiplied by a gain vector of the head size,
  the same for all heads; scores ``c * tanh(scale * q.k / c)`` over keys ``j <= i``, softmax,
  weighted sum of ``v`` (its own width), output matrix.  Query head ``h`` reads key/value head
  ``h // (H / G)``.
* dense feed-forward: ``g = min(Wg x, L)``, ``u = clamp(Wu x, -L, L)``,
  ``Wd (g * sigmoid(1.702 g) * (u + 1))``.
* routed feed-forward: ``z = R x``, ``s = sigmoid(z)``; the experts are cut into equal groups of
  neighbours, a group's mark is the sum of its two largest ``s``, the best ``keep`` groups stay
  eligible; the ``top`` eligible experts with the largest ``s`` are taken with weights
  ``s / (sum of the taken s + 1e-20) * router scale``; an expert is ``Wd (silu(Wg x) * (Wu x))``;
  a shared expert of the same form is added for every token, multiplied by ``sigmoid(sg . x)``.
* end: ``norm`` with ``final.norm``, then the matrix ``head``.
"""

from __future__ import annotations

import math
from collections.abc import Mapping, Sequence

import torch

Tensors = Mapping[str, torch.Tensor]


def unit_gain_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * (1 + gain)`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * (1.0 + gain)


def plain_gain_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * gain`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


def sinusoid_rows(positions: Sequence[int], width: int, dtype=torch.float32) -> torch.Tensor:
    """``[len(positions), width]``: entry ``2i`` is ``sin(p * 10000^(-2i/width))``, ``2i+1`` the cosine."""
    out = torch.zeros((len(positions), width), dtype=dtype)
    for row, p in enumerate(positions):
        for i in range((width + 1) // 2):
            angle = p * 10000.0 ** (-2.0 * i / width)
            out[row, 2 * i] = math.sin(angle)
            if 2 * i + 1 < width:
                out[row, 2 * i + 1] = math.cos(angle)
    return out


def start(tokens: Sequence[int], tensors: Tensors, width: int, first_position: int = 0) -> torch.Tensor:
    table = tensors["embed"].to(torch.float32)
    rows = table[torch.tensor(list(tokens), dtype=torch.long)]
    return rows + sinusoid_rows(range(first_position, first_position + len(tokens)), width)


def capped_attention(h: torch.Tensor, tensors: Tensors, prefix: str, sizes: Mapping, eps: float) -> torch.Tensor:
    """The attention mixer over one whole sequence ``h [T, W]`` -> ``[T, W]``."""
    heads, kv_heads = int(sizes["heads"]), int(sizes["kv_heads"])
    dim, vdim = int(sizes["dim"]), int(sizes["vdim"])
    scale, cap = float(sizes["scale"]), float(sizes["softcap"])
    f = lambda name: tensors[f"{prefix}.{name}"].to(torch.float32)
    count = h.shape[0]
    q = (h @ f("q").T).view(count, heads, dim)
    k = (h @ f("k").T).view(count, kv_heads, dim)
    v = (h @ f("v").T).view(count, kv_heads, vdim)
    q = plain_gain_norm(q, f("q.norm"), eps)
    k = plain_gain_norm(k, f("k.norm"), eps)
    per_kv = heads // kv_heads
    out = torch.zeros((count, heads, vdim), dtype=torch.float32)
    hidden = torch.ones((count, count), dtype=torch.bool).triu(1)  # key j > query i
    for head in range(heads):
        kv = head // per_kv
        scores = (q[:, head] @ k[:, kv].T) * scale
        scores = cap * torch.tanh(scores / cap)
        weights = torch.softmax(scores.masked_fill(hidden, float("-inf")), dim=1)
        out[:, head] = weights @ v[:, kv]
    return out.reshape(count, heads * vdim) @ f("o").T


def clamped_glu(h: torch.Tensor, tensors: Tensors, prefix: str, limit: float) -> torch.Tensor:
    f = lambda name: tensors[f"{prefix}.{name}"].to(torch.float32)
    g = torch.clamp(h @ f("gate").T, max=limit)
    u = torch.clamp(h @ f("up").T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ f("down").T


def silu_glu(h: torch.Tensor, tensors: Tensors, prefix: str) -> torch.Tensor:
    f = lambda name: tensors[f"{prefix}.{name}"].to(torch.float32)
    g = h @ f("gate").T
    return (g * torch.sigmoid(g) * (h @ f("up").T)) @ f("down").T


def route(scores: Sequence[float], top: int, groups: int, keep: int) -> list[int]:
    """The experts one token takes, given its scores: the ``top`` largest among the experts of
    the ``keep`` groups with the largest marks (a mark: the sum of a group's two largest)."""
    count = len(scores)
    size = count // groups
    marks = []
    for g in range(groups):
        members = sorted(scores[g * size:(g + 1) * size], reverse=True)
        marks.append(sum(members[:2]))
    kept = sorted(range(groups), key=lambda g: (-marks[g], g))[:keep]
    eligible = [e for e in range(count) if e // size in kept]
    return sorted(eligible, key=lambda e: (-scores[e], e))[:top]


def routed_experts(h: torch.Tensor, tensors: Tensors, prefix: str, mlp: Mapping) -> torch.Tensor:
    router = mlp["router"]
    count, top = int(router["experts"]), int(router["top"])
    groups, keep = int(router["groups"]["count"]), int(router["groups"]["keep"])
    z = h @ tensors[f"{prefix}.router"].to(torch.float32).T
    s = torch.sigmoid(z)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        taken = route(s[t].tolist(), top, groups, keep)
        total = sum(float(s[t, e]) for e in taken) + 1e-20
        for e in taken:
            weight = float(s[t, e]) / total * float(router["scale"])
            out[t] += weight * silu_glu(h[t:t + 1], tensors, f"{prefix}.e{e}")[0]
    if mlp.get("shared"):
        gate = torch.sigmoid(h @ tensors[f"{prefix}.shared.sg"].to(torch.float32).T)  # [T, 1]
        out = out + gate * silu_glu(h, tensors, f"{prefix}.shared")
    return out


def layer(x: torch.Tensor, tensors: Tensors, index: int, spec: Mapping, eps: float) -> torch.Tensor:
    prefix = f"l{index}"
    f = lambda name: tensors[f"{prefix}.{name}"].to(torch.float32)
    if spec["type"] != "attention":
        raise ValueError(f"unknown mixer {spec['type']!r}")
    x = x + capped_attention(unit_gain_norm(x, f("norm1"), eps), tensors, f"{prefix}.mix", spec["mixer"], eps)
    mlp = spec.get("mlp")
    if mlp is None:
        return x
    h = unit_gain_norm(x, f("norm2"), eps)
    if mlp["kind"] == "dense":
        return x + clamped_glu(h, tensors, f"{prefix}.mlp", float(mlp["limit"]))
    if mlp["kind"] == "moe":
        return x + routed_experts(h, tensors, f"{prefix}.mlp", mlp)
    raise ValueError(f"unknown feed-forward {mlp['kind']!r}")


def run_order(cfg: Mapping) -> list[tuple[int, int | None]]:
    """``(layer, pass number or None)`` of every layer run; the pass number stands at the first
    layer of each pass through the repeated slice."""
    count = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, r = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order: list[tuple[int, int | None]] = [(i, None) for i in range(a)]
    for t in range(r):
        order += [(i, t if i == a else None) for i in range(a, b)]
    order += [(i, None) for i in range(b, count)]
    return order


def forward(cfg: Mapping, tensors: Tensors, tokens: Sequence[int], *, trace: list | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence; ``trace`` collects ``x`` after every layer run."""
    width, eps = int(cfg["width"]), float(cfg["norm"]["eps"])
    x0 = start(tokens, tensors, width)
    x = x0.clone()
    for index, entering in run_order(cfg):
        if entering is not None:
            if entering > 0:
                x = x + x0
            x = x + tensors["loop.step"].to(torch.float32)[entering]
        x = layer(x, tensors, index, cfg["layers"][index], eps)
        if trace is not None:
            trace.append(x.clone())
    return unit_gain_norm(x, tensors["final.norm"].to(torch.float32), eps) @ tensors["head"].to(torch.float32).T
