"""Plain, slow Kisadra forward pass: whole sequences, no cache, no paging, one function per part.

The oracle of the Kisadra tests.  It shares no code with ``turboserve_amd``: it reads a raw
``config.json`` mapping and a ``{tensor name: tensor}`` mapping and computes with ordinary torch
arithmetic on the CPU in one dtype (32-bit, or 64-bit where ``dtype`` says so).

The design in this file's notation.  ``W`` width, ``T`` tokens of ONE sequence at positions
``0..T-1``; matrices are stored ``[out, in]``.

* start: ``x_p = E[token_p]``, kept as ``x0``.
* layers ``l0 .. l(n-1)``; the slice ``[a, b)`` runs ``r`` times in a row with the same weights,
  then the rest.  Entering any pass (the first too): ``x = M [x ; x0]`` with ``M = loop.in``
  ``[W, 2W]``.
* a layer: ``h = n(x)``, ``x = x + mix(h) + ff(h)`` (both read the same ``h``; ``ff`` may be
  absent); ``n(x) = x / sqrt(mean(x^2) + eps) * g``.
* mixer ``attention``: ``q, k, v`` by three matrices; ``q`` as a whole (all heads at once) and
  ``k`` as a whole go through ``n`` with gains of their full size; head ``h`` of ``H`` reads
  key/value head ``h // (H / G)``; the score of key ``j`` for query ``i`` is ``scale q_i.k_j -
  m_h (i - j)``, ``m_h = 2^(-8 (h + 1) / H)``; visible are the ``j <= i`` with ``j // C == i //
  C`` (``C`` the chunk size); weights ``exp(s_j) / (1 + sum_j exp(s_j))``; output matrix.
* mixer ``latent_attention``: per head the query has ``D`` plain and ``R`` rotated elements (in
  that order); one matrix makes ``c'`` (``kv_rank`` elements) and ``r`` (``R`` elements) per
  token; ``c = n(c')``; head ``h``'s plain key is ``Uk_h c``, its value ``Uv_h c``, its rotated
  key is ``r`` for every head; rotation by position ``p`` turns the pair ``(i, i + d/2)`` of the
  first ``d`` rotated elements by the angle ``p base^(-2i/d)``; score ``scale (q_plain.k_plain +
  q_rot.k_rot)``, all ``j <= i`` visible, ordinary softmax, output matrix.
* mixer ``gla``: per head a state ``S [D, Dv]``, zero at the start; ``q = Wq h / sqrt(D)``, ``k =
  Wk h``, ``v = Wv h``; ``a = sigmoid(A2 (A1 h) + b)^(1/tau)`` per key channel; ``S <- diag(a) S +
  k v^T``, ``o = S^T q``; ``o`` of each head through ``n`` with one gain of size ``Dv``, heads side by
  side, times ``silu(Wg h)``, output matrix.
* dense feed-forward: ``Wd (gelu_tanh(Wg h) * (Wu h))``.
* routed feed-forward: ``s = softmax(R h)`` over ``E + I`` outputs; the ``top`` largest of ``s +
  correction`` are taken, each weighted with its ``s`` as it is; outputs ``>= E`` stand for ``h``
  itself, the others for expert ``e``: ``g = min(Wg h, L)``, ``u = clamp(Wu h, -L, L)``, ``Wd (g
  sigmoid(1.702 g) (u + 1))``.
* end: ``n`` with ``final.norm``, then the matrix ``head``.
"""

from __future__ import annotations

import math
from collections.abc import Mapping, Sequence

import torch

Tensors = Mapping[str, torch.Tensor]


def gain_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * gain`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def distance_slopes(heads: int) -> list[float]:
    return [2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)]


def _getter(tensors: Tensors, prefix: str, dtype):
    return lambda name: tensors[f"{prefix}.{name}"].to(dtype)


def chunked_sink_attention(h: torch.Tensor, tensors: Tensors, prefix: str, sizes: Mapping, eps: float) -> torch.Tensor:
    """The ``attention`` mixer over one whole sequence ``h [T, W]`` -> ``[T, W]``."""
    f = _getter(tensors, prefix, h.dtype)
    heads, kv_heads, dim, vdim = (int(sizes[key]) for key in ("heads", "kv_heads", "dim", "vdim"))
    scale = float(sizes["scale"])
    chunk = int(sizes["mask"]["size"]) if sizes.get("mask") else None
    count = h.shape[0]
    q = gain_norm(h @ f("q").T, f("q.norm"), eps).view(count, heads, dim)
    k = gain_norm(h @ f("k").T, f("k.norm"), eps).view(count, kv_heads, dim)
    v = (h @ f("v").T).view(count, kv_heads, vdim)
    slopes = distance_slopes(heads)
    out = torch.zeros((count, heads, vdim), dtype=h.dtype)
    for head in range(heads):
        kv = head // (heads // kv_heads)
        for i in range(count):
            first = 0 if chunk is None else (i // chunk) * chunk
            seen = torch.arange(first, i + 1)
            s = (k[seen, kv] @ q[i, head]) * scale - slopes[head] * (i - seen).to(h.dtype)
            e = torch.exp(s)
            out[i, head] = (e / (1.0 + e.sum())) @ v[seen, kv]
    return out.reshape(count, heads * vdim) @ f("o").T


def turn_pairs(x: torch.Tensor, positions: Sequence[int], dims: int, base: float) -> torch.Tensor:
    """``x [T, ..., n]``: of the first ``dims`` elements the pair ``(i, i + dims/2)`` is turned by
    ``p base^(-2i/dims)``; elements from ``dims`` on pass unchanged."""
    half = dims // 2
    out = x.clone()
    for row, p in enumerate(positions):
        for i in range(half):
            angle = p * base ** (-2.0 * i / dims)
            c, s = math.cos(angle), math.sin(angle)
            u, v = x[row, ..., i], x[row, ..., i + half]
            out[row, ..., i] = u * c - v * s
            out[row, ..., i + half] = v * c + u * s
    return out


def latent_attention(h: torch.Tensor, tensors: Tensors, prefix: str, sizes: Mapping, eps: float) -> torch.Tensor:
    """The ``latent_attention`` mixer over one whole sequence."""
    f = _getter(tensors, prefix, h.dtype)
    heads, dim, rot_dim, vdim, rank = (int(sizes[key]) for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    scale, base, dims = float(sizes["scale"]), float(sizes["rot"]["base"]), int(sizes["rot"]["dims"])
    count = h.shape[0]
    positions = list(range(count))
    q = (h @ f("q").T).view(count, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], turn_pairs(q[..., dim:], positions, dims, base)
    down = h @ f("dkv").T
    c = gain_norm(down[:, :rank], f("dkv.norm"), eps)
    k_rot = turn_pairs(down[:, rank:], positions, dims, base)
    k_plain = (c @ f("uk").T).view(count, heads, dim)
    v = (c @ f("uv").T).view(count, heads, vdim)
    out = torch.zeros((count, heads, vdim), dtype=h.dtype)
    for head in range(heads):
        for i in range(count):
            s = (k_plain[: i + 1, head] @ q_plain[i, head] + k_rot[: i + 1] @ q_rot[i, head]) * scale
            out[i, head] = torch.softmax(s, dim=0) @ v[: i + 1, head]
    return out.reshape(count, heads * vdim) @ f("o").T


def gated_linear_attention(h: torch.Tensor, tensors: Tensors, prefix: str, sizes: Mapping, eps: float) -> torch.Tensor:
    """The ``gla`` mixer over one whole sequence, the state walked token by token."""
    f = _getter(tensors, prefix, h.dtype)
    heads, dim, vdim, tau = int(sizes["heads"]), int(sizes["dim"]), int(sizes["vdim"]), float(sizes["tau"])
    count = h.shape[0]
    q = (h @ f("q").T).view(count, heads, dim) * dim ** -0.5
    k = (h @ f("k").T).view(count, heads, dim)
    v = (h @ f("v").T).view(count, heads, vdim)
    z = (h @ f("a1").T) @ f("a2").T + f("a2.b")
    decay = (torch.sigmoid(z) ** (1.0 / tau)).view(count, heads, dim)
    state = torch.zeros((heads, dim, vdim), dtype=h.dtype)
    out = torch.zeros((count, heads, vdim), dtype=h.dtype)
    for t in range(count):
        state = decay[t].unsqueeze(-1) * state + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hdv,hd->hv", state, q[t])
    out = gain_norm(out, f("norm"), eps).reshape(count, heads * vdim)
    gate = h @ f("g").T
    return (out * (gate * torch.sigmoid(gate))) @ f("o").T


MIXERS = {"attention": chunked_sink_attention, "latent_attention": latent_attention, "gla": gated_linear_attention}


def dense_feed_forward(h: torch.Tensor, tensors: Tensors, prefix: str) -> torch.Tensor:
    f = _getter(tensors, prefix, h.dtype)
    return (gelu_tanh(h @ f("gate").T) * (h @ f("up").T)) @ f("down").T


def routing(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int):
    """``(taken [T, top], weights [T, top])``: the ``top`` largest of ``softmax(R h) + correction``
    (the lower index where two are equal), weighted with the softmax alone."""
    s = torch.softmax(h @ router.T, dim=-1)
    choice = s + correction
    taken = torch.zeros((h.shape[0], top), dtype=torch.long)
    for t in range(h.shape[0]):
        order = sorted(range(choice.shape[1]), key=lambda e: (-float(choice[t, e]), e))
        taken[t] = torch.tensor(order[:top])
    return taken, torch.gather(s, 1, taken)


def clamped_expert(h: torch.Tensor, tensors: Tensors, prefix: str, limit: float) -> torch.Tensor:
    f = _getter(tensors, prefix, h.dtype)
    g = torch.clamp(h @ f("gate").T, max=limit)
    u = torch.clamp(h @ f("up").T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ f("down").T


def routed_feed_forward(h: torch.Tensor, tensors: Tensors, prefix: str, mlp: Mapping) -> torch.Tensor:
    f = _getter(tensors, prefix, h.dtype)
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    limit = float(mlp["expert"]["limit"])
    taken, weights = routing(h, f("router"), f("correction"), top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        row = h[t : t + 1]
        for e, w in zip(taken[t].tolist(), weights[t]):
            out[t] += w * (row[0] if e >= experts else clamped_expert(row, tensors, f"{prefix}.e{e}", limit)[0])
    return out


def feed_forward(h: torch.Tensor, tensors: Tensors, prefix: str, mlp: Mapping | None) -> torch.Tensor | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, tensors, prefix)
    return routed_feed_forward(h, tensors, prefix, mlp)


def run_order(config: Mapping) -> list[tuple[int, bool]]:
    """``(layer, whether a pass begins with this run)`` of every layer run."""
    count = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, count)]


def forward(config: Mapping, tensors: Tensors, tokens: Sequence[int], dtype=torch.float32, streams: list | None = None):
    """Logits ``[T, V]`` of one sequence; with ``streams`` a list, the residual stream after every
    layer run is appended to it."""
    eps = float(config["norm"]["eps"])
    x0 = tensors["embed"].to(dtype)[torch.tensor(list(tokens), dtype=torch.long)]
    x = x0
    for index, begins in run_order(config):
        layer = config["layers"][index]
        if begins:
            x = torch.cat([x, x0], dim=-1) @ tensors["loop.in"].to(dtype).T
        h = gain_norm(x, tensors[f"l{index}.norm1"].to(dtype), eps)
        update = MIXERS[layer["type"]](h, tensors, f"l{index}.mix", layer["mixer"], eps)
        extra = feed_forward(h, tensors, f"l{index}.mlp", layer.get("mlp"))
        x = x + (update if extra is None else update + extra)
        if streams is not None:
            streams.append(x.clone())
    return gain_norm(x, tensors["final.norm"].to(dtype), eps) @ tensors["head"].to(dtype).T
