"""Gated linear attention: a mixer whose memory is one matrix per head and request, not a cache of keys."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import CacheNeed, FixedState, FixedStateView, Mixer, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_mixer


@register_mixer("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Per head a state ``S [D, Dv]`` (32-bit, zero when the request starts) that every token updates
    and reads: ``S <- diag(a) S + k v^T``, ``o = S^T q`` with ``q = Wq x / sqrt(D)``, ``k = Wk x``, ``v =
    Wv x`` and a decay per key channel ``a = sigmoid(A2 (A1 x) + b)^(1 / tau)``.  Each head's ``o`` is
    divided by its root mean square and multiplied by one gain ``[Dv]``; the heads side by side are
    multiplied by ``silu(Wg x)`` and go through the output matrix.

    ``Wq, Wk, Wv, Wg, A1`` are held as one matrix (one product a step).  ``decay_rank`` is the width
    of ``A1 x``; ``None`` takes it from the checkpoint's tensors.  The state is a ``FixedState`` of
    the cache: the request's slot holds it between steps.  Steps of single tokens and short
    portions walk each request's tokens in one launch; long portions are cut into pieces that run
    side by side (``ops.linear_state``).  ``names``: tensor names under the part's prefix of ``q, k,
    v, gate, o, norm, a1, a2, a2_bias``."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        value_dim: int,
        tau: float,
        norm_eps: float,
        decay_rank: int | None = None,
        names: Mapping[str, str] | None = None,
    ) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.tau = float(tau)
        self.norm_eps = float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        if min(self.num_heads, self.head_dim, self.value_dim) < 1 or not self.tau > 0:
            raise ValueError(f"{prefix or 'gated linear attention'}: sizes and tau must be positive")
        if self.head_dim > 256 or self.num_heads > 65535:
            raise ValueError(f"{prefix or 'gated linear attention'}: the kernel takes up to 256 key channels a head")
        if self.decay_rank is not None and not 1 <= self.decay_rank <= 128:
            raise ValueError(f"{prefix or 'gated linear attention'}: a decay input of {self.decay_rank} is outside 1..128")
        self.names = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2",
                      "a2_bias": "a2.b", **(names or {})}
        self.key_size = self.num_heads * self.head_dim
        self.value_size = self.num_heads * self.value_dim
        self.fused: torch.Tensor | None = None      # [2 H D + 2 H Dv + R, hidden]
        self.a2: torch.Tensor | None = None         # [H D, R]
        self.a2_bias: torch.Tensor | None = None    # [H D]
        self.gain: torch.Tensor | None = None       # [Dv]
        self.o_weight: torch.Tensor | None = None   # [hidden, H Dv]

    def cache_need(self) -> CacheNeed:
        return FixedState((self.num_heads, self.head_dim, self.value_dim), torch.float32)

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        pieces = -(-tokens // 64) + 1
        state = pieces * self.num_heads * self.head_dim * (self.value_dim + 1) * 4
        return tokens * ((2 * self.key_size + 3 * self.value_size + 64) * itemsize + self.value_size * 4 + self.hidden_size * 4) + state

    def tensor_specs(self) -> dict[str, TensorSpec]:
        n = self.names
        rank = -1 if self.decay_rank is None else self.decay_rank
        return {
            self.name(n["q"]): TensorSpec((self.key_size, self.hidden_size)),
            self.name(n["k"]): TensorSpec((self.key_size, self.hidden_size)),
            self.name(n["v"]): TensorSpec((self.value_size, self.hidden_size)),
            self.name(n["gate"]): TensorSpec((self.value_size, self.hidden_size)),
            self.name(n["o"]): TensorSpec((self.hidden_size, self.value_size)),
            self.name(n["norm"]): TensorSpec((self.value_dim,), init="ones"),
            self.name(n["a1"]): TensorSpec((rank, self.hidden_size)),
            self.name(n["a2"]): TensorSpec((self.key_size, rank)),
            self.name(n["a2_bias"]): TensorSpec((self.key_size,), init="zeros"),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.names
        a1 = tensors[self.name(n["a1"])]
        self.a2 = tensors[self.name(n["a2"])].contiguous()
        if a1.shape[0] != self.a2.shape[1] or not 1 <= a1.shape[0] <= 128:
            raise ValueError(f"{self.prefix}: the decay's two matrices meet at {a1.shape[0]} and {self.a2.shape[1]} "
                             "elements; they must agree and be 1..128")
        self.low = int(a1.shape[0])
        self.fused = torch.cat([tensors[self.name(n[key])] for key in ("q", "k", "v", "gate")] + [a1], dim=0).contiguous()
        del a1
        self.a2_bias = tensors[self.name(n["a2_bias"])].contiguous()
        self.gain = tensors[self.name(n["norm"])].contiguous()
        self.o_weight = tensors[self.name(n["o"])].contiguous()

    def forward(self, x: torch.Tensor, ctx, cache: FixedStateView) -> torch.Tensor:
        ops, dtype = self.runtime.ops, self.runtime.dtype
        tokens = ctx.num_tokens
        proj = ops.linear(x, self.fused)
        o = torch.empty((tokens, self.value_size), dtype=torch.float32, device=x.device)
        common = dict(tokens=tokens, heads=self.num_heads, head_dim=self.head_dim, value_dim=self.value_dim, dtype=dtype, out=o)
        piece = ops.linear_state_piece
        if ctx.recorded or ctx.max_query_len <= piece:
            ops.linear_state(proj, self.a2, self.a2_bias, self.tau, cache.state, ctx.state_slots, ctx.query_start_loc,
                             first_seq=0, num_seqs=ctx.num_seqs, **common)
        else:
            # The requests that bring several tokens (they come first) in pieces side by side, the
            # single tokens behind them each whole.
            plan = ctx.derive(("linear_state_pieces", piece), lambda step: self._plan(step, piece, x.device))
            ops.linear_state(proj, self.a2, self.a2_bias, self.tau, cache.state, ctx.state_slots, ctx.query_start_loc,
                             first_seq=0, num_seqs=ctx.num_prefill_seqs, plan=plan, **common)
            if ctx.num_decode_seqs > 0:
                ops.linear_state(proj, self.a2, self.a2_bias, self.tau, cache.state, ctx.state_slots, ctx.query_start_loc,
                                 first_seq=ctx.num_prefill_seqs, num_seqs=ctx.num_decode_seqs, **common)
        y = ops.linear_state_finish(o, proj, self.gain, self.norm_eps, heads=self.num_heads, head_dim=self.head_dim,
                                    value_dim=self.value_dim, low=self.low, dtype=dtype)
        return ops.linear(y, self.o_weight, for_residual=True)

    def _plan(self, step, piece: int, device) -> tuple:
        pieces, carries = self.runtime.ops.linear_state_pieces(step.query_lens[: step.num_prefill_seqs], piece)
        both = self.runtime.ops.device_ints(pieces + carries)
        return both[: len(pieces)], both[len(pieces):], len(pieces), len(carries)
