"""Steps on the residual stream between layer calls."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import ResidualStream, Runtime, StreamStep, TensorSpec
from turboserve_amd.parts.registry import register_stream_step


@register_stream_step("pass_offset")
class PassOffset(StreamStep):
    """What a model whose layers run several passes adds to the stream when pass ``index`` begins:
    the embedding's output of the step (``add_origin``: every pass but the first, usually) and
    row ``index`` of a table ``[passes, H]`` stored under the part's prefix, summed in 32-bit.
    All passes' steps name the same table."""

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int, passes: int, index: int, add_origin: bool) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.passes = int(passes)
        self.index = int(index)
        if not 0 <= self.index < self.passes:
            raise ValueError(f"{prefix}: pass {self.index} of {self.passes}")
        self.needs_origin = bool(add_origin)
        self.offset: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name(""): TensorSpec((self.passes, self.hidden_size))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.offset = tensors[self.name("")][self.index].contiguous()

    def forward(self, stream: ResidualStream, ctx, origin: torch.Tensor | None) -> ResidualStream:
        if self.needs_origin and origin is None:
            raise ValueError(f"{self.prefix}: the step needs the embedding's output and was not given it")
        self.runtime.ops.stream_offset(stream.residual, origin if self.needs_origin else None, self.offset)
        return stream


@register_stream_step("origin_mix")
class OriginMix(StreamStep):
    """``x <- M [x ; x0]``: the stream and the embedding's output of the step side by side through one
    matrix ``M [H, 2 H]`` (the stream's half first), stored under the part's prefix; what a looped
    model does when a pass begins.  The product's operand is rounded to the run dtype; its result
    replaces the 32-bit stream."""

    needs_origin = True

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name(""): TensorSpec((self.hidden_size, 2 * self.hidden_size))}

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return tokens * self.hidden_size * (2 * itemsize + 4)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("")].contiguous()

    def forward(self, stream: ResidualStream, ctx, origin: torch.Tensor | None) -> ResidualStream:
        if origin is None:
            raise ValueError(f"{self.prefix}: the step needs the embedding's output and was not given it")
        ops, dtype = self.runtime.ops, self.runtime.dtype
        for waiting in (stream.pending, stream.also):
            if waiting is not None:
                ops.stream_fold(stream.residual, waiting, dtype)
        stream.pending = stream.also = None
        mixed = ops.linear(ops.stream_pair(stream.residual, origin, dtype), self.weight, for_residual=True)
        ops.stream_fold(stream.residual, mixed, dtype, assign=True)
        return stream
