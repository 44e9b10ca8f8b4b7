"""Kisadra: from its configuration to a plan of parts.

A decoder of parallel blocks: one norm (plain gain) whose output both the mixer and the
feed-forward read, their outputs added to the stream together.  The stream starts as the token's
row of ``embed``.  A slice of the layers runs several passes with the same weights and a cache or
state per pass; entering any pass, the first too, the stream and the embedding's output go side by
side through the matrix ``loop.in``.  Each layer is described on its own, with one of three mixers:

* ``attention``: grouped-query attention without rotation; queries and keys are normalised over
  their whole projection; a score loses ``2^(-8 (h + 1) / H)`` per position of distance; a token
  sees its own chunk of positions only; the softmax's denominator counts one more key of score 0.
* ``latent_attention``: keys and values of all heads from one cached latent per token and a
  rotated key part that the heads share (rotation in halves).
* ``gla``: a decaying state matrix per head (gated linear attention).

Feed-forward: a dense gated one with the tanh form of GELU on the gate, a routed one (softmax
router, a correction added only where experts are chosen, weights not normalised, experts with
clamped inputs, steepness 1.702 and ``up + 1``, identity experts at the end of the router's
outputs), or none.  Tensors are named ``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mlp.e<j>.gate`` and so
on, without a ``weight`` suffix.
"""

from __future__ import annotations

from turboserve_amd.config.kisadra_config import (
    ChunkedAttentionSizes,
    DenseSizes,
    KisadraConfig,
    LatentAttentionSizes,
    LinearStateSizes,
    RoutedSizes,
)
from turboserve_amd.kernels.ops import GELU_TANH_RULE
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec

#: Fixed by the design.
SLOPE_EXPONENT = 8.0
ATTENTION_SINKS = 1.0
EXPERT_GATE_STEEPNESS = 1.702
EXPERT_UP_SHIFT = 1.0

GLU_NAMES = ("gate", "up", "down")
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}


def _mixer(width: int, eps: float, sizes) -> PartSpec:
    if isinstance(sizes, ChunkedAttentionSizes):
        return PartSpec("gqa_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
            "value_dim": sizes.vdim, "scale": sizes.scale, "qkv_bias": False, "out_bias": False, "window": None,
            "position": PartSpec("distance_slopes", {"exponent": SLOPE_EXPONENT}),
            "span_norm": {"eps": eps, "gain_offset": 0.0}, "chunk": sizes.chunk, "sinks": ATTENTION_SINKS,
            "names": ATTENTION_NAMES,
        })
    if isinstance(sizes, LatentAttentionSizes):
        return PartSpec("latent_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "head_dim": sizes.dim, "rot_dim": sizes.rot_dim,
            "value_dim": sizes.vdim, "rank": sizes.kv_rank, "scale": sizes.scale, "norm_eps": eps,
            "rotation": PartSpec("rope", {"head_dim": sizes.rot_dims, "theta": sizes.rot_base, "max_positions": 4096}),
        })
    if isinstance(sizes, LinearStateSizes):
        return PartSpec("gated_linear_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "head_dim": sizes.dim, "value_dim": sizes.vdim,
            "tau": sizes.tau, "norm_eps": eps, "decay_rank": sizes.rank,
        })
    raise TypeError(f"no mixer for {sizes!r}")


def _feed_forward(width: int, mlp) -> PartSpec | None:
    if mlp is None:
        return None
    if isinstance(mlp, DenseSizes):
        return PartSpec("swiglu", {"hidden_size": width, "intermediate_size": mlp.ff, "names": GLU_NAMES,
                                   "rule": GELU_TANH_RULE})
    if isinstance(mlp, RoutedSizes):
        return PartSpec("routed_experts", {
            "hidden_size": width, "expert_size": mlp.ff, "experts": mlp.experts, "top": mlp.top, "identity": mlp.identity,
            "router_scores": "softmax", "correction_name": "correction", "normalise": False,
            "rule": (EXPERT_GATE_STEEPNESS, mlp.limit, EXPERT_UP_SHIFT), "router_name": "router",
            "expert_names": ("e{index}", *GLU_NAMES),
        })
    raise TypeError(f"no feed-forward for {mlp!r}")


def kisadra_plan(config: KisadraConfig) -> ModelPlan:
    width = config.hidden_size
    norm = PartSpec("rmsnorm", {"size": width, "eps": config.norm_eps, "one_rounding": True, "weight_name": ""})
    layers = []
    for index, layer in enumerate(config.layers):
        block = PartSpec("parallel", {
            "mixer": _mixer(width, config.norm_eps, layer.mixer), "feed_forward": _feed_forward(width, layer.mlp),
            "norm": norm, "mixer_name": "mix", "ff_name": "mlp", "norm_name": "norm1",
        })
        layers.append(LayerSpec(prefix=f"l{index}", block=block))
    schedule = []
    for index, begins in config.run_order():
        enter = PartSpec("origin_mix", {"hidden_size": width}) if begins else None
        schedule.append(LayerCall(index, enter=enter, enter_prefix="loop.in"))
    # A loop over no layers enters no pass: its matrix may be in the file and is not read.
    unread = () if any(call.enter is not None for call in schedule) else ("loop.in",)
    return ModelPlan(
        ignorable=unread,
        vocab_size=config.vocab_size,
        hidden_size=width,
        layers=tuple(layers),
        schedule=tuple(schedule),
        embedding=PartSpec("token_table", {"vocab_size": config.vocab_size, "hidden_size": width, "weight_name": ""}),
        head=PartSpec("norm_linear", {"vocab_size": config.vocab_size, "hidden_size": width, "norm": norm,
                                      "norm_prefix": "final.norm", "tied_to": None, "weight_name": ""}),
        embedding_prefix="embed",
        head_prefix="head",
    )
