"""Sisisun: from its configuration to a plan of parts.

A decoder of pre-norm blocks whose norms store their gain around zero.  The residual stream
starts as the token's row of ``embed`` plus a sinusoidal vector of its position (base 10000) and
is never rotated again: the attention layers are position-free.  Each layer is described on its
own: grouped-query attention with a norm per q and k head, a cap on the scores
(``c * tanh(s / c)``) and values of a width of their own; then a dense gated feed-forward with
clamped inputs (gate steepness 1.702, up + 1), a routed one (sigmoid router, group-limited
top-k, a gated shared expert), or none.  A slice of the layers runs several passes with the
same weights and a cache per pass; entering a pass adds the embedding's output again (not in the
first pass) and a row of ``loop.step``.  Tensors are named ``l<i>.norm1``, ``l<i>.mix.q``,
``l<i>.mlp.e<j>.gate`` and so on, without a ``weight`` suffix.
"""

from __future__ import annotations

from turboserve_amd.config.sisisun_config import DenseSizes, RoutedSizes, SisisunConfig
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec

#: Fixed by the design.
POSITION_BASE = 10000.0
DENSE_GATE_STEEPNESS = 1.702
DENSE_UP_SHIFT = 1.0

GLU_NAMES = ("gate", "up", "down")
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}


def sisisun_plan(config: SisisunConfig) -> ModelPlan:
    width = config.hidden_size
    norm = PartSpec("rmsnorm", {"size": width, "eps": config.norm_eps, "gain_offset": 1.0, "one_rounding": True,
                                "weight_name": ""})
    layers = []
    for index, layer in enumerate(config.layers):
        sizes = layer.mixer
        mixer = PartSpec("gqa_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
            "value_dim": sizes.vdim, "scale": sizes.scale, "softcap": sizes.softcap, "qkv_bias": False, "out_bias": False,
            "window": None, "position": PartSpec("none"), "head_norm": {"eps": config.norm_eps, "gain_offset": 0.0},
            "names": ATTENTION_NAMES,
        })
        feed_forward = None
        if isinstance(layer.mlp, DenseSizes):
            feed_forward = PartSpec("swiglu", {
                "hidden_size": width, "intermediate_size": layer.mlp.ff, "names": GLU_NAMES,
                "rule": (DENSE_GATE_STEEPNESS, layer.mlp.limit, DENSE_UP_SHIFT),
            })
        elif isinstance(layer.mlp, RoutedSizes):
            routed = layer.mlp
            shared = None
            if routed.shared_ff:
                shared = PartSpec("swiglu", {"hidden_size": width, "intermediate_size": routed.shared_ff, "names": GLU_NAMES})
            feed_forward = PartSpec("routed_experts", {
                "hidden_size": width, "expert_size": routed.ff, "experts": routed.experts, "top": routed.top,
                "groups": routed.groups, "keep": routed.keep, "route_scale": routed.scale, "shared": shared,
                "shared_name": "shared", "shared_gate_name": "sg" if shared is not None else None,
                "router_name": "router", "expert_names": ("e{index}", *GLU_NAMES),
            })
        block = PartSpec("prenorm", {
            "mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm,
            "ff_norm": norm if feed_forward is not None else None,
            "mixer_name": "mix", "ff_name": "mlp", "mixer_norm_name": "norm1", "ff_norm_name": "norm2",
        })
        layers.append(LayerSpec(prefix=f"l{index}", block=block))
    schedule = []
    for index, entering in config.run_order():
        enter = None
        if entering is not None:
            enter = PartSpec("pass_offset", {"hidden_size": width, "passes": config.loop_times, "index": entering,
                                             "add_origin": entering > 0})
        schedule.append(LayerCall(index, enter=enter, enter_prefix="loop.step"))
    # A loop over no layers enters no pass: its table of offsets may be in the file and is not read.
    unread = () if any(call.enter is not None for call in schedule) else ("loop.step",)
    return ModelPlan(
        ignorable=unread,
        vocab_size=config.vocab_size,
        hidden_size=width,
        layers=tuple(layers),
        schedule=tuple(schedule),
        embedding=PartSpec("token_table_sinusoid", {"vocab_size": config.vocab_size, "hidden_size": width,
                                                    "base": POSITION_BASE, "weight_name": ""}),
        head=PartSpec("norm_linear", {"vocab_size": config.vocab_size, "hidden_size": width, "norm": norm,
                                      "norm_prefix": "final.norm", "tied_to": None, "weight_name": ""}),
        embedding_prefix="embed",
        head_prefix="head",
    )
