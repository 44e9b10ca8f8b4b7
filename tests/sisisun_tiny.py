"""Small Sisisun configurations that differ in every size, constant and layer order, and helpers
that write their random model folders and compute the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from plain import sisisun_plain as plain


def attention(heads, kv_heads, dim, vdim, softcap, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "softcap": softcap,
            "scale": dim ** -0.5 if scale is None else scale}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, count, keep, scale, ff, shared_ff):
    return {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared_ff} if shared_ff else None,
            "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


def layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


#: P: grouped heads with values narrower and wider than the keys, a layer without a feed-forward,
#: routed layers with and without a shared expert, groups of two and plain top-1; the middle
#: layers run three passes.  Head sizes the matrix-core kernels take and ones they do not.
CONFIG_P = {
    "architecture": "Sisisun", "vocab": 211, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        layer(attention(4, 2, 32, 16, 6.0), dense(96, 1.5)),
        layer(attention(2, 2, 16, 40, 12.0, scale=0.3), moe(8, 2, 4, 2, 1.5, 48, 64)),
        layer(attention(4, 1, 16, 16, 30.0), None),
        layer(attention(3, 3, 24, 24, 8.0), moe(6, 1, 1, 1, 0.7, 40, 0)),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
PAGE_P = 16

#: Q: one pass only (the loop's offset is still added once), every expert a group of its own
#: (a group's mark is its one score), as many taken as kept, sizes that 16-byte accesses do not
#: divide, one head.
CONFIG_Q = {
    "architecture": "Sisisun", "vocab": 97, "width": 52, "norm": {"eps": 1e-6},
    "layers": [
        layer(attention(1, 1, 20, 12, 4.0), moe(5, 3, 5, 3, 2.5, 28, 20)),
        layer(attention(5, 1, 12, 12, 50.0, scale=0.5), dense(44, 0.75)),
    ],
    "loop": {"start": 0, "stop": 2, "times": 1},
}
PAGE_Q = 8

#: R: the matrix-core attention path in bfloat16 (head sizes 32 and 64, values as wide as the
#: keys), two passes over the first layer alone, pages of 32.
CONFIG_R = {
    "architecture": "Sisisun", "vocab": 160, "width": 96, "norm": {"eps": 1e-6},
    "layers": [
        layer(attention(6, 2, 32, 32, 15.0), moe(12, 3, 3, 2, 2.0, 32, 48)),
        layer(attention(2, 1, 64, 64, 25.0), dense(160, 3.0)),
    ],
    "loop": {"start": 0, "stop": 1, "times": 2},
}
PAGE_R = 32

TINY = {"P": (CONFIG_P, 11, PAGE_P), "Q": (CONFIG_Q, 12, PAGE_Q), "R": (CONFIG_R, 13, PAGE_R)}


def draw_tensors(config: dict, seed: int, dtype: torch.dtype, std: float) -> dict[str, torch.Tensor]:
    """Random tensors by the names and shapes the engine's own description of the model gives
    (the plain implementation reads them by name): matrices N(0, std), gains around their rest
    value, the loop's offsets and the router wide enough to matter."""
    from turboserve_amd.weights.random_init import describe_model

    _, model = describe_model(config)
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in model.tensor_specs().items():
        values = torch.randn(spec.shape, generator=generator)
        if name.endswith((".q.norm", ".k.norm")):
            values = 1.0 + 0.3 * values
        elif name.endswith(("norm1", "norm2", "final.norm")):
            values = 0.3 * values
        elif name == "loop.step":
            values = 0.5 * values
        elif name == "embed":
            values = 0.7 * values
        elif name.endswith((".router", ".sg")):
            values = 4.0 * std * values
        else:
            values = std * values
        tensors[name] = values.to(dtype).contiguous()
    return tensors


def make_model_dir(folder: Path, config: dict, seed: int, dtype: torch.dtype = torch.float32, std: float = 0.15,
                   tensors: dict[str, torch.Tensor] | None = None) -> Path:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors if tensors is not None else draw_tensors(config, seed, dtype, std), str(folder / "model.safetensors"))
    return folder


def read_model_dir(folder: Path) -> tuple[dict, dict[str, torch.Tensor]]:
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    tensors = {name: t.to(torch.float32) for name, t in load_file(str(Path(folder) / "model.safetensors")).items()}
    return config, tensors


def plain_logits(folder: Path, tokens: list[int]) -> torch.Tensor:
    config, tensors = read_model_dir(folder)
    return plain.forward(config, tensors, tokens)


def greedy(config: dict, tensors: dict[str, torch.Tensor], prompt: list[int], new: int) -> list[int]:
    tokens = list(prompt)
    for _ in range(new):
        tokens.append(int(plain.forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
