"""Small Kisadra configurations that differ in every size, constant and layer order, and helpers
that write their random model folders and compute the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from plain import kisadra_plain as plain


def attention(heads, kv_heads, dim, vdim, chunk, scale=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": dim ** -0.5 if scale is None else scale, "mask": {"size": chunk}}}


def latent(heads, dim, rot_dim, vdim, rank, turned=None, base=10000.0, scale=None):
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
        "scale": (dim + rot_dim) ** -0.5 if scale is None else scale,
        "rot": {"base": base, "dims": rot_dim if turned is None else turned}}}


def gla(heads, dim, vdim, tau, rank):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "identity": identity, "top": top}}


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


#: A: the three mixers in the order state, chunks, latent; the last two run three passes; values
#: narrower and wider than keys; a layer without a feed-forward; one identity expert.
CONFIG_A = {
    "architecture": "Kisadra", "vocab": 211, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        layer(gla(2, 16, 24, 4.0, 8), dense(96)),
        layer(attention(4, 2, 16, 8, 20, scale=0.3), moe(6, 1, 2, 40, 1.5)),
        layer(latent(3, 16, 8, 12, 24, base=1000.0), None),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
PAGE_A = 16

#: B: sizes that 16-byte accesses do not divide; one head; as many key heads as query heads; a
#: chunk shorter than a page; fewer turned elements than rotated ones; every expert taken; no
#: identity expert in one layer and more identity experts than real ones in another, with one
#: taken; a state whose values span two column tiles; one pass (the entering matrix still acts).
CONFIG_B = {
    "architecture": "Kisadra", "vocab": 97, "width": 52, "norm": {"eps": 1e-6},
    "layers": [
        layer(latent(1, 12, 12, 20, 10, turned=4, base=50.0, scale=0.4), moe(3, 0, 3, 28, 0.75)),
        layer(attention(5, 5, 12, 12, 7, scale=0.5), dense(44)),
        layer(gla(1, 20, 70, 1.0, 3), moe(2, 3, 1, 20, 3.0)),
    ],
    "loop": {"start": 0, "stop": 3, "times": 1},
}
PAGE_B = 8

#: C: larger heads, a chunk of two pages, a long state memory, two passes over the first layer
#: alone, pages of 32.
CONFIG_C = {
    "architecture": "Kisadra", "vocab": 160, "width": 96, "norm": {"eps": 1e-6},
    "layers": [
        layer(attention(6, 2, 32, 32, 64), moe(12, 4, 4, 32, 2.5)),
        layer(gla(4, 64, 32, 16.0, 16), dense(160)),
        layer(latent(4, 32, 32, 16, 64), moe(5, 1, 2, 24, 1.0)),
    ],
    "loop": {"start": 0, "stop": 1, "times": 2},
}
PAGE_C = 32

TINY = {"A": (CONFIG_A, 11, PAGE_A), "B": (CONFIG_B, 12, PAGE_B), "C": (CONFIG_C, 13, PAGE_C)}


def draw_tensors(config: dict, seed: int, dtype: torch.dtype, std: float) -> dict[str, torch.Tensor]:
    """Random tensors by the names and shapes the engine's own description of the model gives
    (the plain implementation reads them by name): matrices N(0, std), gains around one, routers,
    corrections and decay biases wide enough to matter."""
    from turboserve_amd.weights.random_init import describe_model

    _, model = describe_model(config)
    generator = torch.Generator().manual_seed(seed)
    width = config["width"]
    tensors = {}
    for name, spec in model.tensor_specs().items():
        values = torch.randn(spec.shape, generator=generator)
        if name.endswith(("norm", "norm1")):
            values = 1.0 + 0.3 * values
        elif name == "embed":
            values = 0.7 * values
        elif name == "loop.in":
            values = values / (2 * width) ** 0.5
        elif name.endswith(".router"):
            values = 4.0 * std * values
        elif name.endswith(".correction"):
            values = 0.05 * values
        elif name.endswith(".a2.b"):
            values = 1.5 + values
        elif name.endswith((".a1", ".a2")):
            values = 3.0 * std * values
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


def without_ranks(config: dict) -> dict:
    """The configuration as a checkpoint's own file has it: the decay input's width is not named."""
    out = json.loads(json.dumps(config))
    for entry in out["layers"]:
        entry["mixer"].pop("rank", None)
    return out


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
