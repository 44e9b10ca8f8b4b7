"""Typed view of a Kisadra ``config.json``.

The file names the design under ``architecture`` and describes every layer on its own::

    {"architecture": "Kisadra", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": s, "mask": {"size": C}},
                 "mlp": ...},
                {"type": "latent_attention",
                 "mixer": {"heads": H, "dim": D, "rot_dim": R, "vdim": Dv, "kv_rank": C, "scale": s,
                           "rot": {"base": b, "dims": d}},
                 "mlp": ...},
                {"type": "gla",
                 "mixer": {"heads": H, "dim": D, "vdim": Dv, "tau": t},
                 "mlp": null
                      | {"kind": "dense", "ff": I}
                      | {"kind": "moe", "expert": {"ff": I, "limit": L},
                         "router": {"experts": E, "identity": n, "top": k}}}, ...],
     "loop": {"start": a, "stop": b, "times": r}}

Every size and constant a model of the design can choose comes from here (the width of a ``gla``
layer's decay input comes from its tensors unless ``mixer.rank`` names it, which a folder of random
weights needs); what the design fixes lives where the plan is put together.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any

from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.sisisun_config import _count, _mapping, _real

ARCHITECTURE = "Kisadra"
MIXER_TYPES = ("attention", "latent_attention", "gla")


@dataclass(frozen=True)
class ChunkedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int | None

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "ChunkedAttentionSizes":
        chunk = None
        if data.get("mask") is not None:
            chunk = _count(f"{where}.mask", _mapping(where, data, "mask"), "size")
        sizes = cls(heads=_count(where, data, "heads"), kv_heads=_count(where, data, "kv_heads"), dim=_count(where, data, "dim"),
                    vdim=_count(where, data, "vdim"), scale=_real(where, data, "scale"), chunk=chunk)
        if sizes.heads % sizes.kv_heads != 0:
            raise UnsupportedModelError(f"config.json: {where}: {sizes.heads} heads are not a multiple of {sizes.kv_heads} kv_heads")
        return sizes

    def cached_elements(self) -> int:
        return self.kv_heads * (self.dim + self.vdim)


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "LatentAttentionSizes":
        rot = _mapping(where, data, "rot")
        sizes = cls(heads=_count(where, data, "heads"), dim=_count(where, data, "dim"), rot_dim=_count(where, data, "rot_dim"),
                    vdim=_count(where, data, "vdim"), kv_rank=_count(where, data, "kv_rank"), scale=_real(where, data, "scale"),
                    rot_base=_real(f"{where}.rot", rot, "base"), rot_dims=_count(f"{where}.rot", rot, "dims", least=2))
        if sizes.rot_dims > sizes.rot_dim or sizes.rot_dims % 2 != 0:
            raise UnsupportedModelError(f"config.json: {where}.rot.dims {sizes.rot_dims} must be even and at most rot_dim {sizes.rot_dim}")
        return sizes

    def cached_elements(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class LinearStateSizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int | None  # None: from the tensors

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "LinearStateSizes":
        return cls(heads=_count(where, data, "heads"), dim=_count(where, data, "dim"), vdim=_count(where, data, "vdim"),
                   tau=_real(where, data, "tau"), rank=None if data.get("rank") is None else _count(where, data, "rank"))

    def cached_elements(self) -> int:
        return 0


@dataclass(frozen=True)
class DenseSizes:
    ff: int


@dataclass(frozen=True)
class RoutedSizes:
    ff: int
    limit: float
    experts: int
    identity: int
    top: int

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "RoutedSizes":
        router = _mapping(where, data, "router")
        expert = _mapping(where, data, "expert")
        sizes = cls(ff=_count(f"{where}.expert", expert, "ff"), limit=_real(f"{where}.expert", expert, "limit"),
                    experts=_count(f"{where}.router", router, "experts"),
                    identity=0 if router.get("identity") is None else _count(f"{where}.router", router, "identity", least=0),
                    top=_count(f"{where}.router", router, "top"))
        if sizes.top > sizes.experts + sizes.identity:
            raise UnsupportedModelError(f"config.json: {where}.router: top {sizes.top} is more than the router's outputs")
        return sizes


@dataclass(frozen=True)
class KisadraLayer:
    type: str
    mixer: ChunkedAttentionSizes | LatentAttentionSizes | LinearStateSizes
    mlp: DenseSizes | RoutedSizes | None


@dataclass(frozen=True)
class KisadraConfig:
    """One checkpoint's numbers (frozen: model, cache sizing and runner share it)."""

    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple[KisadraLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eos_token_ids: tuple[int, ...] = ()
    name_or_path: str = ""

    def run_order(self) -> list[tuple[int, bool]]:
        """``(layer, whether a pass begins with this run)`` of every layer run: the layers
        ``loop_start .. loop_stop - 1`` run ``loop_times`` times in a row, the others once."""
        order = [(i, False) for i in range(self.loop_start)]
        for _ in range(self.loop_times):
            order += [(i, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return order + [(i, False) for i in range(self.loop_stop, len(self.layers))]

    def kv_bytes_per_token(self, dtype) -> int:
        """Bytes one token takes in the pages of all layer runs (a ``gla`` layer keeps none)."""
        return sum(self.layers[i].mixer.cached_elements() for i, _ in self.run_order()) * dtype.itemsize

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "KisadraConfig":
        if str(data.get("architecture")) != ARCHITECTURE:
            raise UnsupportedModelError(f"architecture {data.get('architecture')!r} is not {ARCHITECTURE}")
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise UnsupportedModelError("config.json: layers must be a non-empty list")
        readers = {"attention": ChunkedAttentionSizes, "latent_attention": LatentAttentionSizes, "gla": LinearStateSizes}
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping):
                raise UnsupportedModelError(f"config.json: {where} must be an object")
            kind = entry.get("type")
            if kind not in readers:
                raise UnsupportedModelError(f"config.json: {where}.type {kind!r} is not implemented; supported: {list(MIXER_TYPES)}")
            mixer = readers[kind].read(f"{where}.mixer", _mapping(where, entry, "mixer"))
            mlp = entry.get("mlp")
            if mlp is not None:
                mlp = _mapping(where, entry, "mlp")
                if mlp.get("kind") == "dense":
                    mlp = DenseSizes(ff=_count(f"{where}.mlp", mlp, "ff"))
                elif mlp.get("kind") == "moe":
                    mlp = RoutedSizes.read(f"{where}.mlp", mlp)
                else:
                    raise UnsupportedModelError(f"config.json: {where}.mlp.kind {mlp.get('kind')!r} is not implemented; supported: ['dense', 'moe']")
            layers.append(KisadraLayer(kind, mixer, mlp))
        start = stop = 0
        times = 1
        if data.get("loop") is not None:
            loop = _mapping("config", data, "loop")
            start, stop = _count("loop", loop, "start", least=0), _count("loop", loop, "stop", least=0)
            times = _count("loop", loop, "times")
            if not start <= stop <= len(layers):
                raise UnsupportedModelError(f"config.json: loop {start}..{stop} does not lie inside {len(layers)} layers")
        named = data.get("eos_token_id")
        eos = () if named is None else (int(named),) if isinstance(named, int) else tuple(int(t) for t in named)
        return cls(
            architecture=ARCHITECTURE, vocab_size=_count("config", data, "vocab"), hidden_size=_count("config", data, "width"),
            norm_eps=_real("norm", _mapping("config", data, "norm"), "eps"), layers=tuple(layers),
            loop_start=start, loop_stop=stop, loop_times=times, eos_token_ids=eos, name_or_path=name_or_path,
        )
