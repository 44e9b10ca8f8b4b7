"""Typed view of a Sisisun ``config.json``.

The file names the design under ``architecture`` and describes every layer on its own::

    {"architecture": "Sisisun", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": s, "softcap": c},
                 "mlp": null
                      | {"kind": "dense", "ff": I, "limit": L}
                      | {"kind": "moe", "expert": {"ff": I},
                         "router": {"experts": E, "top": k, "scale": r, "groups": {"count": n, "keep": m}},
                         "shared": {"ff": J} | null}}, ...],
     "loop": {"start": a, "stop": b, "times": r}}

Every size and constant a model of the design can choose comes from here; what the design
fixes (the steepness 1.702 of the dense feed-forward's gate, the base 10000 of the position
vectors) lives where the plan is put together.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any

from turboserve_amd.config.model_config import UnsupportedModelError

ARCHITECTURE = "Sisisun"


def _count(where: str, data: Mapping[str, Any], key: str, least: int = 1) -> int:
    raw = data.get(key)
    if isinstance(raw, bool) or not isinstance(raw, int) or raw < least:
        raise UnsupportedModelError(f"config.json: {where}.{key} must be an int of at least {least}, got {raw!r}")
    return raw


def _real(where: str, data: Mapping[str, Any], key: str, *, positive: bool = True) -> float:
    raw = data.get(key)
    if isinstance(raw, bool) or not isinstance(raw, (int, float)) or (positive and not raw > 0):
        raise UnsupportedModelError(f"config.json: {where}.{key} must be a {'positive ' if positive else ''}number, got {raw!r}")
    return float(raw)


def _mapping(where: str, data: Mapping[str, Any], key: str) -> Mapping[str, Any]:
    raw = data.get(key)
    if not isinstance(raw, Mapping):
        raise UnsupportedModelError(f"config.json: {where}.{key} must be an object, got {raw!r}")
    return raw


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "AttentionSizes":
        sizes = cls(
            heads=_count(where, data, "heads"), kv_heads=_count(where, data, "kv_heads"), dim=_count(where, data, "dim"),
            vdim=_count(where, data, "vdim"), scale=_real(where, data, "scale"), softcap=_real(where, data, "softcap"),
        )
        if sizes.heads % sizes.kv_heads != 0:
            raise UnsupportedModelError(f"config.json: {where}: {sizes.heads} heads are not a multiple of {sizes.kv_heads} kv_heads")
        return sizes


@dataclass(frozen=True)
class DenseSizes:
    ff: int
    limit: float


@dataclass(frozen=True)
class RoutedSizes:
    ff: int
    experts: int
    top: int
    groups: int
    keep: int
    scale: float
    shared_ff: int  # 0: no shared expert

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "RoutedSizes":
        router = _mapping(where, data, "router")
        groups = router.get("groups")
        count, keep = 1, 1
        if groups is not None:
            groups = _mapping(f"{where}.router", router, "groups")
            count, keep = _count(f"{where}.router.groups", groups, "count"), _count(f"{where}.router.groups", groups, "keep")
        shared = data.get("shared")
        sizes = cls(
            ff=_count(f"{where}.expert", _mapping(where, data, "expert"), "ff"),
            experts=_count(f"{where}.router", router, "experts"), top=_count(f"{where}.router", router, "top"),
            groups=count, keep=keep, scale=_real(f"{where}.router", router, "scale"),
            shared_ff=0 if shared is None else _count(f"{where}.shared", _mapping(where, data, "shared"), "ff"),
        )
        if sizes.experts % sizes.groups != 0 or sizes.keep > sizes.groups:
            raise UnsupportedModelError(
                f"config.json: {where}.router: {sizes.experts} experts in {sizes.groups} groups, {sizes.keep} kept")
        if sizes.top > (sizes.experts // sizes.groups) * sizes.keep:
            raise UnsupportedModelError(f"config.json: {where}.router: top {sizes.top} is more than the kept groups hold")
        return sizes


@dataclass(frozen=True)
class SisisunLayer:
    mixer: AttentionSizes
    mlp: DenseSizes | RoutedSizes | None


@dataclass(frozen=True)
class SisisunConfig:
    """One checkpoint's numbers (frozen: model, cache sizing and runner share it)."""

    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple[SisisunLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eos_token_ids: tuple[int, ...] = ()
    name_or_path: str = ""

    def run_order(self) -> list[tuple[int, int | None]]:
        """``(layer, pass)`` of every layer run: the layers ``loop_start .. loop_stop - 1`` run
        ``loop_times`` times in a row, the others once; ``pass`` is the number of the pass that
        begins with this run, ``None`` for every other run."""
        order: list[tuple[int, int | None]] = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            order += [(i, t if i == self.loop_start else None) for i in range(self.loop_start, self.loop_stop)]
        order += [(i, None) for i in range(self.loop_stop, len(self.layers))]
        return order

    def kv_bytes_per_token(self, dtype) -> int:
        """Bytes of keys and values one token takes over all layer runs."""
        per_layer = [l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) for l in self.layers]
        return sum(per_layer[i] for i, _ in self.run_order()) * dtype.itemsize

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "SisisunConfig":
        if str(data.get("architecture")) != ARCHITECTURE:
            raise UnsupportedModelError(f"architecture {data.get('architecture')!r} is not {ARCHITECTURE}")
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise UnsupportedModelError("config.json: layers must be a non-empty list")
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping):
                raise UnsupportedModelError(f"config.json: {where} must be an object")
            if entry.get("type") != "attention":
                raise UnsupportedModelError(f"config.json: {where}.type {entry.get('type')!r} is not implemented; supported: ['attention']")
            mixer = AttentionSizes.read(f"{where}.mixer", _mapping(where, entry, "mixer"))
            mlp = entry.get("mlp")
            if mlp is not None:
                mlp = _mapping(where, entry, "mlp")
                kind = mlp.get("kind")
                if kind == "dense":
                    mlp = DenseSizes(ff=_count(f"{where}.mlp", mlp, "ff"), limit=_real(f"{where}.mlp", mlp, "limit"))
                elif kind == "moe":
                    mlp = RoutedSizes.read(f"{where}.mlp", mlp)
                else:
                    raise UnsupportedModelError(f"config.json: {where}.mlp.kind {kind!r} is not implemented; supported: ['dense', 'moe']")
            layers.append(SisisunLayer(mixer, mlp))
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
