"""Typed configuration of the Bimepel design: a decoder whose layers are listed one by one in ``config.json``, each
with the kind of its token mixer (``attention`` or ``lightning``), that mixer's sizes and constants, and its
feed-forward (dense with a clamped gate, routed experts, or none); a run of layers may be run several times in a row
with the same weights.

Keys of ``config.json``: ``architecture`` ("Bimepel"), ``vocab``, ``width``, ``norm`` (``{"eps"}``), ``layers`` (a
list of ``{"type", "mixer": {...}, "mlp": {...} or null}``), ``loop`` (``{"start", "stop", "times"}`` or absent).

Mixer ``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``rot`` (``{"base", "dims", "scaling":
{"factor", "original", "fast", "slow"} or absent}``, or absent for no rotation), ``mask`` (``{"size"}``: tokens see the
keys of their own block of so many positions; absent: every key before them).  Mixer ``lightning``: ``heads``,
``dim``, ``vdim``, ``decay`` (one per head).  ``mlp``: ``{"kind": "dense", "ff", "limit"}`` or ``{"kind": "moe",
"expert": {"ff"}, "router": {"experts", "top", "scale"}}``.

Every size and constant is read from there (or, by the weight loader, checked against the tensors' shapes).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, List, Optional

from .base import ConfigError, ModelConfig

MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale"),
    "lightning": ("heads", "dim", "vdim", "decay"),
}
MLP_KINDS = ("dense", "moe")


def _positive_int(where: str, d: Dict[str, Any], key: str) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {v!r}")
    return v


def _number(where: str, d: Dict[str, Any], key: str) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}: {key!r} must be a number, got {v!r}")
    return float(v)


@dataclasses.dataclass
class BimepelConfig(ModelConfig):
    model_type: ClassVar[str] = "bimepel"

    architecture: str = "Bimepel"
    vocab: int = 512
    width: int = 256
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    loop: Optional[Dict[str, Any]] = None
    norm: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    initializer_range: float = 0.05

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def run_order(self) -> List[int]:
        """The layers' indices in the order they run: those of the loop ``times`` times in a row."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, t = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    def validate(self) -> None:
        for key in ("vocab", "width"):
            _positive_int("config", dataclasses.asdict(self), key)
        if not isinstance(self.norm, dict) or "eps" not in self.norm:
            raise ConfigError("config: 'norm' must be an object with the key 'eps'")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config: 'layers' must list at least one layer")
        if self.loop:
            for key in ("start", "stop", "times"):
                v = self.loop.get(key) if isinstance(self.loop, dict) else None
                if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                    raise ConfigError(f"config.loop: {key!r} must be an integer from 0, got {v!r}")
            if not (self.loop["start"] <= self.loop["stop"] <= len(self.layers)) or self.loop["times"] < 1:
                raise ConfigError(f"config.loop: layers {self.loop['start']} .. {self.loop['stop']} - 1 of "
                                  f"{len(self.layers)}, {self.loop['times']} times, is no run of layers")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            kind = layer.get("type") if isinstance(layer, dict) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"{where}: type {kind!r} is not built; built: {', '.join(sorted(MIXER_KEYS))}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}: 'mixer' must hold the mixer's sizes")
            missing = [k for k in MIXER_KEYS[kind] if k not in mixer]
            if missing:
                raise ConfigError(f"{where} ({kind}): the mixer lacks {', '.join(missing)}")
            for k in MIXER_KEYS[kind]:
                if k not in ("scale", "decay"):
                    _positive_int(f"{where}.mixer", mixer, k)
            if kind == "attention":
                _number(f"{where}.mixer", mixer, "scale")
                if mixer["heads"] % mixer["kv_heads"]:
                    raise ConfigError(f"{where}: {mixer['heads']} heads are no multiple of {mixer['kv_heads']} kv heads")
                rot = mixer.get("rot")
                if rot is not None:
                    if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
                        raise ConfigError(f"{where}.mixer.rot must give 'base' and 'dims'")
                    if rot["dims"] % 2 or not (0 < rot["dims"] <= mixer["dim"]):
                        raise ConfigError(f"{where}.mixer.rot.dims ({rot['dims']}) must be even and at most dim ({mixer['dim']})")
                    sc = rot.get("scaling")
                    if sc is not None:
                        for k in ("factor", "original", "fast", "slow"):
                            if _number(f"{where}.mixer.rot.scaling", sc, k) <= 0:
                                raise ConfigError(f"{where}.mixer.rot.scaling: {k!r} must be positive")
                mask = mixer.get("mask")
                if mask is not None:
                    _positive_int(f"{where}.mixer.mask", mask, "size")
            else:
                decay = mixer["decay"]
                if not isinstance(decay, list) or len(decay) != mixer["heads"]:
                    raise ConfigError(f"{where}.mixer.decay must list one decay for each of the {mixer['heads']} heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"{where}.mlp: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not "
                                      f"built; built: {', '.join(MLP_KINDS)}, or null for no feed-forward")
                if mlp["kind"] == "dense":
                    _positive_int(f"{where}.mlp", mlp, "ff")
                    _number(f"{where}.mlp", mlp, "limit")
                else:
                    _positive_int(f"{where}.mlp.expert", mlp.get("expert"), "ff")
                    router = mlp.get("router")
                    for k in ("experts", "top"):
                        _positive_int(f"{where}.mlp.router", router, k)
                    _number(f"{where}.mlp.router", router, "scale")
                    if router["top"] > router["experts"]:
                        raise ConfigError(f"{where}.mlp.router: top {router['top']} of {router['experts']} experts")
