"""Typed configuration of the Pavodra design: a decoder whose layers are listed one by one in ``config.json``,
each with the kind of its token mixer (``latent_attention``, ``mingru`` or ``mamba2``), that mixer's sizes, and its
feed-forward (or none).

Keys of ``config.json``: ``architecture`` ("Pavodra"), ``vocab``, ``width``, ``layers`` (a list of ``{"type",
"mixer": {...}, "mlp": {"kind": "dense", "ff": n} or null}``), ``norm`` (``{"eps"}``), ``residual_mult``,
``logit_scale``.  Every size is read from there (or, by the weight loader, checked against the tensors' shapes);
nothing about a particular model of the design stands in code.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, List

from .base import ConfigError, ModelConfig

MIXER_KEYS = {
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
    "mingru": ("width",),
    "mamba2": ("heads", "vdim", "state", "groups", "conv", "norm_groups"),
}
MLP_KINDS = ("dense",)


def _positive_int(where: str, d: Dict[str, Any], key: str) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{where}: {key!r} must be a positive integer, got {v!r}")
    return v


@dataclasses.dataclass
class PavodraConfig(ModelConfig):
    model_type: ClassVar[str] = "pavodra"

    architecture: str = "Pavodra"
    vocab: int = 512
    width: int = 256
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    norm: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    initializer_range: float = 0.05

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eps(self) -> float:
        return float(self.norm["eps"])

    def validate(self) -> None:
        for key in ("vocab", "width"):
            _positive_int("config", dataclasses.asdict(self), key)
        if not isinstance(self.norm, dict) or "eps" not in self.norm:
            raise ConfigError("config: 'norm' must be an object with the key 'eps'")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("config: 'layers' must list at least one layer")
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
                if k not in ("scale", "rot"):
                    _positive_int(f"{where}.mixer", mixer, k)
            if kind == "latent_attention":
                rot = mixer["rot"]
                if not isinstance(rot, dict) or "base" not in rot or "dims" not in rot:
                    raise ConfigError(f"{where}.mixer.rot must give 'base' and 'dims'")
                if rot["dims"] % 2 or not (0 < rot["dims"] <= mixer["rot_dim"]):
                    raise ConfigError(f"{where}.mixer.rot.dims ({rot['dims']}) must be even and at most rot_dim ({mixer['rot_dim']})")
            if kind == "mamba2":
                if mixer["heads"] % mixer["groups"]:
                    raise ConfigError(f"{where}: {mixer['heads']} heads do not split into {mixer['groups']} groups")
                if (mixer["heads"] * mixer["vdim"]) % mixer["norm_groups"]:
                    raise ConfigError(f"{where}: {mixer['heads'] * mixer['vdim']} inner features do not split into "
                                      f"{mixer['norm_groups']} norm groups")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                    raise ConfigError(f"{where}.mlp: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not "
                                      f"built; built: {', '.join(MLP_KINDS)}, or null for no feed-forward")
                _positive_int(f"{where}.mlp", mlp, "ff")
