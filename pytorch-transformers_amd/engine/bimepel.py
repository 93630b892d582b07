"""The Bimepel design as a list of parts: the builder registered for ``model_type: bimepel`` (a ``config.json`` that
says ``"architecture": "Bimepel"``).

A layer is a ``ShiftedParallelBlock``: a 32-bit stream, two RMS norms of the same x, the mixer reading its norm mixed
with the token before's, ``x <- x + (mixer + feed-forward)``.  The mixer is attention with normed heads, a partly
rotated head, a mask in blocks and an output gate, or linear attention with a decay per head, by the layer's
``type``; the feed-forward is dense with a clamped gate, routed experts, or absent.  A run of layers may run several
times in a row with the same weights: the run order names the block again, with storage of its own for every pass.
The head is the embedding table on the final norm's output.

Tensor names: ``embed``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.shift``,
``l<i>.mix.<name>``, ``l<i>.mlp.<name>``.

Storage per sequence: attention passes with equal kv heads, page head size and mask share a page pool (of a masked
layer, a sequence holds the pages of its current block only); linear-attention
passes with equal state sizes share a state table; the token-shift rows of all passes are one state table.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..config.bimepel import BimepelConfig
from ..config.registry import register
from ..parts import (DecayLinearAttentionMixer, Embedding, GatedAttentionMixer, GatedFeedForward, NoPositions, OutputHead,
                     RMSNorm, RotaryPositions, RoutedFeedForward, ShiftedParallelBlock)
from ..parts.positions import yarn_ramp_frequencies
from .spec import CACHE_CHUNK, CACHE_FULL, CACHE_STATE, CacheGroupSpec, LayerCall, ModelSpec

GATE_ALPHA = 1.702  # the dense feed-forward's gate is g * sigmoid(1.702 g)


def _positions(m: dict):
    rot = m.get("rot")
    if not rot:
        return NoPositions()
    dims, base = int(rot["dims"]), float(rot["base"])
    sc = rot.get("scaling")
    if not sc:
        return RotaryPositions(m["dim"], base, rotary_dim=dims)
    table, mult = yarn_ramp_frequencies(dims, base, float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                        float(sc["slow"]))
    return RotaryPositions(m["dim"], base, attention_scaling=mult, inv_freq=table, rotary_dim=dims)


def _mixer(cfg: BimepelConfig, prefix: str, layer: dict):
    m = layer["mixer"]
    if layer["type"] == "attention":
        return GatedAttentionMixer(prefix, cfg.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["scale"]),
                                   cfg.eps, _positions(m), chunk=int((m.get("mask") or {}).get("size", 0)))
    return DecayLinearAttentionMixer(prefix, cfg.width, m["heads"], m["dim"], m["vdim"], m["decay"], cfg.eps)


def _feed_forward(cfg: BimepelConfig, prefix: str, mlp: dict):
    if mlp["kind"] == "dense":
        return GatedFeedForward(prefix, cfg.width, mlp["ff"], "clamped", GATE_ALPHA, float(mlp["limit"]))
    r = mlp["router"]
    return RoutedFeedForward(prefix, cfg.width, mlp["expert"]["ff"], r["experts"], r["top"], float(r["scale"]))


def build_bimepel(cfg: BimepelConfig) -> ModelSpec:
    H = cfg.width
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ffn = norm2 = None
        if layer.get("mlp") is not None:
            ffn = _feed_forward(cfg, f"{p}.mlp", layer["mlp"])
            norm2 = RMSNorm(f"{p}.norm2", H, cfg.eps)
        blocks.append(ShiftedParallelBlock(_mixer(cfg, f"{p}.mix", layer), ffn, RMSNorm(f"{p}.norm1", H, cfg.eps), norm2,
                                           f"{p}.shift", H))
    order: List[LayerCall] = []
    groups: Dict[Tuple, List] = {}  # (kind, shape) -> [name, passes so far]
    for run, i in enumerate(cfg.run_order()):
        mixer = blocks[i].mixer
        if isinstance(mixer, GatedAttentionMixer):
            key = ("kv", (mixer.kv_heads, mixer.frame, mixer.chunk))
        else:
            key = ("state", mixer.state_shape)
        entry = groups.setdefault(key, [f"{key[0]}{len(groups)}", 0])
        order.append(LayerCall(i, entry[0], entry[1], more=(("shift", "shift", run),)))
        entry[1] += 1
    cache_groups = [CacheGroupSpec("shift", CACHE_STATE, len(order), state_shape=(H,))]
    for (kind, shape), (name, count) in groups.items():
        if kind == "kv":  # a masked layer's pages behind its sequence's current block go back to the pool
            cache_groups.append(CacheGroupSpec(name, CACHE_CHUNK if shape[2] else CACHE_FULL, count, shape[0], shape[1],
                                               chunk=shape[2] or None))
        else:
            cache_groups.append(CacheGroupSpec(name, CACHE_STATE, count, state_shape=shape))
    return ModelSpec(
        config=cfg,
        embedding=Embedding("embed", cfg.vocab, H, weight_name="embed"),
        blocks=blocks,
        order=order,
        final_norm=RMSNorm("final.norm", H, cfg.eps),
        head=OutputHead("head", cfg.vocab, H, "embed"),
        cache_groups=cache_groups,
    )


register("bimepel", BimepelConfig, build_bimepel, exist_ok=True, aliases=("Bimepel",))
