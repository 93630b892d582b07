"""The Pavodra design as a list of parts: the builder registered for ``model_type: pavodra`` (a ``config.json``
that says ``"architecture": "Pavodra"``).

A layer is a ``PostNormBlock``: the mixer and the feed-forward read the stream itself, an RMS norm with a gain
stored around zero stands on each one's output, and the result enters the stream times ``residual_mult``; after
every layer the streams of all layers so far are mixed by learned weights (``DepthMix``).  The mixer is attention
over a cache of latents, a gated recurrence, or a state-space recurrence, by the layer's ``type``.  The head is the
embedding table, on the final norm's output, times ``logit_scale``.

Tensor names: ``embed``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.dwa``,
``l<i>.mix.<name>``, ``l<i>.mlp.up``, ``l<i>.mlp.down``.

Layers of one kind and one shape share a cache group (a page pool of latent rows, or a state table).
"""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..config.pavodra import PavodraConfig
from ..config.registry import register
from ..parts import (DenseFeedForward, DepthMix, Embedding, GatedScanMixer, LatentAttentionMixer, OutputHead,
                     PostNormBlock, RMSNorm, RotaryPositions, StateSpaceMixer)
from .spec import CACHE_FULL, CACHE_STATE, CacheGroupSpec, LayerCall, ModelSpec


def _mixer(cfg: PavodraConfig, prefix: str, layer: dict):
    m, kind = layer["mixer"], layer["type"]
    if kind == "latent_attention":
        positions = RotaryPositions(m["rot_dim"], float(m["rot"]["base"]), rotary_dim=int(m["rot"]["dims"]),
                                    pairing="interleaved")
        return LatentAttentionMixer(prefix, cfg.width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                    float(m["scale"]), cfg.eps, positions)
    if kind == "mingru":
        return GatedScanMixer(prefix, cfg.width, m["width"])
    return StateSpaceMixer(prefix, cfg.width, m["heads"], m["vdim"], m["state"], m["groups"], m["conv"],
                           m["norm_groups"], cfg.eps)


def build_pavodra(cfg: PavodraConfig) -> ModelSpec:
    H, L = cfg.width, len(cfg.layers)
    blocks, order = [], []
    groups: Dict[Tuple, List] = {}  # (kind, shape) -> [name, layers so far]
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        mixer = _mixer(cfg, f"{p}.mix", layer)
        ffn = norm2 = None
        if layer.get("mlp") is not None:
            ffn = DenseFeedForward(f"{p}.mlp", H, layer["mlp"]["ff"], False, "relu2", "up", "down", bare_names=True)
            norm2 = RMSNorm(f"{p}.norm2", H, cfg.eps, offset=1.0)
        blocks.append(PostNormBlock(mixer, ffn, RMSNorm(f"{p}.norm1", H, cfg.eps, offset=1.0), norm2,
                                    cfg.residual_mult, DepthMix(f"{p}.dwa", i, L)))
        if isinstance(mixer, LatentAttentionMixer):
            key = ("latent", mixer.cache_row)
        else:
            key = ("state", mixer.state_shape)
        entry = groups.setdefault(key, [f"{key[0]}{len(groups)}", 0])
        order.append(LayerCall(i, entry[0], entry[1]))
        entry[1] += 1
    cache_groups = []
    for (kind, shape), (name, count) in groups.items():
        if kind == "latent":
            cache_groups.append(CacheGroupSpec(name, CACHE_FULL, count, 1, shape, values=False))
        else:
            cache_groups.append(CacheGroupSpec(name, CACHE_STATE, count, state_shape=shape))
    return ModelSpec(
        config=cfg,
        embedding=Embedding("embed", cfg.vocab, H, weight_name="embed"),
        blocks=blocks,
        order=order,
        final_norm=RMSNorm("final.norm", H, cfg.eps, offset=1.0),
        head=OutputHead("head", cfg.vocab, H, "embed", scale=cfg.logit_scale),
        cache_groups=cache_groups,
    )


register("pavodra", PavodraConfig, build_pavodra, exist_ok=True, aliases=("Pavodra",))
