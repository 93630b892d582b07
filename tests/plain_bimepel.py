"""A plain, slow implementation of the Bimepel design in float64 on the CPU: one function per mechanism, written
from the equations in each docstring, sharing no code with the package.  A sequence is walked token by token;
what a sequence keeps between tokens is a dict per layer run that the functions read and update.

``weights``: name -> float64 tensor, under the names of the weight file.  ``cfg``: the dict of ``config.json``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last dimension."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def shift_mix(h: torch.Tensor, before: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h + (before - h) * mu, element by element; ``before`` is the preceding token's h (zeros at position 0)."""
    return h + (before - h) * mu


def yarn_frequencies(rot: dict):
    """The rotation's frequencies [dims / 2] and the factor on cosines and sines.

    f_i = base^(-2i / dims).  With ``scaling`` (factor s, original length L, fast, slow): the index at which a
    frequency turns t times within L is n(t) = dims * ln(L / (2 pi t)) / (2 ln base); lo = max(floor(n(fast)), 0),
    hi = min(ceil(n(slow)), dims - 1); r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); the frequency becomes
    f_i / s * r_i + f_i * (1 - r_i), and cosines and sines are multiplied by 0.1 ln(s) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0
    s, L = float(sc["factor"]), float(sc["original"])
    n = lambda t: dims * math.log(L / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(n(float(sc["fast"]))), 0)
    hi = min(math.ceil(n(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / s * r + f[i] * (1.0 - r))
    return torch.tensor(out, dtype=F), 0.1 * math.log(s) + 1.0


def rotate(v: torch.Tensor, pos: int, freqs: torch.Tensor, mult: float) -> torch.Tensor:
    """The first 2 * len(freqs) elements of every head (last dimension) rotated in pairs (i, i + half) by the
    angle pos * freqs[i]; cosine and sine times ``mult``; the rest unchanged."""
    half = freqs.shape[0]
    a = pos * freqs
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    u, w = v[..., :half], v[..., half:2 * half]
    return torch.cat([u * c - w * s, w * c + u * s, v[..., 2 * half:]], dim=-1)


def attention_token(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor, pos: int, kept: dict):
    """One token through the attention mixer.  ``kept["k"]``, ``kept["v"]``: lists of the keys and values so far."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (W[f"{p}.q"] @ h).view(H, d)
    k = (W[f"{p}.k"] @ h).view(G, d)
    v = (W[f"{p}.v"] @ h).view(G, dv)
    q = rms(q, eps) * W[f"{p}.q.norm"]
    k = rms(k, eps) * W[f"{p}.k.norm"]
    rot = m.get("rot")
    if rot:
        freqs, mult = yarn_frequencies(rot)
        q, k = rotate(q, pos, freqs, mult), rotate(k, pos, freqs, mult)
    v = rms(v, eps)
    kept.setdefault("k", []).append(k)
    kept.setdefault("v", []).append(v)
    size = (m.get("mask") or {}).get("size")
    first = (pos // size) * size if size else 0
    keys = torch.stack(kept["k"][first:pos + 1])  # [n, G, d]
    vals = torch.stack(kept["v"][first:pos + 1])
    out = []
    for head in range(H):
        g = head // (H // G)
        s = (keys[:, g] @ q[head]) * float(m["scale"])
        w = torch.softmax(s, dim=0)
        out.append(w @ vals[:, g])
    o = torch.cat(out) * torch.sigmoid(W[f"{p}.g"] @ h)
    return W[f"{p}.o"] @ o


def lightning_token(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor, kept: dict):
    """One token through the linear-attention mixer: S <- decay_head * S + k v^T, o = S^T q per head, with q, k, v
    = silu of their projections; the heads side by side are RMS-normed with a weight, gated by sigmoid(W_g h),
    and projected."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = silu(W[f"{p}.q"] @ h).view(H, d)
    k = silu(W[f"{p}.k"] @ h).view(H, d)
    v = silu(W[f"{p}.v"] @ h).view(H, dv)
    S = kept.get("S")
    if S is None:
        S = torch.zeros(H, d, dv, dtype=F)
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=F).view(H, 1, 1)
    S = decay * S + k.unsqueeze(2) * v.unsqueeze(1)
    kept["S"] = S
    o = torch.einsum("hde,hd->he", S, q).reshape(-1)
    o = rms(o, eps) * W[f"{p}.norm"] * torch.sigmoid(W[f"{p}.g"] @ h)
    return W[f"{p}.o"] @ o


def dense_ff(W, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g * sigmoid(1.702 g) * (u + 1))."""
    lim = float(mlp["limit"])
    g = torch.clamp(W[f"{p}.gate"] @ h, max=lim)
    u = torch.clamp(W[f"{p}.up"] @ h, -lim, lim)
    return W[f"{p}.down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1.0))


def routed_ff(W, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    """Scores sigmoid(W_router h); the ``top`` largest are taken, divided by their sum (+ 1e-20), times
    ``scale``; the result is the so weighted sum of W_down (silu(W_gate h) * (W_up h)) of the taken experts."""
    r = mlp["router"]
    s = torch.sigmoid(W[f"{p}.router"] @ h)
    top = torch.topk(s, int(r["top"]))
    wts = top.values / (top.values.sum() + 1e-20) * float(r["scale"])
    out = torch.zeros(W[f"{p}.e0.down"].shape[0], dtype=F)
    for w, e in zip(wts.tolist(), top.indices.tolist()):
        a = torch.nn.functional.silu(W[f"{p}.e{e}.gate"] @ h) * (W[f"{p}.e{e}.up"] @ h)
        out = out + w * (W[f"{p}.e{e}.down"] @ a)
    return out


def run_order(cfg: dict) -> List[int]:
    """Indices of the layers in the order they run: layers start .. stop - 1 ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, t = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


class PlainBimepel:
    def __init__(self, cfg: dict, weights: Dict[str, torch.Tensor]):
        self.cfg = cfg
        self.W = {k: v.to(F) for k, v in weights.items()}
        self.eps = float(cfg["norm"]["eps"])
        self.order = run_order(cfg)

    def new_sequence(self) -> dict:
        return {"pos": 0, "runs": [dict() for _ in self.order]}

    def token(self, seq: dict, tok: int, streams: Optional[list] = None) -> torch.Tensor:
        """Feed one token; returns its logits.  ``streams``: gets the stream after every layer run."""
        W, eps = self.W, self.eps
        x = W["embed"][tok]
        pos = seq["pos"]
        for run, li in enumerate(self.order):
            layer, p, kept = self.cfg["layers"][li], f"l{li}", seq["runs"][run]
            h = rms(x, eps) * W[f"{p}.norm1"]
            before = kept.get("h", torch.zeros_like(h))
            kept["h"] = h
            h = shift_mix(h, before, W[f"{p}.shift"])
            if layer["type"] == "attention":
                mixed = attention_token(W, f"{p}.mix", layer["mixer"], eps, h, pos, kept)
            else:
                mixed = lightning_token(W, f"{p}.mix", layer["mixer"], eps, h, kept)
            mlp = layer.get("mlp")
            if mlp is not None:
                n2 = rms(x, eps) * W[f"{p}.norm2"]
                ff = dense_ff(W, f"{p}.mlp", mlp, n2) if mlp["kind"] == "dense" else routed_ff(W, f"{p}.mlp", mlp, n2)
                mixed = mixed + ff
            x = x + mixed
            if streams is not None:
                streams.append(x)
        seq["pos"] = pos + 1
        return W["embed"] @ (rms(x, eps) * W["final.norm"])

    def logits(self, tokens) -> torch.Tensor:
        seq = self.new_sequence()
        return torch.stack([self.token(seq, int(t)) for t in tokens])
