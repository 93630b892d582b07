"""Linear attention with a constant decay per head, as a mixer with a state of fixed size.

With h the mixer's input and H heads of ``key_dim`` (queries, keys) and ``value_dim`` (values) elements:

    q = act(W_q h), k = act(W_k h), v = act(W_v h)         act: silu by default
    S_t = decay[head] * S_(t-1) + k_t v_t^T                per head, S: [key_dim, value_dim], zero at the start
    o_t = S_t^T q_t                                        (no other scale)
    out = W_o (rmsnorm(heads side by side) * w * sigmoid(W_g h))

The state is a row of a state table of the cache, 32-bit, as is the recurrence; the four products of h run as one.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..engine.spec import INIT_ONE_NOISE, VECTOR, TensorSpec
from .base import Part, StepContext, register_part
from .linear import Linear


class DecayLinearAttentionMixer(Part):
    def __init__(self, name: str, hidden_size: int, heads: int, key_dim: int, value_dim: int, decay: Sequence[float],
                 eps: float, act: Optional[str] = "silu"):
        if len(decay) != heads:
            raise ValueError(f"{name}: {len(decay)} decays for {heads} heads")
        self.name, self.hidden_size = name, int(hidden_size)
        self.heads, self.key_dim, self.value_dim = int(heads), int(key_dim), int(value_dim)
        self.eps, self.act = float(eps), act
        self.decay = torch.tensor([float(d) for d in decay], dtype=torch.float32)
        bare = lambda short, i, o: Linear(f"{name}.{short}", i, o, False, weight_name=f"{name}.{short}")
        self.q = bare("q", hidden_size, self.heads * self.key_dim)
        self.k = bare("k", hidden_size, self.heads * self.key_dim)
        self.v = bare("v", hidden_size, self.heads * self.value_dim)
        self.g = bare("g", hidden_size, self.heads * self.value_dim)
        self.out = bare("o", self.heads * self.value_dim, hidden_size)
        self.norm_w = None
        self.inp: Optional[Linear] = None

    @property
    def state_shape(self) -> Tuple[int, ...]:
        return (self.heads * self.key_dim * self.value_dim,)

    def children(self) -> Sequence[Part]:
        return (self.q, self.k, self.v, self.g, self.out)

    def to(self, device) -> None:
        self.decay = self.decay.to(device)

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(f"{self.name}.norm", (self.heads * self.value_dim,), VECTOR, INIT_ONE_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.norm_w = tensors[f"{self.name}.norm"]

    def after_load(self) -> None:
        self.inp = Linear.stacked(f"{self.name}.qkvg", [self.q, self.k, self.v, self.g])

    def check_sizes(self) -> None:
        if self.key_dim > 256:
            raise ValueError(f"{self.name}: keys of {self.key_dim} elements are more than the 256 the kernel holds")

    def input_projection(self):
        """The first product of ``forward`` (see ``GatedAttentionMixer.input_projection``)."""
        return self.inp, {}

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None, projected=None):
        state = ctx.cache.state_layer(call.cache_group, call.cache_layer)
        H, dk, dv = self.heads, self.key_dim, self.value_dim
        proj = projected if projected is not None else self.inp(x)
        a, b, c = H * dk, 2 * H * dk, 2 * H * dk + H * dv
        o = ops.decay_scan(proj[:, :a], proj[:, a:b], proj[:, b:c], self.decay, state, ctx.cu_tokens, ctx.seq_slot, H, dk,
                           dv, act=self.act, max_new=max(ctx.new_tokens))
        gated = ops.gated_heads(o, dv, proj[:, c:], H, dv, x.dtype, w=self.norm_w, eps=self.eps)
        return self.out(gated, add1=residual)


register_part("mixer", "decay_linear_attention", DecayLinearAttentionMixer)
