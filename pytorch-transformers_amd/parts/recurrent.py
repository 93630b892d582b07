"""Mixers that carry a state of fixed size per sequence instead of keys and values.

``GatedScanMixer`` (minGRU): ``z = sigmoid(W_z h + b_z)``, ``u = W_x h + b_x``, candidate ``c = u + 1/2`` where
``u >= 0`` and ``sigmoid(u)`` below, ``S_t = (1 - z) S_(t-1) + z c`` element by element, output
``W_o (S_t * silu(W_g h))``.

``StateSpaceMixer`` (Mamba-2): one input product laid out ``[z | x | B | C | dt]``; x, B and C pass a short causal
convolution per channel and silu; ``dt = softplus(dt + dt_bias)``; per head, with the group's B and C,
``S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T`` and ``y_t = S_t^T C_t + D x_t``; y times ``silu(z)`` is
RMS-normed in equal groups, weighted, and projected out.

Both keep their state in 32-bit in a row of a state table of the cache (zero when a slot is handed out), read
and left by one launch per step that walks each sequence's tokens in order; the convolution's last inputs are part
of the state row.  The matrix products run in the compute type like any other layer's; gates, decays, step sizes and
states are 32-bit.  A file holds every tensor under ``name.<short name>`` as it stands.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..engine.spec import INIT_NORMAL, INIT_ONE_NOISE, INIT_ZERO_NOISE, VECTOR, TensorSpec
from .base import Part, StepContext, register_part
from .linear import Linear
from .norms import RMSNorm


def _bare(name: str, short: str, fan_in: int, fan_out: int, bias: bool = False) -> Linear:
    return Linear(f"{name}.{short}", fan_in, fan_out, bias, weight_name=f"{name}.{short}", bias_name=f"{name}.{short}.b")


class GatedScanMixer(Part):
    def __init__(self, name: str, hidden_size: int, width: int):
        self.name, self.hidden_size, self.width = name, int(hidden_size), int(width)
        self.z = _bare(name, "z", hidden_size, width, True)
        self.x = _bare(name, "x", hidden_size, width, True)
        self.g = _bare(name, "g", hidden_size, width)
        self.out = _bare(name, "o", width, hidden_size)
        self.zxg: Optional[Linear] = None

    @property
    def state_shape(self) -> Tuple[int, ...]:
        return (self.width,)

    def children(self) -> Sequence[Part]:
        return (self.z, self.x, self.g, self.out)

    def after_load(self) -> None:
        self.zxg = Linear.stacked(f"{self.name}.zxg", [self.z, self.x, self.g])  # the three read one input: one product

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None):
        state = ctx.cache.state_layer(call.cache_group, call.cache_layer)
        zxg = self.zxg(x)
        y = ops.gated_scan(zxg, self.z.bias, self.x.bias, state, ctx.cu_tokens, ctx.seq_slot, max_new=max(ctx.new_tokens))
        return self.out(y, add1=residual)


class StateSpaceMixer(Part):
    def __init__(self, name: str, hidden_size: int, heads: int, head_dim: int, state_rows: int, groups: int, taps: int,
                 norm_groups: int, eps: float):
        if heads % groups:
            raise ValueError(f"{name}: {heads} heads do not split into {groups} groups")
        self.name, self.hidden_size = name, int(hidden_size)
        self.heads, self.head_dim, self.state_rows, self.groups, self.taps = int(heads), int(head_dim), int(state_rows), int(groups), int(taps)
        self.inner = self.heads * self.head_dim
        self.channels = self.inner + 2 * self.groups * self.state_rows  # what the convolution runs over
        self.inp = _bare(name, "in", hidden_size, self.inner + self.channels + self.heads)
        self.out = _bare(name, "o", self.inner, hidden_size)
        self.norm = RMSNorm(f"{name}.norm", self.inner, eps, offset=0.0, groups=norm_groups)
        self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d_skip = None

    @property
    def state_shape(self) -> Tuple[int, ...]:
        """The recurrence's state ``[heads, state_rows, head_dim]``, then the convolution's last ``taps - 1`` inputs."""
        return (self.heads * self.state_rows * self.head_dim + (self.taps - 1) * self.channels,)

    def children(self) -> Sequence[Part]:
        return (self.inp, self.out, self.norm)

    def check_sizes(self) -> None:
        if not (1 <= self.taps <= 16):
            raise ValueError(f"{self.name}: a convolution of {self.taps} taps is outside the 1..16 that the kernel takes")
        if self.state_rows > 256:
            raise ValueError(f"{self.name}: a state of {self.state_rows} rows per head is more than the kernel's 256")

    def tensor_specs(self) -> List[TensorSpec]:
        n = self.name
        return [TensorSpec(f"{n}.conv", (self.channels, self.taps), VECTOR, INIT_NORMAL),
                TensorSpec(f"{n}.conv.b", (self.channels,), VECTOR, INIT_ZERO_NOISE),
                TensorSpec(f"{n}.dt_bias", (self.heads,), VECTOR, INIT_ZERO_NOISE),
                TensorSpec(f"{n}.A_log", (self.heads,), VECTOR, INIT_ZERO_NOISE),
                TensorSpec(f"{n}.D", (self.heads,), VECTOR, INIT_ONE_NOISE)]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.name
        self.conv_w, self.conv_b = tensors[f"{n}.conv"], tensors[f"{n}.conv.b"]
        self.dt_bias, self.a_log, self.d_skip = tensors[f"{n}.dt_bias"], tensors[f"{n}.A_log"], tensors[f"{n}.D"]

    def forward(self, x: torch.Tensor, ctx: StepContext, call, residual: Optional[torch.Tensor] = None):
        row = ctx.cache.state_layer(call.cache_group, call.cache_layer)
        cut = self.heads * self.state_rows * self.head_dim
        proj = self.inp(x)
        gate = proj[:, :self.inner]
        xbc = ops.conv_silu(proj[:, self.inner:self.inner + self.channels], self.conv_w, self.conv_b, row[:, cut:],
                            ctx.cu_tokens, ctx.token_seq, ctx.seq_slot)
        y = ops.ssm_scan(xbc, proj[:, self.inner + self.channels:], self.dt_bias, self.a_log, self.d_skip, row[:, :cut],
                         ctx.cu_tokens, ctx.seq_slot, self.heads, self.head_dim, self.state_rows, self.groups,
                         max_new=max(ctx.new_tokens))
        normed = self.norm.apply(y, ctx.dtype, gate=gate)[0]
        return self.out(normed, add1=residual)


register_part("mixer", "gated_scan", GatedScanMixer)
register_part("mixer", "state_space", StateSpaceMixer)
