"""A short causal convolution over time on every channel, added to its input:

    out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j),   j = 0 .. taps - 1,

with zeros before a request's first row. The last taps - 1 inputs of a request are
per-request state (32-bit, in the request's state slot), so a request may be cut into
steps anywhere. The input is the 32-bit residual; the sum is 32-bit and the result is
rounded once to the activation dtype. Weights: one tensor [channels, taps], no bias.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import Part, StepContext, WeightBinder


class ShortConv(Part):
    def __init__(self, tensor: str, channels: int, taps: int):
        if taps < 1:
            raise ValueError(f"a convolution has at least one tap, got {taps}")
        self.tensor = tensor
        self.channels = channels
        self.taps = taps
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.channels, self.taps))}

    def bind(self, w: WeightBinder) -> None:
        self.weight = w.float32(self.tensor)

    def state_floats(self) -> int:
        return (self.taps - 1) * self.channels

    def forward(self, ctx: StepContext, residual: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        """`state`: this convolution's columns of the per-request state, [slots, state_floats()]."""
        out = ctx.empty((residual.shape[0], self.channels))
        ctx.ops.short_conv(residual, self.weight, state, ctx, out)
        return out


register_part("input", "short_conv", ShortConv)
