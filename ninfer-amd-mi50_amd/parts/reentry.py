"""The embedding's output mixed into the residual stream again: x <- W [x ; x0], one product
over the stream x and the embedding output x0 side by side (W: [hidden, 2 hidden], x's
columns first). A model's plan names such a part in front of a layer's run; the new stream
is 32-bit like the old one."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import Part, StepContext, WeightBinder, settle


class StreamReentry(Part):
    def __init__(self, tensor: str, hidden: int):
        self.tensor = tensor
        self.hidden = hidden
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.hidden, 2 * self.hidden))}

    def bind(self, w: WeightBinder) -> None:
        self.weight = w.matrix(self.tensor)

    def forward(self, ctx: StepContext, residual: torch.Tensor, pending,
                first: torch.Tensor) -> torch.Tensor:
        """The new residual from the old one (+ what is still to be added to it) and the
        embedding output `first`."""
        rows = settle(ctx, residual, pending)
        if rows is not None:
            residual.add_(rows)
        both = ctx.empty((ctx.T, 2 * self.hidden))
        ctx.ops.concat_rows(residual, first, both)
        out = ctx.empty((ctx.T, self.hidden), torch.float32)
        ctx.ops.linear(both, self.weight, out)
        return out


register_part("input", "stream_reentry", StreamReentry)
