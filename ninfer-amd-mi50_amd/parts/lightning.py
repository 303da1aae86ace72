"""Lightning attention: linear attention with a fixed decay per head.

    q = silu(W_q h), k = silu(W_k h)   (heads x dim),   v = silu(W_v h)   (heads x vdim)
    S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t          (per head, no other scale)
    y = W_o ( rmsnorm(concat_h o_t) * weight * sigmoid(W_g h) )

The four input products are one product over the stacked weight [2 H dim + 2 H vdim, hidden]
(q, k, v, gate); the recurrence, its state and the norm are 32-bit. The state S ([heads, dim,
vdim] per request) lives in the request's state slot, starts at zero, and is carried from
step to step: nothing is kept per token, so the mixer asks for no pages.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CallInfo, Mixer, StepContext, WeightBinder


class LightningAttention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int,
                 decay: Sequence[float], eps: float,
                 names=("q", "k", "v", "g", "o", "norm")):
        """`decay` [heads]: the factor on the state per token, one per head. `names`: what
        follows the prefix in the names of W_q, W_k, W_v, W_g, W_o and the norm's weight."""
        if len(decay) != heads:
            raise ValueError(f"decay has {len(decay)} entries for {heads} heads")
        self.prefix = prefix
        self.hidden = hidden
        self.heads = heads
        self.dim = dim
        self.vdim = vdim
        self.decay_values = [float(d) for d in decay]
        self.eps = eps
        self.names = tuple(names)
        self.w_in: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.norm_w: Optional[torch.Tensor] = None
        self.decay: Optional[torch.Tensor] = None

    def state_floats(self) -> int:
        return self.heads * self.dim * self.vdim

    def _widths(self):
        qk, v = self.heads * self.dim, self.heads * self.vdim
        return qk, qk, v, v

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, n = self.prefix, self.names
        qk, _, v, _ = self._widths()
        return {p + n[0]: TensorSpec((qk, self.hidden)), p + n[1]: TensorSpec((qk, self.hidden)),
                p + n[2]: TensorSpec((v, self.hidden)), p + n[3]: TensorSpec((v, self.hidden)),
                p + n[4]: TensorSpec((self.hidden, v)), p + n[5]: TensorSpec((v,), "gain")}

    def bind(self, w: WeightBinder) -> None:
        p, n = self.prefix, self.names
        widths = self._widths()
        self.w_in = torch.empty((sum(widths), self.hidden), dtype=w.act_dtype, device=w.device)
        at = 0
        for name, width in zip(n[:4], widths):
            w.matrix_into(p + name, self.w_in[at:at + width])
            at += width
        self.w_o = w.matrix(p + n[4])
        self.norm_w = w.float32(p + n[5])
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=w.device)

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops = ctx.ops
        qk, _, v, _ = self._widths()
        proj = ctx.empty((ctx.T, 2 * qk + 2 * v))
        ops.linear(x, self.w_in, proj)
        o = ctx.empty((ctx.T, v), torch.float32)
        ops.lightning_attention(proj, 0, qk, 2 * qk, self.heads, self.dim, self.vdim, self.decay,
                                call.state, ctx, o)
        gated = ctx.empty((ctx.T, v))
        ops.gated_rmsnorm(o, proj[:, 2 * qk + v:], self.norm_w, self.eps, gated)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(gated, self.w_o, out)
        return out


register_part("mixer", "lightning", LightningAttention)
