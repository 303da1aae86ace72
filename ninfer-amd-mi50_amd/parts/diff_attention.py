"""Differential attention over the paged cache, with grouped key/value heads.

Every query head runs two softmax attentions ("maps") over the same values: q and k hold two
vectors of `dim` numbers per head, laid out head by head as [map 1 | map 2]; values have
`vdim` numbers. With a1 and a2 the two maps' outputs,
    o = a1 - lam a2,   lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff   (one number a layer),
then o is divided by its root mean square over the head's vdim values (eps inside the root)
and multiplied by 1 - diff; the heads go through the output projection. Scores are
(q . k) scale temp(p), with temp(p) = 1 + temp_coef ln(floor((p + 1) / temp_every) + 1) at
the row's position p (no rotation: positions enter here only), then softcap tanh(score /
softcap); causal. Query head h reads kv head h // (heads / kv_heads). Scores, softmax, the
difference and the norm are 32-bit; the cache holds k [2 dim] and v [vdim] per kv head in
pools of their own.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CacheNeed, CallInfo, Mixer, PoolSpec, StepContext, WeightBinder


class DifferentialAttention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 scale: float, diff: float, eps: float, softcap: float = 0.0,
                 temp_coef: float = 0.0, temp_every: int = 1, page_size: Optional[int] = None,
                 names=("q", "k", "v", "o", "lq1", "lk1", "lq2", "lk2")):
        """`names`: what follows the prefix in the names of the three projections, the output
        projection and the four vectors [dim] that lam is made of. `softcap` 0: scores are not
        capped; `temp_coef` 0: no query temperature."""
        if heads % kv_heads:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = hidden, heads, kv_heads, dim, vdim
        self.scale, self.diff, self.eps, self.softcap = float(scale), float(diff), float(eps), float(softcap)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.page_size = page_size
        self.lam: Optional[float] = None
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    @property
    def qkv_width(self) -> int:
        return (self.heads + self.kv_heads) * 2 * self.dim + self.kv_heads * self.vdim

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed((PoolSpec("k", (self.kv_heads,), (2 * self.dim,)),
                          PoolSpec("v", (self.kv_heads,), (self.vdim,))), None, self.page_size)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, n, d = self.prefix, self.names, self.dim
        specs = {p + n[0]: TensorSpec((self.heads * 2 * d, self.hidden)),
                 p + n[1]: TensorSpec((self.kv_heads * 2 * d, self.hidden)),
                 p + n[2]: TensorSpec((self.kv_heads * self.vdim, self.hidden)),
                 p + n[3]: TensorSpec((self.hidden, self.heads * self.vdim))}
        for leaf in n[4:]:
            specs[p + leaf] = TensorSpec((d,), "bias")
        return specs

    def bind(self, w: WeightBinder) -> None:
        p, n = self.prefix, self.names
        nq, nk = self.heads * 2 * self.dim, self.kv_heads * 2 * self.dim
        self.w_qkv = torch.empty((self.qkv_width, self.hidden), dtype=w.act_dtype, device=w.device)
        w.matrix_into(p + n[0], self.w_qkv[:nq])
        w.matrix_into(p + n[1], self.w_qkv[nq:nq + nk])
        w.matrix_into(p + n[2], self.w_qkv[nq + nk:])
        self.w_o = w.matrix(p + n[3])
        lq1, lk1, lq2, lk2 = (w.float32(p + leaf) for leaf in n[4:])
        # one number for the layer, formed once in 32-bit
        lam = torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) \
            + torch.tensor(self.diff, dtype=torch.float32, device=lq1.device)
        self.lam = float(lam)
        if not math.isfinite(self.lam):
            raise ValueError(f"{p}: the vectors of the maps' weight give no finite number")

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops, cache = ctx.ops, call.cache
        qkv = ctx.empty((ctx.T, self.qkv_width))
        ops.linear(x, self.w_qkv, qkv)
        attn = ctx.empty((ctx.T, self.heads * self.vdim))
        ops.diff_attention(qkv, cache["k"], cache["v"], cache.block_table, ctx, self.heads,
                           self.kv_heads, self.dim, self.vdim, cache.page_size, self.scale,
                           self.softcap, self.temp_coef, self.temp_every, self.lam, self.eps,
                           1.0 - self.diff, attn, write_kv=call.writes_cache)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(attn, self.w_o, out)
        return out


register_part("mixer", "differential_attention", DifferentialAttention)
