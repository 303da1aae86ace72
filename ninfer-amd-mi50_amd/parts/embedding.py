"""Token embedding and the logits head.

Embedding: x[t] = table[token[t]] (reference src/ops/kernels.hip:150-159),
written straight into the 32-bit residual; with `positions` > 0 a table of that many learned
absolute positions (`position_prefix + "weight"`) is gathered by the rows' positions and added
in the same kernel (no counterpart in the reference: its models rotate). Head: logits = n W^T in 32-bit for
the asked rows only (reference src/models/model.hip:735-752); with tied
embeddings the head is the embedding table itself, not a copy (the reference
loads a second copy, :496-500).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.source import TensorSpec
from .base import Part, StepContext, WeightBinder


class TokenEmbedding(Part):
    def __init__(self, prefix: str, vocab: int, hidden: int, positions: int = 0,
                 position_prefix: Optional[str] = None, leaf: str = "weight", scale: float = 1.0,
                 pairs: Optional[Dict[str, object]] = None):
        """`leaf`: what follows the prefixes in the tensors' names ('' when a prefix is the
        whole name). `scale` multiplies the token's row. `pairs` ({'tensor', 'buckets',
        'mul_prev', 'mul_cur'}): a hashed table of token pairs [buckets + 1, hidden] whose row
        (previous token x mul_prev + token x mul_cur) mod buckets is added, its last row for a
        request's first token; the previous token is one number of per-request state."""
        self.scale = float(scale)
        self.pairs = dict(pairs) if pairs else None
        if self.pairs and positions:
            raise ValueError("a table of token pairs and learned positions are not built together")
        self.pair_table: Optional[torch.Tensor] = None
        self.prefix = prefix
        self.leaf = leaf
        self.vocab = vocab
        self.hidden = hidden
        self.positions = positions   # rows of the table of learned positions (0: none)
        self.position_prefix = position_prefix
        if positions and not position_prefix:
            raise ValueError("learned positions need the name prefix of their table")
        self.table: Optional[torch.Tensor] = None
        self.position_table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {self.prefix + self.leaf: TensorSpec((self.vocab, self.hidden))}
        if self.positions:
            specs[self.position_prefix + self.leaf] = TensorSpec((self.positions, self.hidden))
        if self.pairs:
            specs[self.pairs["tensor"]] = TensorSpec((int(self.pairs["buckets"]) + 1, self.hidden))
        return specs

    def state_floats(self) -> int:
        """32-bit numbers of per-request state: the previous token, where pairs are hashed."""
        return 1 if self.pairs else 0

    def bind(self, w: WeightBinder) -> None:
        self.table = w.matrix(self.prefix + self.leaf)
        if self.positions:
            self.position_table = w.matrix(self.position_prefix + self.leaf)
        if self.pairs:
            self.pair_table = w.matrix(self.pairs["tensor"])

    def max_positions(self) -> Optional[int]:
        return self.positions or None

    def forward(self, ctx: StepContext, state: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`state`: this part's columns of the per-request state ([slots, 1]) when it keeps any."""
        residual = ctx.empty((ctx.T, self.hidden), torch.float32)
        if self.pairs or self.scale != 1.0:
            p = self.pairs or {}
            ctx.ops.embed_pairs(ctx, self.table, residual, self.scale, self.pair_table,
                                int(p.get("buckets", 0)), int(p.get("mul_prev", 0)),
                                int(p.get("mul_cur", 0)), state)
            return residual
        ctx.ops.embed(ctx.tokens, self.table, residual, positions=ctx.positions,
                      pos_table=self.position_table)
        return residual


class LMHead(Part):
    def __init__(self, prefix: str, vocab: int, hidden: int,
                 tied_to: Optional[TokenEmbedding] = None, leaf: str = "weight",
                 softcap: float = 0.0):
        """`softcap` > 0: logits <- softcap tanh(logits / softcap)."""
        self.softcap = float(softcap)
        self.prefix = prefix
        self.leaf = leaf
        self.vocab = vocab
        self.hidden = hidden
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.tied_to is not None:
            return {}
        return {self.prefix + self.leaf: TensorSpec((self.vocab, self.hidden))}

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        # a checkpoint of a tied model may still carry the head: a copy of the table
        if self.tied_to is not None:
            return {self.prefix + self.leaf: TensorSpec((self.vocab, self.hidden))}
        return {}

    def bind(self, w: WeightBinder) -> None:
        if self.tied_to is None:
            self.weight = w.matrix(self.prefix + self.leaf)

    def forward(self, ctx: StepContext, normed_rows: torch.Tensor) -> torch.Tensor:
        weight = self.tied_to.table if self.tied_to is not None else self.weight
        logits = ctx.empty((normed_rows.shape[0], self.vocab), torch.float32)
        ctx.ops.linear(normed_rows, weight, logits)
        if self.softcap > 0:
            ctx.ops.tanh_cap(logits, self.softcap)
        return logits
