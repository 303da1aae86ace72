"""A model as data: its parts and the order they run in.

`blocks` are the model's layers; `plan` is the order they run in, one
`LayerCall` per run. The plan is data: it may name a layer twice (the layer's
weights run again, with a cache of their own unless told otherwise) or let a
call read the cache another call wrote (`cache_from`), in which case the call
writes no keys and values of its own. An entry may name a part that the residual stream
passes through in front of the layer's run (`before`, an index into `joins`): such a part
makes a new stream from the old one and the embedding's output.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..parts.base import Block, CallInfo, Norm, Part, StepContext, WeightBinder
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.source import TensorSpec


@dataclass(frozen=True)
class LayerCall:
    layer: int                       # index into ModelSpec.blocks
    cache_from: Optional[int] = None  # index of an earlier plan entry whose cache is read
    before: Optional[int] = None     # index into ModelSpec.joins: what the stream passes first


class ModelSpec:
    def __init__(self, embedding: TokenEmbedding, blocks: List[Block], final_norm: Norm,
                 head: LMHead, plan: Optional[List[LayerCall]] = None,
                 vocab_size: Optional[int] = None, eos_token_ids=(),
                 joins: Optional[List[Part]] = None):
        self.embedding = embedding
        self.blocks = blocks
        # parts that plan entries name in `before`: forward(ctx, residual, pending, first)
        # -> the new residual, `first` being the embedding's output
        self.joins: List[Part] = list(joins or [])
        self.final_norm = final_norm
        self.head = head
        self.vocab_size = vocab_size if vocab_size is not None else head.vocab
        self.eos_token_ids = tuple(eos_token_ids)   # ids that end a generation by default
        self.plan: List[LayerCall] = []
        self.set_plan(plan if plan is not None else [LayerCall(i) for i in range(len(blocks))])

    def set_plan(self, plan: List[LayerCall]) -> None:
        """Replace the order the layers run in (before the model is bound to a
        cache); refuses entries that name no layer or read a cache that is not
        written earlier."""
        for i, call in enumerate(plan):
            if not 0 <= call.layer < len(self.blocks):
                raise ValueError(f"plan entry {i} names layer {call.layer}; the model has "
                                 f"{len(self.blocks)}")
            if call.before is not None and not 0 <= call.before < len(self.joins):
                raise ValueError(f"plan entry {i} names join {call.before}; the model has "
                                 f"{len(self.joins)}")
            if call.cache_from is not None:
                if not 0 <= call.cache_from < i:
                    raise ValueError(f"plan entry {i} reads the cache of entry "
                                     f"{call.cache_from}, which does not run before it")
                if plan[call.cache_from].cache_from is not None:
                    raise ValueError(f"plan entry {i} reads the cache of entry "
                                     f"{call.cache_from}, which has no cache of its own")
        self.plan = list(plan)

    def parts(self) -> List[Part]:
        return [self.embedding, *self.joins, *self.blocks, self.final_norm, self.head]

    def max_positions(self) -> Optional[int]:
        """The longest request the parts allow (None: no part limits it)."""
        limits = [x for x in (p.least_max_positions() for p in self.parts()) if x is not None]
        return min(limits) if limits else None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for p in self.parts():
            out.update(p.all_tensor_specs())
        return out

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for p in self.parts():
            out.update(p.all_unused_tensor_specs())
        return out

    def bind(self, w: WeightBinder) -> None:
        for p in self.parts():
            p.bind_all(w)

    # ---- one step over the rows of `ctx` -----------------------------------
    def forward(self, ctx: StepContext, calls: List[CallInfo],
                logit_rows: Optional[torch.Tensor],
                embedding_state: Optional[torch.Tensor] = None,
                tap=None) -> Optional[torch.Tensor]:
        """Run all plan entries over the step's rows; logits [R, vocab] (32-bit)
        at `logit_rows`, or None when no logits are asked for. `embedding_state`: the
        embedding's columns of the per-request state, when it keeps any. `tap(i, residual,
        pending)` is called after plan entry i (debugging, tests)."""
        if embedding_state is not None:
            residual = self.embedding.forward(ctx, embedding_state)
        else:
            residual = self.embedding.forward(ctx)
        # the embedding's output, kept when a join will read it (the blocks add into `residual`)
        first = residual.clone() if any(c.before is not None for c in self.plan) else None
        pending = None
        for i, (call, info) in enumerate(zip(self.plan, calls)):
            if call.before is not None:
                residual = self.joins[call.before].forward(ctx, residual, pending, first)
                pending = None
            pending = self.blocks[call.layer].forward(ctx, residual, pending, info)
            if tap is not None:
                tap(i, residual, pending)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        normed = self.final_norm.forward_rows(ctx, residual, logit_rows, pending)
        return self.head.forward(ctx, normed)
