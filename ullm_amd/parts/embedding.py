"""Embedders: token ids to the first rows of the residual stream.

``table_sum``: the token's row times a scale, plus optionally a row of a second table chosen by a hash of
the previous and the current id (a hashed bigram table whose last row serves a request's first token),
plus optionally a fixed sinusoidal row for the token's position (entry 2i = sin(p * base^(-2i/width)),
entry 2i+1 = the cosine of the same angle).  The id before an entry's first token is state: one int32
per request slot, written by the step that saw it.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Embedder, LayerCache, PartEnv, StateNeed, StepContext, WeightDecl, register_part


def sinusoid_table(rows: int, width: int, base: float = 10000.0) -> torch.Tensor:
    """float32 [rows, width]; the angles are formed in 64-bit and rounded once."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    freq = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / width)
    angle = torch.arange(rows, dtype=torch.float64)[:, None] * freq[None, :]
    table = torch.stack((angle.sin(), angle.cos()), dim=-1).reshape(rows, -1)[:, :width]
    return table.to(torch.float32).contiguous()


@register_part("embedding", "table_sum")
class TableSumEmbedding(Embedder):
    def __init__(self, vocab_size: int, hidden_size: int, weight_name: str, scale: float = 1.0,
                 pair_weight_name: Optional[str] = None, pair_buckets: int = 0, pair_mul_prev: int = 0,
                 pair_mul_cur: int = 0, sinusoid_base: Optional[float] = None):
        self.vocab_size, self.hidden_size, self.weight_name = vocab_size, hidden_size, weight_name
        self.scale = float(scale)
        self.pair_weight_name = pair_weight_name
        self.pair_buckets, self.pair_mul_prev, self.pair_mul_cur = int(pair_buckets), int(pair_mul_prev), int(pair_mul_cur)
        if pair_weight_name is not None and self.pair_buckets < 1:
            raise ValueError("a hashed pair table needs at least one bucket")
        self.sinusoid_base = None if sinusoid_base is None else float(sinusoid_base)
        self.table = self.pair_table = self.position_table = None

    def cache_need(self):
        # the id before the step's first token: read and rewritten on the device, so a step can be captured
        return StateNeed((1,), torch.int32, graph_safe=True) if self.pair_weight_name is not None else None

    def weights(self) -> List[WeightDecl]:
        out = [WeightDecl(self.weight_name, (self.vocab_size, self.hidden_size))]
        if self.pair_weight_name is not None:
            out.append(WeightDecl(self.pair_weight_name, (self.pair_buckets + 1, self.hidden_size)))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.table = tensors[self.weight_name].contiguous()
        if self.pair_weight_name is not None:
            self.pair_table = tensors[self.pair_weight_name].contiguous()
        if self.sinusoid_base is not None:
            rows, width, base = env.context_len, self.hidden_size, self.sinusoid_base
            self.position_table = env.shared(("sinusoid", rows, width, base),
                                             lambda: sinusoid_table(rows, width, base).to(env.device))

    def forward(self, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        return ops.embedding_sum(ctx.token_ids, self.table, self.scale, self.pair_table, self.pair_mul_prev,
                                 self.pair_mul_cur, self.position_table, ctx.positions, ctx.token_entry, ctx.q_start,
                                 ctx.entry_slot, cache.state if self.pair_table is not None else None)
