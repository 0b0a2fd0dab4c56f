"""Learned absolute positions on the residual stream."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from .base import StepContext, StreamPart
from .registry import register_part
from .spec import ParamSpec


@register_part("stream", "learned_positions")
class LearnedPositions(StreamPart):
    """resid[t] += table[position of t], in float32; the table has one row per position a request can reach
    (``max_positions``), and a step that would read beyond it is refused where the engine is built
    (``ModelSpec.max_position``)."""
    graph_safe_prompts = True

    def __init__(self, size: int, max_positions: int, name: str = "weight", act_dtype: torch.dtype = torch.bfloat16):
        self.size, self.max_positions, self.name = size, max_positions, name
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.name, (self.max_positions, self.size))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.table = tensors[self.name].to(device).contiguous()

    def weight_bytes(self) -> int:
        return 0                     # a step reads one row a token, not the table

    def forward(self, resid: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return kernels.add_rows(resid, self.table, ctx.positions[:ctx.num_tokens])


@register_part("stream", "pair_embedding")
class PairEmbedding(StreamPart):
    """resid[t] += table[(previous token * mul_prev + token * mul_cur) mod buckets]; a sequence's first token has no
    previous one and takes the table's last row (row ``buckets``).  The previous token of a portion's first token is
    the last token of the step before: it is part of the request's state (one int32 a state slot, written at the end
    of every step on the device, so a step may start before the host knows the token that the step before sampled)."""
    graph_safe_prompts = True

    def __init__(self, size: int, buckets: int, mul_prev: int, mul_cur: int, name: str = "weight",
                 act_dtype: torch.dtype = torch.bfloat16):
        if buckets < 1:
            raise ValueError("the table of pairs needs at least one bucket")
        self.size, self.buckets, self.mul_prev, self.mul_cur, self.name = size, int(buckets), int(mul_prev), int(mul_cur), name
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        from .spec import CacheSpec
        return CacheSpec("state", state_shape=(1,), state_dtype="int32")

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.name, (self.buckets + 1, self.size))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.table = tensors[self.name].to(device).contiguous()

    def weight_bytes(self) -> int:
        return 0                     # a step reads one row a token, not the table

    def forward(self, resid: torch.Tensor, ctx: StepContext, cache=None) -> torch.Tensor:
        return kernels.pair_embed(resid, self.table, ctx, cache.state.view(-1), self.mul_prev, self.mul_cur, self.buckets)
