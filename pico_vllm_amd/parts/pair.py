"""Two mixers side by side that read the same input."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .base import Mixer, StepContext
from .registry import build_part, register_part
from .spec import CacheSpec, ParamSpec, PartSpec


@register_part("mixer", "mixer_pair")
class MixerPair(Mixer):
    """out = (rms(left(h)) * w_left + rms(right(h)) * w_right) / 2: two mixers of any kinds, each with the cache or state
    it asks for, their outputs RMS-normed over the model width with a weight each before they are averaged.  The pair
    hands both outputs and weights to an arrangement that norms and sums them in one launch (``forward_pair``; the
    arrangement "postnorm" does).  ``left`` / ``right``: the two mixers as PartSpecs; their tensors stand behind
    ``prefixes``; ``out_names``: the two weights."""

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, left: PartSpec, right: PartSpec, norm_eps: float, prefixes=("left", "right"),
                 out_names=("left.out", "right.out"), act_dtype: torch.dtype = torch.bfloat16):
        self.hidden_size, self.norm_eps = hidden_size, float(norm_eps)
        self.prefixes, self.out_names = tuple(prefixes), tuple(out_names)
        self.left = build_part("mixer", left, act_dtype=act_dtype)
        self.right = build_part("mixer", right, act_dtype=act_dtype)
        self.act_dtype = act_dtype
        self.w_left: Optional[torch.Tensor] = None
        self.w_right: Optional[torch.Tensor] = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("several", parts=(self.left.cache_spec(), self.right.cache_spec()))

    def param_specs(self) -> List[ParamSpec]:
        out = []
        for pre, part in zip(self.prefixes, (self.left, self.right)):
            out += [ParamSpec(f"{pre}.{p.name}", p.shape, p.role, p.std) for p in part.param_specs()]
        return out + [ParamSpec(n, (self.hidden_size,), role="norm") for n in self.out_names]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        for pre, part in zip(self.prefixes, (self.left, self.right)):
            part.load({p.name: tensors[f"{pre}.{p.name}"] for p in part.param_specs()}, device, dtype)
        self.w_left, self.w_right = (tensors[n].to(device=device, dtype=torch.float32).contiguous() for n in self.out_names)

    def forward_pair(self, x: torch.Tensor, ctx: StepContext, cache):
        """(left's output, its weight, right's output, its weight); the outputs as their output projections leave them
        ([T, H], or float32 stacks of partial sums)."""
        left_cache, right_cache = cache
        return self.left.forward(x, ctx, left_cache), self.w_left, self.right.forward(x, ctx, right_cache), self.w_right

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        raise NotImplementedError("a pair of mixers runs in an arrangement that norms and sums its two outputs (forward_pair)")
