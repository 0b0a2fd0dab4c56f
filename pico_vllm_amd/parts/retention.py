"""Retention: linear attention with one fixed decay a head, no softmax and no denominator."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .gla import GatedLinearAttention
from .registry import register_part
from .rotary import RotaryPairs
from .spec import CacheSpec, ParamSpec


@register_part("mixer", "retention")
class Retention(Mixer):
    """q = Wq x, k = Wk x (heads x dk), v = Wv x, g = Wg x (heads x dv), one product.  The first ``rotary_dim`` entries
    of every q and k head are turned by position * f_i, entry i with entry i + rotary_dim / 2; k is scaled by dk^(-1/2).
    Per head, with the head's constant decay gamma_h:

      S_t = gamma_h S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t

    Every head's o is divided by its root mean square (no weight), the heads side by side are multiplied by silu(g),
    and the output matrix follows.  The state [heads, dk, dv] is float32, zero for a new request, and lives in the
    request's state slot.  The recurrence is the one of ``parts.gla`` with a constant in place of the token's decays
    (``kernels.gla_scan(head_decay=...)``: the constant is multiplied in as it is); the scale on k is applied to the
    read-out instead, which is the same sum.  Decays, recurrence, state and head norm are float32 in both engines."""

    graph_safe_prompts = True
    CHUNK, CHUNKED_FROM = GatedLinearAttention.CHUNK, GatedLinearAttention.CHUNKED_FROM

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay: Sequence[float], norm_eps: float,
                 rotary_dim: int = 0, base: float = 10000.0, scaling=None, names: Optional[Dict[str, str]] = None,
                 act_dtype: torch.dtype = torch.bfloat16):
        if not 1 <= key_dim <= kernels.GLA_MAX_KEY_DIM:
            raise ValueError(f"key size {key_dim} outside what the recurrence kernel takes (1 to {kernels.GLA_MAX_KEY_DIM})")
        if len(decay) != num_heads or not all(0.0 < float(g) <= 1.0 for g in decay):
            raise ValueError(f"retention: one decay in (0, 1] a head, got {len(decay)} for {num_heads} heads")
        if rotary_dim % 2 or not 0 <= rotary_dim <= key_dim:
            raise ValueError(f"{rotary_dim} rotated entries do not fit a head of {key_dim}")
        self.hidden_size, self.heads, self.dk, self.dv = hidden_size, num_heads, key_dim, value_dim
        self.decay_values, self.norm_eps, self.rotary_dim = tuple(float(g) for g in decay), float(norm_eps), int(rotary_dim)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.position = RotaryPairs(rotary_dim, base, scaling, act_dtype=act_dtype) if rotary_dim else None
        self.proj: Optional[Linear] = None               # rows [q | k | v | g]
        self.o: Optional[Linear] = None
        self.decay = self.ones = None
        hk, hv = num_heads * key_dim, num_heads * value_dim
        self.q_col, self.k_col, self.v_col, self.g_col = 0, hk, 2 * hk, 2 * hk + hv

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("state", state_shape=(self.heads, self.dk, self.dv), state_dtype="float32")

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + tokens * self.heads * self.dk * 5.0 * self.dv

    def param_specs(self) -> List[ParamSpec]:
        H, n = self.hidden_size, self.names
        hk, hv = self.heads * self.dk, self.heads * self.dv
        return [ParamSpec(n["q"], (hk, H)), ParamSpec(n["k"], (hk, H)), ParamSpec(n["v"], (hv, H)), ParamSpec(n["g"], (hv, H)),
                ParamSpec(n["o"], (H, hv))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in ("q", "k", "v", "g")]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.o = Linear(tensors[n["o"]].to(device))
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(device)
        self.ones = torch.ones(self.dv, dtype=torch.float32, device=device)
        if self.position is not None:
            self.position.load({}, device, dtype)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.mix(x, ctx, cache))

    def mix(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The normed and gated heads' outputs [T, H dv] in front of the output projection."""
        y = self.proj(x)                                   # [T, q | k | v | g]
        if self.position is not None:                      # q and k heads stand side by side: 2 H heads of dk entries
            kernels.rope_inplace(y, self.q_col, 2 * self.heads, self.dk, self.rotary_dim, self.position.table(ctx), halves=True)
        # the bfloat16 engine cuts long portions into chunks that run side by side (the same sums in another order);
        # the 32-bit engine walks every sequence whole
        chunked = self.act_dtype == torch.bfloat16 and not ctx.all_decode and ctx.num_tokens >= self.CHUNKED_FROM
        o = kernels.gla_scan(y, self.q_col, self.k_col, self.v_col, None, ctx.cu_seqlens, ctx.state_slots, cache.state,
                             ctx.num_seqs, self.heads, self.dk, self.dv, self.dk ** -0.5, chunk=self.CHUNK if chunked else 0,
                             head_decay=self.decay)
        return kernels.gla_out(o, y, self.g_col, self.ones, self.norm_eps, self.heads, self.dv)
