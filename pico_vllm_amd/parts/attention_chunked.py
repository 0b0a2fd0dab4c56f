"""Chunked attention with a sink in the softmax, whose values are its keys as projected."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .attention_bias import kv_page_tensors
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, ParamSpec


@register_part("mixer", "chunked_sink_attention")
class ChunkedSinkAttention(Mixer):
    """q = x Wq^T + bq (heads x d), k = x Wk^T + bk (kv heads x d); there is no value matrix: v = k as projected.
    q and k are RMS-normed over their WHOLE rows (all heads at once) with weights of the rows' sizes, then the first
    ``rotary_dim`` entries of every head are turned (entry i with entry i + rotary_dim / 2, by position base^(-2i / rotary_dim)).

      s_ij = (q_i . k_j) scale;  key j <= i is seen iff floor(i / chunk) == floor(j / chunk)   (chunk 0: every j <= i)
      p_ij = exp(s_ij) / (1 + sum_j exp(s_ij))                                                  (a sink of score 0, no value)

    Head h's output is multiplied by sigmoid(x Wg^T)_h, one number a head, and the heads side by side go through Wo.
    One product makes q, k and the gate.  Chunks are counted from position 0 of the request; the cache gives the pages
    of earlier chunks back.  Norms, angles, scores and softmax are float32 in both engines."""

    graph_safe_prompts = True

    NAMES = {"q": "q", "k": "k", "g": "g", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "q_norm": "q.norm", "k_norm": "k.norm"}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, scale: float, norm_eps: float,
                 chunk: int = 0, rotary_dim: int = 0, base: float = 10000.0, proj_bias: bool = True,
                 names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if not 1 <= dim <= 256:
            raise ValueError(f"head size {dim} outside what the kernels take (1 to 256: the values are the keys)")
        if chunk < 0 or rotary_dim < 0 or rotary_dim % 2 or rotary_dim > dim:
            raise ValueError(f"chunk {chunk} must not be negative; {rotary_dim} turned entries must be even and fit a head of {dim}")
        self.hidden_size, self.nq, self.nkv, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, dim, dim
        self.scale, self.norm_eps, self.chunk, self.rotary_dim, self.base = float(scale), float(norm_eps), int(chunk), int(rotary_dim), float(base)
        self.proj_bias = proj_bias
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        # what the attention kernels see (ops.attention_bias_fast.choose reads these)
        self.window, self.temp_coef, self.temp_every, self.slope_span = 0, 0.0, 0, 0.0
        self.sink, self.gated, self.gate_heads = True, True, True
        self.k_col = self.nq * dim
        self.g_col = self.k_col + self.nkv * dim
        self.proj: Optional[Linear] = None               # rows [q | k | g]
        self.o: Optional[Linear] = None
        self.q_norm = self.k_norm = self.inv_freq = None
        self.fast = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", chunk=self.chunk, page_tensors=kv_page_tensors(self.nkv, self.dk, self.dv))

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + 2.0 * self.nq * (self.dk + self.dv) * pairs

    def param_specs(self) -> List[ParamSpec]:
        D, n = self.hidden_size, self.names
        nqd, nkd = self.nq * self.dk, self.nkv * self.dk
        out = [ParamSpec(n["q"], (nqd, D)), ParamSpec(n["k"], (nkd, D)), ParamSpec(n["g"], (self.nq, D)),
               ParamSpec(n["o"], (D, self.nq * self.dv)),
               ParamSpec(n["q_norm"], (nqd,), role="norm"), ParamSpec(n["k_norm"], (nkd,), role="norm")]
        if self.proj_bias:
            out += [ParamSpec(n["q_bias"], (nqd,), role="bias"), ParamSpec(n["k_bias"], (nkd,), role="bias")]
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in "qkg"]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        b = None
        if self.proj_bias:
            qb, kb = tensors[n["q_bias"]].float(), tensors[n["k_bias"]].float()
            b = torch.cat([qb, kb, torch.zeros(self.nq, device=qb.device)], dim=0).to(device)      # the gate has no bias
        self.proj = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device), b)
        self.o = Linear(tensors[n["o"]].to(device))
        self.q_norm = tensors[n["q_norm"]].to(device=device, dtype=torch.float32).contiguous()
        self.k_norm = tensors[n["k_norm"]].to(device=device, dtype=torch.float32).contiguous()
        if self.rotary_dim:
            half = self.rotary_dim // 2
            f = torch.tensor([self.base ** (-2.0 * i / self.rotary_dim) for i in range(half)], dtype=torch.float64)
            self.inv_freq = f.to(device=device, dtype=torch.float32).contiguous()
        if self.act_dtype == torch.bfloat16:
            from ..ops import attention_bias_fast
            self.fast = attention_bias_fast.choose(self)

    def graph_variant(self, ctx: StepContext) -> tuple:
        own = (("chunked_sink_attention",) + self.fast.plan(ctx),) if self.fast is not None else ()
        return own + super().graph_variant(ctx)

    def _angles(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """cos and sin of the step's positions, once a step for all layers that turn alike."""
        if not self.rotary_dim:
            return None
        key = ("rotate_half_table", self.rotary_dim, self.base)
        if key not in ctx.shared:
            ctx.shared[key] = kernels.rope_table(ctx.positions[:ctx.num_tokens], self.inv_freq)
        return ctx.shared[key]

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.attend(x, ctx, cache))

    def attend(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The gated heads' outputs [T, H d] in front of the output projection."""
        bt = ctx.block_tables[cache.group]
        y = self.proj(x)                                   # [T, H d | G d | H]
        q = kernels.qk_norm_store(y, 0, self.k_col, self.k_col, self.nq, self.nkv, self.nkv, self.dk, self.dv, 1,
                                  kernels.QK_NORM_ROW, self.q_norm, self.k_norm, self.norm_eps, self._angles(ctx),
                                  self.rotary_dim, ctx.slot_mapping[cache.group], cache.k, cache.v)
        gate = y[:, self.g_col:]
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            return self.fast(q, cache, bt, ctx, gate=gate)
        return kernels.attn_bias_plain(q, cache.k, cache.v, bt, ctx.positions, ctx.token_seq, self.nq, self.nkv, self.dk,
                                       self.dv, self.scale, gate=gate, chunk=self.chunk, sink=True, gate_heads=True)
