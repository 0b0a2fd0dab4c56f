"""Differential attention: two softmax attentions a head over the same values, one subtracted from the other."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, PageTensor, ParamSpec


@register_part("mixer", "differential_attention")
class DifferentialAttention(Mixer):
    """q = x Wq^T (heads x 2 x dk: every head holds two maps [map 1 | map 2]), k = x Wk^T (kv heads x 2 x dk),
    v = x Wv^T (kv heads x dv); no biases, no rotation.  Every (head, map) of q and k is RMS-normed over its dk entries
    with one weight [dk] for all of q and one for all of k.  Per map m of head h, over kv head g = h // (H / G):

      s_ij = (q_i^m . k_j^m) scale temp(i),  temp(i) = 1 + temp_coef ln(floor((i + 1) / temp_every) + 1)   (temp_every 0: 1)
      a^m  = softmax over keys j <= i of s, times v

    and o = a^1 - lambda a^2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number a layer, made at load),
    then o over its root mean square (eps inside, no weight) times (1 - diff); the heads side by side go through Wo.

    The attention kernels see 2 H query heads over 2 G kv heads of keys (one a (group, map)) and G heads of values (a
    value head serves both maps); the queries are laid out (group, map, head in group) for that.  The maps' outputs stay
    float32 until they are combined.  Scores, softmax, norms and the combination are float32 in both engines."""

    graph_safe_prompts = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
             "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 diff: float, norm_eps: float, temp_coef: float = 0.0, temp_every: int = 0,
                 names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if not (1 <= key_dim <= 1024 and 1 <= value_dim <= 256):
            raise ValueError(f"key size {key_dim} (1 to 1024) or value size {value_dim} (1 to 256) outside what the kernels take")
        self.hidden_size, self.heads, self.kv_heads, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, key_dim, value_dim
        self.scale, self.diff, self.norm_eps = float(scale), float(diff), float(norm_eps)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        # what the attention kernels see (ops.attention_bias_fast.choose reads these)
        self.nq, self.nkv, self.v_div, self.out_f32, self.window, self.slope_span = 2 * num_heads, 2 * num_kv_heads, 2, True, 0, 0.0
        self.k_col = self.nq * key_dim
        self.v_col = self.k_col + self.nkv * key_dim
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.q_norm = self.k_norm = None
        self.lam = 0.0
        self.fast = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", page_tensors=(PageTensor("k", (self.nkv, "page", self.dk)),
                                                   PageTensor("v", (self.kv_heads, self.dv, "page"))))

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + 2.0 * self.nq * (self.dk + self.dv) * pairs

    def param_specs(self) -> List[ParamSpec]:
        D, n = self.hidden_size, self.names
        out = [ParamSpec(n["q"], (self.nq * self.dk, D)), ParamSpec(n["k"], (self.nkv * self.dk, D)),
               ParamSpec(n["v"], (self.kv_heads * self.dv, D)), ParamSpec(n["o"], (D, self.heads * self.dv)),
               ParamSpec(n["q_norm"], (self.dk,), role="norm"), ParamSpec(n["k_norm"], (self.dk,), role="norm")]
        return out + [ParamSpec(n[x], (self.dk,), role="f32", std=0.1) for x in ("lq1", "lk1", "lq2", "lk2")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in "qkv"]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.qkv = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.o = Linear(tensors[n["o"]].to(device))
        self.q_norm = tensors[n["q_norm"]].to(device=device, dtype=torch.float32).contiguous()
        self.k_norm = tensors[n["k_norm"]].to(device=device, dtype=torch.float32).contiguous()
        dot = lambda a, b: float((tensors[n[a]].double() * tensors[n[b]].double()).sum())
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff
        if self.act_dtype == torch.bfloat16:
            from ..ops import attention_bias_fast
            self.fast = attention_bias_fast.choose(self)

    def graph_variant(self, ctx: StepContext) -> tuple:
        own = (("differential_attention",) + self.fast.plan(ctx),) if self.fast is not None else ()
        return own + super().graph_variant(ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.attend(x, ctx, cache))

    def attend(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The combined heads' outputs [T, H dv] in front of the output projection."""
        bt = ctx.block_tables[cache.group]
        y = self.qkv(x)                                    # [T, 2 H dk | 2 G dk | G dv]
        q = kernels.qk_norm_store(y, 0, self.k_col, self.v_col, self.nq, self.nkv, self.kv_heads, self.dk, self.dv, 2,
                                  kernels.QK_NORM_UNIT, self.q_norm, self.k_norm, self.norm_eps, None, 0,
                                  ctx.slot_mapping[cache.group], cache.k, cache.v)
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            a = self.fast(q, cache, bt, ctx)
        else:
            a = kernels.attn_bias_plain(q, cache.k, cache.v, bt, ctx.positions, ctx.token_seq, self.nq, self.nkv, self.dk,
                                        self.dv, self.scale, temp_coef=self.temp_coef, temp_every=self.temp_every,
                                        v_div=2, out_f32=True)
        return kernels.diff_combine(a, self.lam, self.norm_eps, 1.0 - self.diff, self.heads, self.kv_heads, self.dv, self.act_dtype)
