"""Attention whose queries, keys and values come out of low-rank latents; the cache keeps the latent, not the heads."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .rotary import RotaryPairs
from .spec import CacheSpec, PageTensor, ParamSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """With x a token's normed activations, H heads, per head d unrotated and r rotated query/key entries:

      cq = rmsnorm(Wdq x) wq,                q_h = Wuq cq                      (laid out head by head as [d | r])
      [c' | kr] = Wdkv x,  c = rmsnorm(c') wkv                                 (c: ``kv_rank`` entries; kr: r entries)
      k_h = [Wuk_h c | rot(kr)],  v_h = Wuv_h c,  q_h <- [q_h[:d] | rot(q_h[d:])]
      score_ij = (q_i . k_j) scale, causal softmax, heads side by side, Wo

    rot turns neighbouring pairs of the r entries by position * f (``parts.rotary.scaled_frequencies``); the unrotated
    part has no position.  The cache keeps per token [c | rot(kr)] and nothing per head: since
    q_h[:d] . (Wuk_h c) = (Wuk_h^T q_h[:d]) . c, a head's query is carried into the latent's space
    (q'_h = [Wuk_h^T q_h[:d] | rot(q_h[d:])], ``kv_rank + r`` entries), attention runs with ONE key/value head whose key
    is [c | rot(kr)] and whose value is c, and a head's output (in the latent's space) goes through Wuv_h afterwards.
    That is attention with keys of kv_rank + r and values of kv_rank entries, which this package's attention kernels
    serve (the value pages are laid out [dv, page], so c is stored a second time as the value column).
    Norms, angles, scores and softmax are float32.  ``names``: the tensors' names behind the part's prefix."""

    graph_safe_prompts = True

    NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}
    # steps of more bfloat16 rows than this make the products a head through the library (batched); fewer, and every
    # 32-bit step, through this package's kernel, in which a row does not depend on the rows beside it
    LIBRARY_FROM = 65

    def __init__(self, hidden_size: int, num_heads: int, dim: int, rot_dim: int, value_dim: int, q_rank: int, kv_rank: int,
                 scale: float, base: float, scaling=None, norm_eps: float = 1e-5, names: Optional[Dict[str, str]] = None,
                 act_dtype: torch.dtype = torch.bfloat16):
        if rot_dim % 2 or rot_dim < 0 or dim < 1 or value_dim < 1 or num_heads < 1 or q_rank < 1 or kv_rank < 1:
            raise ValueError("latent attention: sizes must be positive and the rotated part even")
        if kv_rank + rot_dim > 1024 or kv_rank > 512:
            raise ValueError(f"latent of {kv_rank} + {rot_dim} rotated entries outside what the attention kernels take (512, 1024 together)")
        self.hidden_size, self.heads, self.d, self.r, self.dv = hidden_size, num_heads, dim, rot_dim, value_dim
        self.q_rank, self.kv_rank, self.scale, self.norm_eps = q_rank, kv_rank, float(scale), float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.position = RotaryPairs(rot_dim, base, scaling, act_dtype=act_dtype) if rot_dim else None
        # as the attention kernels of this package call these: one kv head, no window, no penalty, no temperature
        self.nq, self.nkv, self.dk, self.window = num_heads, 1, kv_rank + rot_dim, 0
        self.temp_coef, self.temp_every, self.slope_span = 0.0, 0, 0.0
        self.down: Optional[Linear] = None        # rows [dq | dkv]
        self.uq: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.uk_t: Optional[torch.Tensor] = None  # [H, d, kv_rank]: head h's key matrix, inner index first
        self.uv_t: Optional[torch.Tensor] = None  # [H, kv_rank, dv]
        self.wq = self.wkv = None
        self.fast = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", page_tensors=(PageTensor("k", (1, "page", self.kv_rank + self.r)),
                                                   PageTensor("v", (1, self.kv_rank, "page"))))

    def flops(self, tokens: int, pairs: int) -> float:
        H = self.heads
        per_head = 2.0 * tokens * H * self.kv_rank * (self.d + self.dv)
        return super().flops(tokens, pairs) + per_head + 2.0 * H * (self.dk + self.kv_rank) * pairs

    def weight_bytes(self) -> int:
        return super().weight_bytes() + sum(t.numel() * t.element_size() for t in (self.uk_t, self.uv_t))

    def param_specs(self) -> List[ParamSpec]:
        D, n, H = self.hidden_size, self.names, self.heads
        return [ParamSpec(n["dq"], (self.q_rank, D)), ParamSpec(n["dq_norm"], (self.q_rank,), role="norm"),
                ParamSpec(n["uq"], (H * (self.d + self.r), self.q_rank)),
                ParamSpec(n["dkv"], (self.kv_rank + self.r, D)), ParamSpec(n["dkv_norm"], (self.kv_rank,), role="norm"),
                ParamSpec(n["uk"], (H * self.d, self.kv_rank)), ParamSpec(n["uv"], (H * self.dv, self.kv_rank)),
                ParamSpec(n["o"], (D, H * self.dv))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n, H = self.names, self.heads
        ws = [tensors[n["dq"]], tensors[n["dkv"]]]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.down = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.uq = Linear(tensors[n["uq"]].to(device))
        self.o = Linear(tensors[n["o"]].to(device))
        self.uk_t = tensors[n["uk"]].to(device).view(H, self.d, self.kv_rank).contiguous()
        self.uv_t = tensors[n["uv"]].to(device).view(H, self.dv, self.kv_rank).transpose(1, 2).contiguous()
        self.wq = tensors[n["dq_norm"]].to(device=device, dtype=torch.float32).contiguous()
        self.wkv = tensors[n["dkv_norm"]].to(device=device, dtype=torch.float32).contiguous()
        if self.position is not None:
            self.position.load({}, device, dtype)
        if self.act_dtype == torch.bfloat16 and self.uk_t.dtype == torch.bfloat16:
            from ..ops import attention_bias_fast
            # (the matrix-core kernel reads query rows in 16-byte pieces)
            if attention_bias_fast.supported(self.dk, self.kv_rank) and (self.heads * self.dk) % 8 == 0:
                self.fast = attention_bias_fast.FastBiasAttention(self.nq, 1, self.dk, self.kv_rank, self.scale)

    def graph_variant(self, ctx: StepContext) -> tuple:
        return (("latent_attention",) + self.fast.plan(ctx),) if self.fast is not None else ()

    def _per_head(self, x: torch.Tensor, x_head: int, w: torch.Tensor, copy: int = 0, turn=None) -> torch.Tensor:
        """out[t, h] = [x[t, h, :in] @ w[h] | x[t, h, in : in + copy]]; x [T, H * x_head].  ``turn``: the table of the
        angles by which the copied part is turned on the way (this package's kernel does it in its launch)."""
        T, H = x.shape[0], self.heads
        if x.dtype == torch.bfloat16 and T >= self.LIBRARY_FROM:
            if turn is not None:
                kernels.rope_inplace(x, w.shape[1], H, x_head, copy, turn, halves=False)
            # The library's batched product on operands laid out batch by batch ([H, T, in] and [H, T, out], both made
            # here), and never under the library's tuner: handed the rows' own layout (a head's matrix interleaved
            # with the other heads', the batch stride smaller than the row stride) the tuner's copies of the operands
            # are sized for batch-major ones and it reads beyond them.
            from ..ops.linear import no_library_tuning
            n_in, n_out = w.shape[1], w.shape[2]
            xv = x.view(T, H, x_head)
            out = torch.empty(T, H, n_out + copy, dtype=x.dtype, device=x.device)
            with no_library_tuning():
                res = torch.bmm(xv[:, :, :n_in].transpose(0, 1).contiguous(), w)          # [H, T, out]
            out[:, :, :n_out] = res.transpose(0, 1)
            if copy:
                out[:, :, n_out:] = xv[:, :, n_in:n_in + copy]
            return out.view(T, H * (n_out + copy))
        return kernels.head_linear(x, 0, x_head, w, H, copy=copy, turn=turn)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.attend(x, ctx, cache))

    def attend(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The heads' outputs [T, H dv] in front of the output projection."""
        H, d, r = self.heads, self.d, self.r
        table = self.position.table(ctx) if self.position is not None else None
        y = self.down(x)                                         # [T, query latent | key/value latent | rotated key part]
        cq = kernels.latent_prepare(y, self.q_rank, self.kv_rank, r, self.wq, self.wkv, self.norm_eps, table,
                                    ctx.slot_mapping[cache.group], cache.k, cache.v)
        q = self.uq(cq)                                          # [T, H (d + r)]
        # the queries in the latent's space, their rotated part turned on the way: [T, H (kv_rank + r)]
        ql = self._per_head(q, d + r, self.uk_t, copy=r, turn=table if r else None)
        bt = ctx.block_tables[cache.group]
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            ol = self.fast(ql, cache, bt, ctx)
        else:
            ol = kernels.attn_bias_plain(ql, cache.k, cache.v, bt, ctx.positions, ctx.token_seq, H, 1, self.dk, self.kv_rank,
                                         self.scale, 0)
        return self._per_head(ol, self.kv_rank, self.uv_t)       # [T, H dv]
