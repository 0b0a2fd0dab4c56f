"""A selective state-space mixer: a short causal convolution and a recurrence with token-dependent step sizes."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, ParamSpec


@register_part("mixer", "selective_state_space")
class SelectiveStateSpace(Mixer):
    """[u | z] = Win x (``inner`` channels each); u <- silu(conv(u) + b) with a causal convolution of ``taps`` taps a
    channel; [d | B | C] = Wx u (``dt_rank`` | ``state`` | ``state``); dt = softplus(Wdt d + bdt) a channel;
    A = -exp(A_log) [inner, state].  Per channel c and state element n:

      S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c u_c B_n,      y_c = sum_n S[c, n] C_n + D_c u_c

    and the output is Wo (y * silu(z)).  A request's state (float32, zero for a new request) is S and the last
    taps - 1 inputs of the convolution, together [inner, state + taps - 1] in its state slot.  Step sizes, decays, the
    recurrence and its state are float32 in both engines; the sums run in an order that depends on the sizes alone,
    so a token's output does not depend on how its sequence was cut into steps."""

    graph_safe_prompts = True

    # In the bfloat16 engine a step with a prompt portion cuts its sequences into chunks of this many tokens that run
    # side by side (``kernels.selective_scan``); decided from the step's shape alone.  The 32-bit engine walks every
    # sequence whole, so that its sums do not depend on how a prompt was cut.
    CHUNK, CHUNKED_FROM = 64, 128

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b", "a_log": "A_log",
             "d": "D", "o": "o"}

    def __init__(self, hidden_size: int, inner: int, state: int, taps: int, dt_rank: int,
                 names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if not (1 <= taps <= kernels.SSM_MAX_TAPS and 1 <= state <= kernels.SSM_MAX_STATE and inner >= 1 and dt_rank >= 1):
            raise ValueError(f"selective state space: 1 to {kernels.SSM_MAX_TAPS} taps and 1 to {kernels.SSM_MAX_STATE} state "
                             f"elements a channel, got {taps} and {state}")
        self.hidden_size, self.inner, self.state, self.taps, self.dt_rank = hidden_size, inner, state, taps, dt_rank
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.in_proj: Optional[Linear] = None
        self.x_proj: Optional[Linear] = None
        self.dt_proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("state", state_shape=(self.inner, self.state + self.taps - 1), state_dtype="float32")

    def flops(self, tokens: int, pairs: int) -> float:
        # the products, the convolution, and per token, channel and state element the update and the read
        return super().flops(tokens, pairs) + tokens * self.inner * (2.0 * self.taps + 6.0 * self.state)

    def param_specs(self) -> List[ParamSpec]:
        D, n, I, N, R = self.hidden_size, self.names, self.inner, self.state, self.dt_rank
        return [ParamSpec(n["in"], (2 * I, D)), ParamSpec(n["conv"], (I, self.taps), role="f32"),
                ParamSpec(n["conv_bias"], (I,), role="f32"), ParamSpec(n["x"], (R + 2 * N, I)), ParamSpec(n["dt"], (I, R)),
                ParamSpec(n["dt_bias"], (I,), role="f32"), ParamSpec(n["a_log"], (I, N), role="f32"),
                ParamSpec(n["d"], (I,), role="f32"), ParamSpec(n["o"], (D, I))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        self.in_proj, self.x_proj = Linear(tensors[n["in"]].to(device)), Linear(tensors[n["x"]].to(device))
        self.dt_proj, self.o = Linear(tensors[n["dt"]].to(device)), Linear(tensors[n["o"]].to(device))
        f32 = lambda k: tensors[n[k]].to(device=device, dtype=torch.float32).contiguous()
        self.conv_w = f32("conv").t().contiguous()          # tap by tap, [taps, inner]: neighbouring channels side by side
        self.conv_b, self.dt_bias, self.a_log, self.d = f32("conv_bias"), f32("dt_bias"), f32("a_log"), f32("d")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.mix(x, ctx, cache))

    def mix(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """y * silu(z) [T, inner] in front of the output projection."""
        I, N, R = self.inner, self.state, self.dt_rank
        uz = self.in_proj(x)                                                         # [T, u | z]
        u = kernels.causal_conv(uz, I, self.conv_w, self.conv_b, ctx, cache.state, N, single=ctx.all_decode)
        dbc = self.x_proj(u)                                                         # [T, d | B | C]
        dt_pre = self.dt_proj(dbc[:, :R], out_dtype=torch.float32)                   # step sizes stay float32 from here on
        chunked = self.act_dtype == torch.bfloat16 and not ctx.all_decode and ctx.num_tokens >= self.CHUNKED_FROM
        return kernels.selective_scan(u, dt_pre, self.dt_bias, dbc, R, R + N, self.a_log, self.d, uz[:, I:], ctx, cache.state,
                                      self.taps - 1, chunk=self.CHUNK if chunked else 0)
