"""Recurrent mixers with a matrix state per head that a walk over the tokens updates: the gated delta rule, and the
state-space (duality) layer, which is the same walk without the delta rule's correction."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, ParamSpec


# In the bfloat16 engine a step with a prompt portion cuts its sequences into chunks of this many tokens that run side by
# side (``kernels.delta_scan``); decided from the step's shape alone.  The 32-bit engine walks every sequence whole, so
# that its sums do not depend on how a prompt was cut.
# (With the delta rule a chunk's map of the state is a full matrix, and the walk over the chunks, one product a chunk, is
# a chain of as many steps as a sequence has chunks; longer chunks shorten it and take as much from the two passes.)
CHUNK, CHUNK_DELTA, CHUNKED_FROM = 64, 64, 128


def _chunk(act_dtype: torch.dtype, ctx: StepContext, delta: bool = False) -> int:
    if act_dtype != torch.bfloat16 or ctx.all_decode or ctx.num_tokens < CHUNKED_FROM:
        return 0
    return CHUNK_DELTA if delta else CHUNK


def _conv_state(channels: int, taps: int) -> CacheSpec:
    """The last taps - 1 inputs of a short causal convolution, per channel."""
    return CacheSpec("state", state_shape=(channels, taps - 1), state_dtype="float32")


@register_part("mixer", "gated_delta_rule")
class GatedDeltaRule(Mixer):
    """q = x Wq^T, k = x Wk^T (qk_heads x dk), v = x Wv^T (heads x dv), no biases; head h reads q/k head
    h // (heads / qk_heads).  Each of q, k, v passes a causal convolution of ``taps`` taps a channel (no bias, zeros
    before a request's start) and silu; q and k then become unit vectors per head, x / sqrt(sum x^2 + 1e-6), q also times
    dk^(-1/2).  beta = sigmoid(x Wb^T) a head; a decay per head and key channel

      g = exp(-exp(A_log_h) softplus((x Wa1^T) Wa2^T + dt_bias))                  (heads x dk)

    Per head, token by token:  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
    Every head's o is RMS-normed over dv with one weight [dv], times sigmoid((x Wg1^T) Wg2^T) (heads x dv), then Wo.

    A request keeps S (float32 [heads, dk, dv], zero at its start) and the convolution's last taps - 1 inputs.  Unit norms,
    beta, decays, the walk and the head norm are float32 in both engines; the walk's sums run in an order that depends on
    the sizes alone.  One product makes q, k, v, beta's logits and the two low-rank activations."""

    graph_safe_prompts = True

    NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b",
             "a_log": "A_log", "norm": "norm", "a1": "a1", "a2": "a2", "dt_bias": "dt_bias", "g1": "g1", "g2": "g2", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, num_qk_heads: int, key_dim: int, value_dim: int, taps: int,
                 decay_rank: int, gate_rank: int, norm_eps: float, names: Optional[Dict[str, str]] = None,
                 act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_qk_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_qk_heads} query/key heads")
        if not (1 <= key_dim <= kernels.DELTA_MAX_KEY_DIM and value_dim >= 1 and 1 <= taps <= kernels.SSM_MAX_TAPS):
            raise ValueError(f"key size 1 to {kernels.DELTA_MAX_KEY_DIM} and 1 to {kernels.SSM_MAX_TAPS} taps, got {key_dim} and {taps}")
        if decay_rank < 1 or gate_rank < 1:
            raise ValueError("the low-rank projections have at least one dimension")
        self.hidden_size, self.heads, self.qk_heads, self.dk, self.dv, self.taps = hidden_size, num_heads, num_qk_heads, key_dim, value_dim, taps
        self.decay_rank, self.gate_rank, self.norm_eps = int(decay_rank), int(gate_rank), float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        qk, hv = num_qk_heads * key_dim, num_heads * value_dim
        self.channels = 2 * qk + hv                       # what the convolution runs over: [q | k | v]
        self.k_col, self.v_col = qk, 2 * qk
        self.b_col = self.channels
        self.a_col = self.b_col + num_heads
        self.g_col = self.a_col + self.decay_rank
        self.proj: Optional[Linear] = None                # rows [q | k | v | b | a1 | g1]
        self.g2: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.conv_w = self.a2 = self.dt_bias = self.a_log = self.norm_weight = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("several", parts=(CacheSpec("state", state_shape=(self.heads, self.dk, self.dv), state_dtype="float32"),
                                           _conv_state(self.channels, self.taps)))

    def flops(self, tokens: int, pairs: int) -> float:
        # the products, the convolution, the low-rank decay, and per token and head the state's decay, read, write and read
        return super().flops(tokens, pairs) + tokens * (2.0 * self.taps * self.channels
                                                        + self.heads * self.dk * (2.0 * self.decay_rank + 7.0 * self.dv))

    def param_specs(self) -> List[ParamSpec]:
        D, n = self.hidden_size, self.names
        qk, hv = self.qk_heads * self.dk, self.heads * self.dv
        return [ParamSpec(n["q"], (qk, D)), ParamSpec(n["k"], (qk, D)), ParamSpec(n["v"], (hv, D)),
                ParamSpec(n["q_conv"], (qk, self.taps), role="f32", std=0.3), ParamSpec(n["k_conv"], (qk, self.taps), role="f32", std=0.3),
                ParamSpec(n["v_conv"], (hv, self.taps), role="f32", std=0.3), ParamSpec(n["b"], (self.heads, D)),
                ParamSpec(n["a_log"], (self.heads,), role="f32", std=0.5), ParamSpec(n["norm"], (self.dv,), role="norm"),
                ParamSpec(n["a1"], (self.decay_rank, D)), ParamSpec(n["a2"], (self.heads * self.dk, self.decay_rank)),
                ParamSpec(n["dt_bias"], (self.heads * self.dk,), role="f32", std=0.5),
                ParamSpec(n["g1"], (self.gate_rank, D)), ParamSpec(n["g2"], (hv, self.gate_rank)), ParamSpec(n["o"], (D, hv))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in ("q", "k", "v", "b", "a1", "g1")]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.g2, self.o = Linear(tensors[n["g2"]].to(wdt).to(device)), Linear(tensors[n["o"]].to(device))
        self.a2 = tensors[n["a2"]].to(device=device, dtype=wdt).contiguous()
        f32 = lambda t: t.to(device=device, dtype=torch.float32).contiguous()
        # tap by tap, [taps, channels]: neighbouring channels side by side
        self.conv_w = f32(torch.cat([tensors[n[x]].float() for x in ("q_conv", "k_conv", "v_conv")], dim=0).t())
        self.dt_bias, self.a_log, self.norm_weight = f32(tensors[n["dt_bias"]]), f32(tensors[n["a_log"]]), f32(tensors[n["norm"]])

    def weight_bytes(self) -> int:
        return super().weight_bytes() + self.a2.numel() * self.a2.element_size()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.mix(x, ctx, cache))

    def mix(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The normed and gated heads' outputs [T, H dv] in front of the output projection."""
        state, hist = cache
        y = self.proj(x)                                   # [T, q | k | v | b | a1 | g1]
        xc = kernels.causal_conv(y, self.channels, self.conv_w, None, ctx, hist.state, 0, single=ctx.all_decode)
        qn, kn, g, beta = kernels.delta_prep(xc, 0, self.k_col, y, self.b_col, self.a_col, self.a2, self.dt_bias, self.a_log,
                                             self.dk ** -0.5, self.heads, self.qk_heads, self.dk)
        o = kernels.delta_scan(qn, kn, xc[:, self.v_col:], g, beta, ctx.cu_seqlens, ctx.state_slots, state.state, ctx.num_seqs,
                               self.heads, self.qk_heads, self.dk, self.dv, delta=True, chunk=_chunk(self.act_dtype, ctx, delta=True))
        gate = self.g2(y[:, self.g_col:self.g_col + self.gate_rank])
        return kernels.gla_out(o, gate, 0, self.norm_weight, self.norm_eps, self.heads, self.dv, sigmoid_gate=True)


@register_part("mixer", "state_space_duality")
class StateSpaceDuality(Mixer):
    """[z | x | B | C | dt] = x Win^T with inner = heads x dv entries for z and for x, groups x N for B and for C, one dt a
    head.  x, B and C together pass a causal convolution of ``taps`` taps a channel with bias, then silu;
    dt <- softplus(dt + dt_bias).  Per head h (reading B and C of group h // (heads / groups)), token by token:

      S <- exp(-exp(A_log_h) dt) S + dt B x^T        (S is N x dv)
      y  = S^T C + D_h x

    The heads side by side times silu(z), RMS-normed in ``norm_groups`` equal parts of the row (each by its own root
    mean square), times a weight [inner], then Wo.  A request keeps S (float32 [heads, N, dv], zero at its start) and the
    convolution's last taps - 1 inputs.  Step sizes, decays, the walk and the norm are float32 in both engines."""

    graph_safe_prompts = True

    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D", "norm": "norm", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state: int, groups: int, norm_groups: int, taps: int,
                 norm_eps: float, names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % groups or (num_heads * value_dim) % norm_groups:
            raise ValueError(f"{num_heads} heads are not a multiple of {groups} groups, or {num_heads * value_dim} entries no "
                             f"multiple of {norm_groups} parts")
        if not (1 <= state <= kernels.DELTA_MAX_KEY_DIM and value_dim >= 1 and 1 <= taps <= kernels.SSM_MAX_TAPS):
            raise ValueError(f"1 to {kernels.DELTA_MAX_KEY_DIM} state elements and 1 to {kernels.SSM_MAX_TAPS} taps, got {state} and {taps}")
        self.hidden_size, self.heads, self.dv, self.n, self.groups = hidden_size, num_heads, value_dim, state, groups
        self.norm_groups, self.taps, self.norm_eps = norm_groups, taps, float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.inner = num_heads * value_dim
        self.channels = self.inner + 2 * groups * state   # what the convolution runs over: [x | B | C]
        self.dt_col = self.inner + self.channels
        self.in_proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d = self.norm_weight = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("several", parts=(CacheSpec("state", state_shape=(self.heads, self.n, self.dv), state_dtype="float32"),
                                           _conv_state(self.channels, self.taps)))

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + tokens * (2.0 * self.taps * self.channels + 5.0 * self.heads * self.n * self.dv)

    def param_specs(self) -> List[ParamSpec]:
        D, n = self.hidden_size, self.names
        return [ParamSpec(n["in"], (self.dt_col + self.heads, D)), ParamSpec(n["conv"], (self.channels, self.taps), role="f32", std=0.3),
                ParamSpec(n["conv_bias"], (self.channels,), role="f32"), ParamSpec(n["dt_bias"], (self.heads,), role="f32", std=0.5),
                ParamSpec(n["a_log"], (self.heads,), role="f32", std=0.5), ParamSpec(n["d"], (self.heads,), role="f32", std=0.5),
                ParamSpec(n["norm"], (self.inner,), role="norm"), ParamSpec(n["o"], (D, self.inner))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        self.in_proj, self.o = Linear(tensors[n["in"]].to(device)), Linear(tensors[n["o"]].to(device))
        f32 = lambda k: tensors[n[k]].to(device=device, dtype=torch.float32).contiguous()
        self.conv_w = f32("conv").t().contiguous()          # tap by tap, [taps, channels]
        self.conv_b, self.dt_bias, self.a_log, self.d, self.norm_weight = f32("conv_bias"), f32("dt_bias"), f32("a_log"), f32("d"), f32("norm")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.mix(x, ctx, cache))

    def mix(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The gated and normed heads' outputs [T, inner] in front of the output projection."""
        state, hist = cache
        gn = self.groups * self.n
        y = self.in_proj(x)                                 # [T, z | x | B | C | dt]
        xbc = kernels.causal_conv(y[:, self.inner:], self.channels, self.conv_w, self.conv_b, ctx, hist.state, 0, single=ctx.all_decode)
        bf, cf, g, dt = kernels.ssd_prep(xbc, self.inner, self.inner + gn, gn, y, self.dt_col, self.dt_bias, self.a_log, self.heads)
        o = kernels.delta_scan(cf, bf, xbc, g, dt, ctx.cu_seqlens, ctx.state_slots, state.state, ctx.num_seqs, self.heads,
                               self.groups, self.n, self.dv, delta=False, chunk=_chunk(self.act_dtype, ctx))
        return kernels.gated_group_norm(o, xbc, y, self.d, self.norm_weight, self.norm_eps, self.heads, self.dv, self.norm_groups)
