"""A routed feed-forward: every token runs a few of many small gated feed-forwards."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import FeedForward, StepContext
from .registry import register_part
from .spec import ParamSpec

# the gate's activation is g sigmoid(ACT_ALPHA g)
ACT_ALPHA = 1.702


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """Router: z = x Wr^T in float32, scores s = sigmoid(z); a token's ``top`` experts are those with the largest
    scores, its weights their scores as they are (not renormalised).

    Expert e on a row r: g = min(Wg_e r, limit), u = clamp(Wu_e r, -limit, limit), y = g sigmoid(alpha g) (u + 1),
    out = Wd_e y; no biases.  The weight scales the expert's INPUT: a token's output is sum_e expert_e(s_e x).

    The checkpoint holds every expert's three matrices apart (``expert_names`` with the expert's number filled in); they
    are stacked at load: gate_up [E, 2 F, D], down [E, D, F].  Everything a step decides (which experts, which rows) is
    decided on the device."""
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, limit: float,
                 act_alpha: float = ACT_ALPHA, router_name: str = "router",
                 expert_names: tuple = ("e{}.gate", "e{}.up", "e{}.down"), act_dtype: torch.dtype = torch.bfloat16):
        if not 1 <= top <= min(num_experts, kernels.MOE_MAX_TOP):
            raise ValueError(f"{top} experts per token of {num_experts} (at most {kernels.MOE_MAX_TOP})")
        if not limit > 0:
            raise ValueError(f"the experts' limit must be positive, got {limit}")
        self.hidden_size, self.expert_size, self.num_experts, self.top = hidden_size, expert_size, num_experts, top
        self.limit, self.act_alpha = float(limit), float(act_alpha)
        self.router_name, self.expert_names = router_name, tuple(expert_names)
        self.act_dtype = act_dtype
        self.router: Optional[Linear] = None
        self.gate_up: Optional[Linear] = None       # [E * 2 F, D]: as a matrix, so that reports count its bytes
        self.down: Optional[Linear] = None          # [E * D, F]

    def param_specs(self) -> List[ParamSpec]:
        D, F = self.hidden_size, self.expert_size
        g, u, d = self.expert_names
        out = [ParamSpec(self.router_name, (self.num_experts, D))]
        for e in range(self.num_experts):
            out += [ParamSpec(g.format(e), (F, D)), ParamSpec(u.format(e), (F, D)), ParamSpec(d.format(e), (D, F))]
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        g, u, d = self.expert_names
        E = self.num_experts
        self.router = Linear(tensors[self.router_name].float().to(device))      # routed in float32 in both engines
        ws = [tensors[n.format(e)] for e in range(E) for n in (g, u)]
        wdt = torch.float32 if dtype == torch.float32 or any(w.dtype == torch.float32 for w in ws) else torch.bfloat16
        self.gate_up = Linear(torch.cat([w.to(wdt) for w in ws], dim=0).to(device))
        self.down = Linear(torch.cat([tensors[d.format(e)].to(wdt) for e in range(E)], dim=0).to(device))

    def weight_bytes(self) -> int:
        # what a step of one token streams: the router and ``top`` experts
        per = (self.gate_up.weight.numel() + self.down.weight.numel()) * self.gate_up.weight.element_size() // self.num_experts
        return self.router.weight.numel() * 4 + self.top * per

    def flops(self, tokens: int, pairs: int) -> float:
        D, F = self.hidden_size, self.expert_size
        return 2.0 * tokens * (self.num_experts * D + self.top * 3 * F * D)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        E, F, D = self.num_experts, self.expert_size, self.hidden_size
        experts, weights = kernels.moe_router(x, self.router.weight, self.top)
        gate_up = self.gate_up.weight.view(E, 2 * F, D)
        down = self.down.weight.view(E, D, F)
        if x.dtype != gate_up.dtype:
            x = x.to(gate_up.dtype)
        if kernels.moe_fast_ok(x, gate_up, down):
            # few rows stream their experts' matrices; many are sorted by expert and go to the matrix cores.  The
            # second gives one float32 slab a slot: the next norm adds them up
            return kernels.moe_experts(x, gate_up, down, experts, weights, self.limit, self.act_alpha)
        return kernels.moe_experts_plain(x, gate_up, down, experts, weights, self.limit, self.act_alpha)

    def graph_variant(self, ctx: StepContext) -> tuple:
        return (("routed_experts", kernels.moe_grouped_rows(ctx.num_tokens, self.top)),)


@register_part("feed_forward", "softmax_routed_experts")
class SoftmaxRoutedExperts(FeedForward):
    """Router: z = x Wr^T in float32 over ``num_experts + identity`` outputs, scores s = softmax(z) over all of them.
    The ``top`` outputs with the largest s + correction are chosen (the correction, a stored vector, only steers the
    choice); the weights are the chosen s over their sum (+ 1e-20), times ``scale``.

    Expert e < num_experts on a token x: Wd_e (silu(Wg_e x) * (Wu_e x)), no biases; the last ``identity`` router outputs
    stand for experts without tensors that return x itself.  A token's output is the weighted sum of its experts'
    outputs.  With ``shared_size`` > 0 one more gated feed-forward of that inner size runs for every token and is added.

    The experts' matrices are stacked at load (gate_up [E, 2 F, D], down [E, D, F]); everything a step decides is
    decided on the device.  ``forward`` returns the routed sum, or [routed sum, shared expert's output] (deltas that the
    arrangement adds to the residual stream one after the other)."""
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, identity: int = 0, scale: float = 1.0,
                 shared_size: int = 0, correction_name: Optional[str] = "correction", router_name: str = "router",
                 expert_names: tuple = ("e{}.gate", "e{}.up", "e{}.down"),
                 shared_names: tuple = ("shared.gate", "shared.up", "shared.down"), act_dtype: torch.dtype = torch.bfloat16):
        if num_experts < 1 or identity < 0 or not 1 <= top <= min(num_experts + identity, kernels.MOE_MAX_TOP):
            raise ValueError(f"{top} experts per token of {num_experts} + {identity} (at most {kernels.MOE_MAX_TOP})")
        self.hidden_size, self.expert_size, self.num_experts, self.top = hidden_size, expert_size, num_experts, top
        self.identity, self.scale, self.shared_size = int(identity), float(scale), int(shared_size)
        self.correction_name, self.router_name = correction_name, router_name
        self.expert_names, self.shared_names = tuple(expert_names), tuple(shared_names)
        self.act_dtype = act_dtype
        self.router: Optional[Linear] = None
        self.correction: Optional[torch.Tensor] = None
        self.gate_up: Optional[Linear] = None       # [E * 2 F, D]
        self.down: Optional[Linear] = None          # [E * D, F]
        self.shared = None
        if self.shared_size:
            from .mlp import SwiGLUMLP
            self.shared = SwiGLUMLP(hidden_size, self.shared_size, act_dtype=act_dtype, names=self.shared_names)

    @property
    def outputs(self) -> int:
        return self.num_experts + self.identity

    def param_specs(self) -> List[ParamSpec]:
        D, F = self.hidden_size, self.expert_size
        g, u, d = self.expert_names
        out = []
        for e in range(self.num_experts):
            out += [ParamSpec(g.format(e), (F, D)), ParamSpec(u.format(e), (F, D)), ParamSpec(d.format(e), (D, F))]
        out.append(ParamSpec(self.router_name, (self.outputs, D)))
        if self.correction_name:
            out.append(ParamSpec(self.correction_name, (self.outputs,), role="bias"))
        if self.shared is not None:
            out += self.shared.param_specs()
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        g, u, d = self.expert_names
        E = self.num_experts
        self.router = Linear(tensors[self.router_name].float().to(device))      # routed in float32 in both engines
        if self.correction_name:
            self.correction = tensors[self.correction_name].to(device=device, dtype=torch.float32).contiguous()
        ws = [tensors[n.format(e)] for e in range(E) for n in (g, u)]
        wdt = torch.float32 if dtype == torch.float32 or any(w.dtype == torch.float32 for w in ws) else torch.bfloat16
        self.gate_up = Linear(torch.cat([w.to(wdt) for w in ws], dim=0).to(device))
        self.down = Linear(torch.cat([tensors[d.format(e)].to(wdt) for e in range(E)], dim=0).to(device))
        if self.shared is not None:
            self.shared.load({n: tensors[n] for n in self.shared_names}, device, dtype)

    def weight_bytes(self) -> int:
        # what a step of one token streams: the router, ``top`` experts and the shared expert
        per = (self.gate_up.weight.numel() + self.down.weight.numel()) * self.gate_up.weight.element_size() // self.num_experts
        return self.router.weight.numel() * 4 + self.top * per + (self.shared.weight_bytes() if self.shared is not None else 0)

    def flops(self, tokens: int, pairs: int) -> float:
        D, F = self.hidden_size, self.expert_size
        return 2.0 * tokens * (self.outputs * D + self.top * 3 * F * D) + (self.shared.flops(tokens, pairs) if self.shared is not None else 0.0)

    def forward(self, x: torch.Tensor, ctx: StepContext):
        out = self._routed(x)
        if self.shared is None:
            return out
        return [self.shared.forward(x, ctx), out]

    def forward_into(self, x: torch.Tensor, ctx: StepContext, resid: torch.Tensor):
        """The shared expert's second product adds into the float32 stream ``resid`` itself (its epilogue in a small
        step); the routed sum is returned, for the next norm's launch to add."""
        if self.shared is not None:
            self.shared.down.add_into(self.shared.gate_up.swiglu(x), resid)
        return self._routed(x)

    def _routed(self, x: torch.Tensor) -> torch.Tensor:
        E, F, D = self.num_experts, self.expert_size, self.hidden_size
        experts, weights = kernels.moe_router_softmax(x, self.router.weight, self.correction, self.top, self.scale)
        gate_up = self.gate_up.weight.view(E, 2 * F, D)
        down = self.down.weight.view(E, D, F)
        xe = x if x.dtype == gate_up.dtype else x.to(gate_up.dtype)
        if kernels.moe_fast_ok(xe, gate_up, down):
            out = kernels.moe_experts(xe, gate_up, down, experts, weights, 0.0, 0.0, mode=kernels.MOE_SWIGLU)
        else:
            out = kernels.moe_experts_plain(xe, gate_up, down, experts, weights, 0.0, 0.0, mode=kernels.MOE_SWIGLU)
        if self.identity:
            kernels.moe_identity(xe, experts, weights, out, E)
        return out

    def graph_variant(self, ctx: StepContext) -> tuple:
        return (("softmax_routed_experts", kernels.moe_grouped_rows(ctx.num_tokens, self.top)),)


@register_part("feed_forward", "top_softmax_routed_experts")
class TopSoftmaxRoutedExperts(SoftmaxRoutedExperts):
    """Router: z = x Wr^T + b in float32; the ``top`` experts with the largest logits are chosen (the lowest index among
    equals), and their weights are the softmax over the chosen logits only.  Experts as in ``SoftmaxRoutedExperts``
    (Wd_e (silu(Wg_e x) * (Wu_e x)), the weight on the output).  With ``shared_size`` > 0 one more gated feed-forward
    runs for every token; with ``shared_gate_name`` its output is multiplied by sigmoid(wsg . x), one number a token
    (the gate's row rides behind the router's rows: one launch makes the experts' logits and the gate's).

    ``forward_scaled_into(x, ctx, resid, scale)`` adds scale * (routed sum + gated shared output) to the float32 stream
    in the one launch that puts the pieces together."""

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, shared_size: int = 0,
                 router_name: str = "router", router_bias_name: Optional[str] = "router.b",
                 shared_gate_name: Optional[str] = "shared.sg", expert_names: tuple = ("e{}.gate", "e{}.up", "e{}.down"),
                 shared_names: tuple = ("shared.gate", "shared.up", "shared.down"), act_dtype: torch.dtype = torch.bfloat16):
        super().__init__(hidden_size, expert_size, num_experts, top, identity=0, scale=1.0, shared_size=shared_size,
                         correction_name=None, router_name=router_name, expert_names=expert_names, shared_names=shared_names,
                         act_dtype=act_dtype)
        self.router_bias_name = router_bias_name
        self.shared_gate_name = shared_gate_name if shared_size else None
        self.router_bias: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        out = super().param_specs()
        if self.router_bias_name:
            out.append(ParamSpec(self.router_bias_name, (self.num_experts,), role="f32"))
        if self.shared_gate_name:
            out.append(ParamSpec(self.shared_gate_name, (1, self.hidden_size)))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        super().load(tensors, device, dtype)
        if self.shared_gate_name:       # the gate's row behind the experts' rows, float32 like them
            self.router = Linear(torch.cat([self.router.weight, tensors[self.shared_gate_name].float().to(device)], dim=0))
        if self.router_bias_name:
            self.router_bias = tensors[self.router_bias_name].to(device=device, dtype=torch.float32).contiguous()

    def _pieces(self, x: torch.Tensor, ctx: StepContext):
        """(routed sum, shared expert's output or None, its gate's logits or None)."""
        E, F, D = self.num_experts, self.expert_size, self.hidden_size
        experts, weights, z = kernels.moe_router_top_softmax(x, self.router.weight, self.router_bias, E, self.top)
        gate_up = self.gate_up.weight.view(E, 2 * F, D)
        down = self.down.weight.view(E, D, F)
        xe = x if x.dtype == gate_up.dtype else x.to(gate_up.dtype)
        if kernels.moe_fast_ok(xe, gate_up, down):
            routed = kernels.moe_experts(xe, gate_up, down, experts, weights, 0.0, 0.0, mode=kernels.MOE_SWIGLU)
        else:
            routed = kernels.moe_experts_plain(xe, gate_up, down, experts, weights, 0.0, 0.0, mode=kernels.MOE_SWIGLU)
        if self.shared is None:
            return routed, None, None
        shared = self.shared.down(self.shared.gate_up.swiglu(x))          # [T, D], one piece: the gate multiplies it
        return routed, shared, (z[:, E:] if self.shared_gate_name else None)

    def forward_scaled_into(self, x: torch.Tensor, ctx: StepContext, resid: torch.Tensor, scale: Optional[torch.Tensor]) -> None:
        routed, shared, gate = self._pieces(x, ctx)
        kernels.scaled_add(resid, routed, shared, gate, scale)

    def forward(self, x: torch.Tensor, ctx: StepContext):
        routed, shared, gate = self._pieces(x, ctx)
        out = torch.zeros(x.shape[0], self.hidden_size, dtype=torch.float32, device=x.device)
        kernels.scaled_add(out, routed, shared, gate, None)
        return out

    forward_into = None        # the parent's way of adding the shared expert knows no gate
