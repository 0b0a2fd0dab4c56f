"""RMSNorm with the residual sum fused in front of it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from .base import DeferredNorm, Norm, StreamPart
from .registry import register_part
from .spec import ParamSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight, in float32 (pico_vllm/RMSNorm.py:22-31)."""
    graph_safe_prompts = True

    def __init__(self, size: int, eps: float, act_dtype: torch.dtype = torch.bfloat16, weight_name: str = "weight"):
        # weight_name: the gain's name behind the part's prefix; "" where the prefix itself names the tensor
        self.size, self.eps, self.act_dtype, self.weight_name = size, eps, act_dtype, weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.weight_name, (self.size,), role="norm")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.weight = tensors[self.weight_name].to(device=device, dtype=torch.float32).contiguous()

    def add_norm(self, resid, delta, rows=None):
        return kernels.add_rmsnorm(resid, delta, self.weight, self.eps, self.act_dtype, rows)

    def add_norm_pair(self, other: "RMSNorm", resid, delta):
        """(this norm, ``other``) of resid + delta in one launch where the two differ in their weights only; else None."""
        if not isinstance(other, RMSNorm) or (other.size, other.eps, other.act_dtype) != (self.size, self.eps, self.act_dtype):
            return None
        return kernels.add_rmsnorm2(resid, delta, self.weight, other.weight, self.eps, self.act_dtype)

    def deferred(self, resid, delta):
        # the one row of a bfloat16 step: the projection behind the norm can norm it itself
        if (self.act_dtype == torch.bfloat16 and resid.shape[0] <= kernels.SKINNY_NORM_ROWS
                and (delta is None or delta.dtype == torch.float32)):
            return DeferredNorm(self, resid, delta, "rms", self.weight, self.eps)
        return None


@register_part("norm", "layer_norm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * weight + bias, var the mean squared deviation, in float32.  The sum in front
    of it may be scaled element by element: ``add_norm(resid, delta, delta_scale=s)`` norms resid + s * delta."""
    graph_safe_prompts = True
    takes_delta_scale = True

    def __init__(self, size: int, eps: float, act_dtype: torch.dtype = torch.bfloat16, weight_name: str = "weight",
                 bias_name: str = "bias"):
        self.size, self.eps, self.act_dtype = size, eps, act_dtype
        self.weight_name, self.bias_name = weight_name, bias_name
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.weight_name, (self.size,), role="norm"), ParamSpec(self.bias_name, (self.size,), role="f32")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.weight = tensors[self.weight_name].to(device=device, dtype=torch.float32).contiguous()
        self.bias = tensors[self.bias_name].to(device=device, dtype=torch.float32).contiguous()

    def add_norm(self, resid, delta, rows=None, delta_scale=None):
        if delta is not None and delta.dim() == 3 and delta.shape[0] > kernels.LN_MAX_SLABS:
            raise ValueError(f"a layer norm's launch adds at most {kernels.LN_MAX_SLABS} partial sums")
        return kernels.add_layernorm(resid, delta, self.weight, self.bias, self.eps, self.act_dtype, rows, delta_scale)


# what a step's parts share: the residual stream's rows in the activations' dtype, made by whoever wrote the stream last
# (a sublayer that reads the stream itself, not a norm of it, takes them from here): (the stream tensor, its copy)
STREAM_COPY = "stream_copy"


def stream_rows(resid: torch.Tensor, ctx, act_dtype: torch.dtype) -> torch.Tensor:
    """The residual stream in the activations' dtype: the stream itself in the 32-bit engine, else the copy that the
    kernel which last wrote the stream left, or a fresh one."""
    if act_dtype == torch.float32:
        return resid
    have = ctx.shared.get(STREAM_COPY)
    if have is not None and have[0] is resid:
        return have[1]
    return kernels.cast_rows(resid, act_dtype)


@register_part("stream", "stream_rms_norm")
class StreamRMSNorm(StreamPart):
    """x <- x / sqrt(mean(x^2) + eps) * weight on the residual stream itself, in float32 (a norm of the embeddings in
    front of the first layer).  Leaves the rows in the activations' dtype for the first sublayer that reads the stream."""
    graph_safe_prompts = True

    def __init__(self, size: int, eps: float, act_dtype: torch.dtype = torch.bfloat16, weight_name: str = "weight"):
        self.size, self.eps, self.act_dtype, self.weight_name = size, eps, act_dtype, weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.weight_name, (self.size,), role="norm")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.weight = tensors[self.weight_name].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, resid, ctx):
        copy = kernels.stream_rmsnorm(resid, self.weight, self.eps, None if self.act_dtype == torch.float32 else self.act_dtype)
        if copy is not None:
            ctx.shared[STREAM_COPY] = (resid, copy)
        return resid
