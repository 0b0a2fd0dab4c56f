"""The matrix-core kernel of the attention with a distance penalty, and when it serves."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library
from . import attention_fast
from .attention_fast import compute_units
from .kernels import KernelError, _check, _check_cache2, _ptr, _stream

c_float = ctypes.c_float
MAX_CHUNKS = 32
PROMPT_KERNEL_FROM = 64      # tokens of a step from which the prompt kernel serves it (a tile of its workgroups)


def supported(key_dim: int, value_dim: int) -> bool:
    """Key sizes in steps of 32 up to 512 and value sizes in steps of 16 up to 256; anything else goes to the plain kernel."""
    return key_dim % 32 == 0 and 32 <= key_dim <= 512 and value_dim % 16 == 0 and 16 <= value_dim <= 256


class FastBiasAttention:
    def __init__(self, nq: int, nkv: int, key_dim: int, value_dim: int, scale: float, window: int = 0,
                 temp_coef: float = 0.0, temp_every: int = 0, slope_span: float = 0.0, softcap: float = 0.0,
                 keep_first: int = 0, gated: bool = False, chunk: int = 0, sink: bool = False, gate_heads: bool = False,
                 v_div: int = 1, out_f32: bool = False):
        self.nq, self.nkv, self.dk, self.dv = nq, nkv, key_dim, value_dim
        self.scale, self.window, self.temp_coef, self.temp_every, self.slope_span = scale, window, temp_coef, temp_every, slope_span
        self.softcap, self.keep_first, self.gated = float(softcap), int(keep_first), bool(gated)
        # chunked visibility instead of a window, a sink in the softmax, a gate of one number a head, several kv heads
        # over one head of values, float32 output (see csrc/attention_bias.hip)
        self.chunk, self.sink, self.gate_heads, self.v_div, self.out_f32 = int(chunk), bool(sink), bool(gate_heads), int(v_div), bool(out_f32)
        self.lib = library.attention_bias_library(key_dim, value_dim)
        if self.lib.pico_attnb_key_dim() != key_dim or self.lib.pico_attnb_value_dim() != value_dim:
            raise KernelError("attention library was built for other sizes")
        self.cus = compute_units()
        # keys and values of one size in steps of 32: prompt steps go through the rotary attention's prompt kernel (keys
        # staged in LDS for 64 or 128 queries), which takes the columns' factors and the penalty into its scores
        self.tuned = None
        # (that kernel knows no cap on the scores, no kept first positions and no gate)
        if key_dim == value_dim and key_dim % 32 == 0 and attention_fast.supported(nq, nkv, key_dim, window) \
                and not (self.softcap > 0 or (self.keep_first > 0 and window > 0) or self.gated or self.chunk or self.sink
                         or self.v_div != 1 or self.out_f32):
            self.tuned = attention_fast.FastAttention(nq, nkv, key_dim, window)

    def split(self, num_tokens: int) -> bool:
        """Whether the four waves of a workgroup share ONE block of 16 query columns (few blocks: the chip is filled
        by cutting their keys) or take a block each.  Decided from the number of tokens of the step alone."""
        R = self.nq // self.nkv
        blocks = -(-num_tokens // max(1, 16 // R)) * -(-R // 16) * self.nkv
        return blocks < 8 * self.cus

    def chunks(self, num_tokens: int, num_seqs: int) -> int:
        """Into how many pieces every block's keys are cut, each piece a workgroup of its own (their parts are put
        together by a second launch): as many as bring the step to two workgroups a compute unit, at most MAX_CHUNKS.
        Decided from the step's size alone; a piece is a whole number of 128 keys, found on the device from the block's
        own range of keys."""
        if not self.split(num_tokens):
            return 1
        R = self.nq // self.nkv
        blocks = (-(-num_tokens // max(1, 16 // R)) + num_seqs) * -(-R // 16) * self.nkv
        return max(1, min(MAX_CHUNKS, -(-2 * self.cus // blocks)))

    def prompt_shape(self, ctx) -> int:
        """The shape of the prompt kernel's workgroups for this step (0: that kernel does not serve it)."""
        if self.tuned is None or ctx.num_tokens < PROMPT_KERNEL_FROM:
            return 0
        key = ("bias_attention_shape", self.nq, self.nkv, self.dk, self.window)
        if key not in ctx.shared:
            shape = 1
            if "cu_seqlens" in ctx.host and "context_lens" in ctx.host:
                B = ctx.num_seqs
                cu = ctx.host["cu_seqlens"]
                real = B - int(ctx.host.get("filler", 0))         # the filler behind a recorded portion does not count
                shape = int(self.tuned.prefill_teams((cu[1:B + 1] - cu[:B])[:real], ctx.host["context_lens"][:real]))
            ctx.shared[key] = shape
        return ctx.shared[key]

    def plan(self, ctx) -> tuple:
        return (bool(self.split(ctx.num_tokens)), self.chunks(ctx.num_tokens, ctx.num_seqs), self.prompt_shape(ctx))

    def run(self, q: torch.Tensor, k_cache, v_cache, block_table, cu_seqlens, positions, num_seqs: int,
            split: Optional[bool] = None, out: Optional[torch.Tensor] = None, chunks: Optional[int] = None,
            gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [T, >= nq * dk] bfloat16 (row stride free); any mixture of portions and single tokens; returns [T, nq * dv].
        ``gate`` [T, >= nq * dv] bfloat16 (8-byte aligned rows): the output is multiplied with sigmoid(gate)."""
        T = q.shape[0]
        pages, P = _check_cache2(k_cache, v_cache, self.nkv, self.dk, self.dv, self.nkv // self.v_div)
        if not q.is_cuda or q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16:
            raise KernelError("matrix-core attention wants bfloat16 tensors on the GPU")
        if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < self.nq * self.dk or (T > 1 and q.stride(0) % 8) or q.data_ptr() % 16:
            raise KernelError("q must be [T, >= nq*dk] with unit stride along the row and 16-byte aligned rows")
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous() \
                or block_table.shape[0] < num_seqs:
            raise KernelError("block_table must be contiguous int32 [sequences, pages]")
        for t, n in ((cu_seqlens, num_seqs + 1), (positions, T)):
            if t.dtype != torch.int32 or t.numel() < n or not t.is_contiguous():
                raise KernelError("sequence metadata must be contiguous int32")
        if P < 8 or P & (P - 1):
            raise KernelError("matrix-core attention wants pages of a power of two of at least 8 tokens")
        if gate is not None and (not gate.is_cuda or gate.dtype != torch.bfloat16 or gate.dim() != 2 or gate.shape[0] != T
                                 or gate.stride(1) != 1 or gate.shape[1] < (self.nq if self.gate_heads else self.nq * self.dv)
                                 or (not self.gate_heads and ((T > 1 and gate.stride(0) % 4) or gate.data_ptr() % 8))):
            raise KernelError("the gate must be bfloat16 [T, >= nq*dv] with unit stride along the row and 8-byte aligned rows")
        if out is None:
            out = torch.empty(T, self.nq * self.dv, dtype=torch.float32 if self.out_f32 else torch.bfloat16, device=q.device)
        if split is None:
            split = self.split(T)
        if chunks is None:
            chunks = self.chunks(T, num_seqs) if split else 1
        parts_o = parts_ml = None
        if chunks > 1:
            if not split:
                raise KernelError("pieces of the keys go with one block a workgroup")
            parts_o = torch.empty(chunks, T * self.nq, self.dv, dtype=torch.float32, device=q.device)
            parts_ml = torch.empty(chunks, T * self.nq, 2, dtype=torch.float32, device=q.device)
        _check(self.lib, self.lib.pico_attnb(
            _ptr(q), q.stride(0) if T > 1 else q.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
            _ptr(cu_seqlens), _ptr(positions), num_seqs, T, _ptr(out), self.nq, self.nkv, self.dk, self.dv, P, pages,
            c_float(self.scale), self.window, c_float(self.temp_coef), self.temp_every, c_float(self.slope_span),
            1 if split else 0, chunks, _ptr(parts_o), _ptr(parts_ml), c_float(self.softcap), self.keep_first, _ptr(gate),
            0 if gate is None else (gate.stride(0) if T > 1 else gate.shape[1]), self.chunk, 1 if self.sink else 0,
            1 if self.gate_heads else 0, self.v_div, 1 if self.out_f32 else 0, _stream()))
        return out

    def __call__(self, qkv, cache, block_table, ctx, gate=None):
        split, chunks, shape = self.plan(ctx)
        if shape and cache.k.numel() * cache.k.element_size() < (1 << 32):
            B = ctx.num_seqs
            order, build = None, False
            if B >= 2:      # several sequences: the list of their query tiles, longest first, written by the first layer
                key = ("bias_attention_order", self.dk, shape)
                order, build = ctx.shared.get(key), key not in ctx.shared
                if build:
                    order = ctx.shared[key] = self.tuned.order_list(qkv.shape[0], B, qkv.device)
            return self.tuned.prefill(qkv, cache.k, cache.v, block_table, ctx.cu_seqlens, ctx.context_lens, B, self.scale,
                                      teams=shape, order=order, order_build=build,
                                      scored=(self.temp_coef, self.temp_every, self.slope_span))
        return self.run(qkv, cache.k, cache.v, block_table, ctx.cu_seqlens, ctx.positions, ctx.num_seqs,
                        split=split, chunks=chunks, gate=gate)


def choose(mixer) -> Optional[FastBiasAttention]:
    """The matrix-core kernel for this mixer's sizes, or None where the plain kernel serves."""
    if not supported(mixer.dk, mixer.dv):
        return None
    return FastBiasAttention(mixer.nq, mixer.nkv, mixer.dk, mixer.dv, mixer.scale, mixer.window, mixer.temp_coef,
                             mixer.temp_every, mixer.slope_span, getattr(mixer, "softcap", 0.0),
                             getattr(mixer, "keep_first", 0), getattr(mixer, "gated", False), getattr(mixer, "chunk", 0),
                             getattr(mixer, "sink", False), getattr(mixer, "gate_heads", False), getattr(mixer, "v_div", 1),
                             getattr(mixer, "out_f32", False))
