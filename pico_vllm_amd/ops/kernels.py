"""Python faces of the HIP kernels.

Every function checks on the host that shapes, dtypes and layouts are what the
kernel and its grid assume, then launches on torch's current stream.  Tensors
must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from . import library

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
c_int, c_float, c_void_p, c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


class KernelError(RuntimeError):
    pass


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not supported by the kernels (float32 or bfloat16)") from None


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("the kernels run on the GPU only; got a CPU tensor")


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr() if t is not None else 0)


_bound_stream = None


def _stream():
    if _bound_stream is not None:
        return _bound_stream
    return c_void_p(torch.cuda.current_stream().cuda_stream)


class stream_scope:
    """Look torch's current stream up once for all launches inside the scope (the lookup costs
    more than a launch).  The scope must not span a change of the current stream."""

    def __enter__(self):
        global _bound_stream
        self._outer = _bound_stream
        _bound_stream = c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _bound_stream
        _bound_stream = self._outer
        return False


def _check(lib, code: int) -> None:
    if code != 0:
        lib.pico_last_error.restype = ctypes.c_char_p
        raise KernelError(lib.pico_last_error().decode())


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} entries, {n} are needed")


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 rows (the residual stream)."""
    _gpu(table, ids)
    V, H = table.shape
    T = ids.numel()
    _i32(ids, "ids")
    if not table.is_contiguous():
        raise KernelError("embedding table must be contiguous")
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    elif out.shape != (T, H) or out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embedding: out must be a contiguous float32 [T, H] tensor")
    lib = library.core()
    _check(lib, lib.pico_embedding(_ptr(table), _dt(table), _ptr(ids), _ptr(out), T, H, V, c_float(scale), _stream()))
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap) in place, float32."""
    _gpu(x)
    if x.dtype != torch.float32 or not x.is_contiguous() or not cap > 0:
        raise KernelError("softcap: a contiguous float32 tensor and a positive cap")
    lib = library.core()
    _check(lib, lib.pico_softcap(_ptr(x), c_ll(x.numel()), c_float(cap), _stream()))
    return x


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """rows is None: resid += delta (if given), returns norm(resid).
    rows given: returns norm(resid[rows] + delta[rows]); resid is left alone.
    delta is [T, H], or a float32 stack [S, T, H] of partial sums that are all added."""
    _gpu(resid, delta, weight, rows)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"norm weight must be float32 of shape [{H}]")
    slabs = 1
    if delta is not None:
        if delta.dim() == 3:
            slabs = delta.shape[0]
            if delta.dtype != torch.float32:
                raise KernelError("a stack of partial sums must be float32")
        if tuple(delta.shape[-2:]) != (T, H) or not delta.is_contiguous():
            raise KernelError("delta must be contiguous and shaped like the residual stream")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    elif out.shape != (n, H) or out.dtype != out_dtype or not out.is_contiguous():
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    lib = library.core()
    ddt = _dt(delta) if delta is not None else F32
    _check(lib, lib.pico_add_rmsnorm(_ptr(resid), _ptr(delta), ddt, slabs, c_ll(T * H), _ptr(weight), _ptr(out),
                                     _DT[out_dtype], _ptr(rows), n, H, c_float(eps), _stream()))
    return out


MAX_SLABS = 8           # partial sums that one norm launch adds up


def add_rmsnorm2(resid: torch.Tensor, delta: Optional[torch.Tensor], weight1: torch.Tensor, weight2: torch.Tensor, eps: float,
                 out_dtype: torch.dtype):
    """resid += delta (if given; [T, H] or a float32 stack [S, T, H]), then the row's RMS norm with each of the two
    weights: (norm(resid) * weight1, norm(resid) * weight2), one launch."""
    _gpu(resid, delta, weight1, weight2)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    for w in (weight1, weight2):
        if w.dtype != torch.float32 or w.shape != (H,) or not w.is_contiguous():
            raise KernelError(f"norm weight must be float32 of shape [{H}]")
    slabs = 1
    if delta is not None:
        if delta.dim() == 3:
            slabs = delta.shape[0]
            if delta.dtype != torch.float32:
                raise KernelError("a stack of partial sums must be float32")
        if tuple(delta.shape[-2:]) != (T, H) or not delta.is_contiguous():
            raise KernelError("delta must be contiguous and shaped like the residual stream")
    out1 = torch.empty(T, H, dtype=out_dtype, device=resid.device)
    out2 = torch.empty(T, H, dtype=out_dtype, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_add_rmsnorm2(_ptr(resid), _ptr(delta), _dt(delta) if delta is not None else F32, slabs, c_ll(T * H),
                                      _ptr(weight1), _ptr(weight2), _ptr(out1), _ptr(out2), _DT[out_dtype], T, H, c_float(eps),
                                      _stream()))
    return out1, out2


def residual_add(resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _gpu(resid, delta)
    if resid.dtype != torch.float32 or not resid.is_contiguous() or delta.shape != resid.shape \
            or not delta.is_contiguous():
        raise KernelError("residual_add: float32 contiguous residual and an equally shaped contiguous delta")
    lib = library.core()
    _check(lib, lib.pico_residual_add(_ptr(resid), _ptr(delta), _dt(delta), c_ll(resid.numel()), _stream()))
    return resid


def swiglu(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu(gate_up)
    T, I2 = gate_up.shape
    if I2 % 2 or not gate_up.is_contiguous():
        raise KernelError("swiglu: input must be contiguous [T, 2 I]")
    I = I2 // 2
    if out is None:
        out = torch.empty(T, I, dtype=gate_up.dtype, device=gate_up.device)
    elif out.shape != (T, I) or out.dtype != gate_up.dtype or not out.is_contiguous():
        raise KernelError("swiglu: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_swiglu(_ptr(gate_up), _ptr(out), _dt(gate_up), T, I, _stream()))
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 out = a @ w.T + bias with plain FMA.  a: [M, K] float32 or bfloat16 (rows may be
    strided), w: [N, K] float32."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if w.dtype != torch.float32 or w.stride(1) != 1 or a.stride(1) != 1:
        raise KernelError("gemm_f32: w must be float32 and both operands contiguous along K")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_f32: bias must be contiguous float32 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=a.device)
    elif out.shape != (M, N) or out.dtype != torch.float32 or out.stride(1) != 1:
        raise KernelError("gemm_f32: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_gemm_f32(_ptr(a), _dt(a), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                  a.stride(0) if M > 1 else K, w.stride(0), out.stride(0) if M > 1 else N, _stream()))
    return out


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out_dtype: torch.dtype = torch.bfloat16, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = a @ w.T + bias on the matrix cores; a [M, K], w [N, K] bfloat16, bias float32,
    out float32 or bfloat16."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm_bf16: operands must be bfloat16 and contiguous along K")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_bf16: bias must be contiguous float32 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
    elif out.shape != (M, N) or out.dtype != out_dtype or out.stride(1) != 1:
        raise KernelError("gemm_bf16: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_gemm_bf16(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _DT[out_dtype], M, N, K,
                                   a.stride(0) if M > 1 else K, w.stride(0), out.stride(0) if M > 1 else N,
                                   _stream()))
    return out


EPI_BF16, EPI_F32, EPI_SWIGLU, EPI_RELU2, EPI_F32_ADD = 0, 1, 2, 3, 4
MAX_HEAD_DIM = 256          # the largest head size any attention kernel takes


# The weight-streaming kernel takes any number of rows in blocks of 64, each block reading the matrix
# again.  Up to 64 rows it always serves.  Up to SKINNY_MID_ROWS rows it serves matrices of at most
# SKINNY_MID_WEIGHT elements (the q/k/v and o projections of small models), which the caches hold
# between the blocks: a step of that size is bound by the host's launches, and this kernel costs the
# host less than half of a library call (8 against 19 us) and takes the GPU no longer (10.6 against
# 18.5 us at 128 rows of a 2,048 x 1,536 matrix, 19.5 against 18.9 us at 256).
SKINNY_ROWS, SKINNY_MID_ROWS, SKINNY_MID_WEIGHT = 64, 256, 1 << 22


def skinny_rows(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether a step of this many rows is one the weight-streaming kernel is meant for."""
    return a.dim() == 2 and (a.shape[0] <= SKINNY_ROWS or (a.shape[0] <= SKINNY_MID_ROWS and w.numel() <= SKINNY_MID_WEIGHT))


def skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes these operands (few rows, 16-byte aligned rows)."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2
            and skinny_rows(a, w)
            and a.shape[1] % 8 == 0 and a.stride(1) == 1 and w.stride(1) == 1
            and (a.stride(0) % 8 == 0 or a.shape[0] == 1) and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_BF16,
                k_splits: int = 1, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M <= 64, K] x w [N, K]^T, both bfloat16.  EPI_BF16 -> bf16 [M, N]; EPI_F32 -> float32 [M, N], or with
    k_splits > 1 a stack [k_splits, M, N] of partial sums (bias in the first); EPI_SWIGLU (w = [gate; up])
    -> bf16 [M, N / 2] = silu(gate) * up; EPI_RELU2 -> bf16 [M, N] = max(x w^T + bias, 0)^2; EPI_F32_ADD: ``out``
    (contiguous float32 [M, N], a residual stream) += x w^T + bias, every element by one writer."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if not skinny_ok(a, w):
        raise KernelError("gemm_skinny: operands must be bfloat16, few rows (skinny_ok), K a multiple of 8, rows 16-byte aligned")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny: bias must be contiguous float32 [N]")
    if k_splits > 1 and epilogue != EPI_F32:
        raise KernelError("gemm_skinny: only the float32 epilogue can leave partial sums")
    if epilogue == EPI_F32_ADD:
        if out is None or out.dtype != torch.float32 or tuple(out.shape) != (M, N) or not out.is_contiguous() or not out.is_cuda:
            raise KernelError(f"gemm_skinny: adding needs a contiguous float32 [{M}, {N}] to add into")
        ldo = N
    elif out is not None:
        raise KernelError("gemm_skinny: only the adding epilogue takes an output")
    elif epilogue == EPI_F32:
        shape = (M, N) if k_splits == 1 else (k_splits, M, N)
        out = torch.empty(shape, dtype=torch.float32, device=a.device)
        ldo = N
    elif epilogue == EPI_SWIGLU:
        if N % 2:
            raise KernelError("gemm_skinny: SwiGLU needs an even number of weight rows")
        out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=a.device)
        ldo = N // 2
    else:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
        ldo = N
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny(_ptr(a), a.stride(0) if M > 1 else K, _ptr(w), w.stride(0), _ptr(bias), _ptr(out),
                                     ldo, c_ll(M * N), epilogue, M, N, K, k_splits, _stream()))
    return out


@functools.lru_cache(maxsize=None)
def skinny_k_splits(N: int, K: int, max_splits: int = 8) -> int:
    """Into how many ranges of whole 256-wide steps the k of a small matrix is cut, each range a
    workgroup of its own that leaves a slab of partial sums: the cut with which the fullest compute
    unit reads least.  It depends on the matrix alone, never on the number of tokens."""
    return int(library.core().pico_gemm_skinny_k_splits(N, K, max_splits))


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int):
    """K pages [pages, nkv, P, d]; V pages [pages, nkv, d, P]."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("cache tensors must be contiguous and 4-dimensional")
    pages, h, P, dd = k_cache.shape
    if (h, dd) != (nkv, d) or tuple(v_cache.shape) != (pages, nkv, d, P) or v_cache.dtype != k_cache.dtype:
        raise KernelError(f"cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                          f"{nkv} kv heads of size {d}")
    return pages, P


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0) -> torch.Tensor:
    """cos and sin of position * inv_freq in float32, times ``magnitude``: [T, len(inv_freq), 2].  Every layer of a step
    rotates by the same angles, so a step computes them once."""
    _gpu(positions, inv_freq)
    T = positions.numel()
    _i32(positions, "positions", T)
    if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
        raise KernelError("inv_freq must be contiguous float32")
    out = torch.empty(T, inv_freq.numel(), 2, dtype=torch.float32, device=positions.device)
    lib = library.core()
    _check(lib, lib.pico_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(out), T, inv_freq.numel(), c_float(magnitude),
                                    _stream()))
    return out


def _check_table(cos_sin: Optional[torch.Tensor], T: int, half: int) -> None:
    if half == 0:
        return
    if cos_sin is None or cos_sin.dtype != torch.float32 or cos_sin.shape != (T, half, 2) or not cos_sin.is_contiguous():
        raise KernelError(f"the table of cosines and sines must be contiguous float32 [{T}, {half}, 2]")


def rope_kv_store(qkv: torch.Tensor, cos_sin: Optional[torch.Tensor], slots: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, nq: int, nkv: int, d: int, rotary_dim: int) -> None:
    """Rotate q (in place) and k by the angles of ``cos_sin`` (``rope_table``; None when rotary_dim
    is 0), write k and v of token t to slot ``slots[t]`` (page * page size + offset in the page;
    negative: nothing is stored)."""
    _gpu(qkv, cos_sin, slots, k_cache, v_cache)
    T = qkv.shape[0]
    if qkv.shape != (T, (nq + 2 * nkv) * d) or not qkv.is_contiguous():
        raise KernelError(f"qkv must be contiguous [T, {(nq + 2 * nkv) * d}], got {tuple(qkv.shape)}")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != qkv.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(slots, "slots", T)
    _check_table(cos_sin, T, rotary_dim // 2)
    lib = library.core()
    _check(lib, lib.pico_rope_kv_store(_ptr(qkv), _dt(qkv), _ptr(cos_sin) if rotary_dim else None, _ptr(slots),
                                       _ptr(k_cache), _ptr(v_cache), T, nq, nkv, d, rotary_dim, P, pages, _stream()))


def gemm_skinny_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor,
                     slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     nq: int, nkv: int, d: int) -> torch.Tensor:
    """The q/k/v projection of up to 64 tokens with bias, rotate-half encoding of q and k (over the
    whole head size) and the store of k and v at ``slots`` in one kernel; returns the encoded queries
    [M, nq * d].  w: [(nq + 2 nkv) * d, K] bfloat16, rows [q heads | k heads | v heads]."""
    _gpu(a, w, bias, cos_sin, slots, k_cache, v_cache)
    M, K = a.shape
    if w.shape != ((nq + 2 * nkv) * d, K):
        raise KernelError(f"gemm_skinny_rope: weight {tuple(w.shape)} is not [{(nq + 2 * nkv) * d}, {K}]")
    if not skinny_ok(a, w):
        raise KernelError("gemm_skinny_rope: operands must be bfloat16, few rows (skinny_ok), K a multiple of 8, rows 16-byte aligned")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny_rope: bias must be contiguous float32 [N]")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny_rope: the cache must be bfloat16")
    if d % 32 or P & (P - 1):
        raise KernelError("gemm_skinny_rope: head size must be a multiple of 32 and the page size a power of two")
    _i32(slots, "slots", M)
    _check_table(cos_sin, M, d // 2)
    q = torch.empty(M, nq * d, dtype=torch.bfloat16, device=a.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_rope(_ptr(a), a.stride(0) if M > 1 else K, _ptr(w), w.stride(0), _ptr(bias), _ptr(q),
                                          nq * d, _ptr(cos_sin), _ptr(slots), _ptr(k_cache),
                                          _ptr(v_cache), M, K, nq, nkv, d, P, pages, _stream()))
    return q


# The norm in front of a projection inside the projection's launch: every workgroup norms the row itself, which
# pays for a single row (a decode step of one request: a launch of 4.5 us saved, some reading added).
SKINNY_NORM_ROWS, SKINNY_NORM_MAX_K, SKINNY_NORM_SLABS = 1, 4096, 8


def skinny_norm_ok(resid: torch.Tensor, delta: Optional[torch.Tensor], w: torch.Tensor) -> bool:
    """Whether ``gemm_skinny_norm`` / ``gemm_skinny_rope_norm`` take this residual stream [M, K], these partial
    sums (None, float32 [M, K] or float32 [S, M, K]) and this weight [N, K]."""
    if resid.dim() != 2 or resid.dtype != torch.float32 or not resid.is_contiguous():
        return False
    M, K = resid.shape
    if not (1 <= M <= SKINNY_NORM_ROWS and K % 64 == 0 and K <= SKINNY_NORM_MAX_K):
        return False
    if delta is not None and (delta.dtype != torch.float32 or not delta.is_contiguous() or tuple(delta.shape[-2:]) != (M, K)
                              or delta.dim() not in (2, 3) or (delta.dim() == 3 and delta.shape[0] > SKINNY_NORM_SLABS)):
        return False
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == K and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0)


def _norm_args(resid, delta, norm_w, who):
    M, K = resid.shape
    if norm_w.dtype != torch.float32 or norm_w.shape != (K,) or not norm_w.is_contiguous():
        raise KernelError(f"{who}: norm weight must be float32 of shape [{K}]")
    slabs = 0 if delta is None else (delta.shape[0] if delta.dim() == 3 else 1)
    resid_out = torch.empty_like(resid)
    return M, K, slabs, resid_out


def gemm_skinny_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                     w: torch.Tensor, epilogue: int = EPI_BF16):
    """epilogue(norm(resid + delta) w^T) for one row in one kernel; returns (out, resid + delta).
    The norm is RMSNorm with weight ``norm_w``; epilogues as ``gemm_skinny`` (EPI_F32: one slab)."""
    _gpu(resid, delta, norm_w, w)
    if not skinny_norm_ok(resid, delta, w):
        raise KernelError("gemm_skinny_norm: operands outside what the kernel takes (skinny_norm_ok)")
    M, K, slabs, resid_out = _norm_args(resid, delta, norm_w, "gemm_skinny_norm")
    N = w.shape[0]
    if epilogue == EPI_SWIGLU and N % 2:
        raise KernelError("gemm_skinny_norm: SwiGLU needs an even number of weight rows")
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    out = torch.empty(M, n_out, dtype=torch.float32 if epilogue == EPI_F32 else torch.bfloat16, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_norm(_ptr(resid), _ptr(delta), slabs, c_ll(M * K), _ptr(norm_w), c_float(eps),
                                          _ptr(resid_out), _ptr(w), w.stride(0), _ptr(out), n_out, epilogue, M, N, K,
                                          _stream()))
    return out, resid_out


def gemm_skinny_rope_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                          w: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor, slots: torch.Tensor,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, nq: int, nkv: int, d: int):
    """``gemm_skinny_rope`` on norm(resid + delta) for one row in one kernel; returns (encoded queries
    [M, nq * d], resid + delta)."""
    _gpu(resid, delta, norm_w, w, bias, cos_sin, slots, k_cache, v_cache)
    if not skinny_norm_ok(resid, delta, w):
        raise KernelError("gemm_skinny_rope_norm: operands outside what the kernel takes (skinny_norm_ok)")
    M, K, slabs, resid_out = _norm_args(resid, delta, norm_w, "gemm_skinny_rope_norm")
    if w.shape != ((nq + 2 * nkv) * d, K):
        raise KernelError(f"gemm_skinny_rope_norm: weight {tuple(w.shape)} is not [{(nq + 2 * nkv) * d}, {K}]")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny_rope_norm: bias must be contiguous float32 [N]")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny_rope_norm: the cache must be bfloat16")
    if d % 32 or P & (P - 1):
        raise KernelError("gemm_skinny_rope_norm: head size must be a multiple of 32 and the page size a power of two")
    _i32(slots, "slots", M)
    _check_table(cos_sin, M, d // 2)
    q = torch.empty(M, nq * d, dtype=torch.bfloat16, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_rope_norm(_ptr(resid), _ptr(delta), slabs, c_ll(M * K), _ptr(norm_w), c_float(eps),
                                               _ptr(resid_out), _ptr(w), w.stride(0), _ptr(bias), _ptr(q), nq * d,
                                               _ptr(cos_sin), _ptr(slots), _ptr(k_cache), _ptr(v_cache), M, K, nq, nkv, d,
                                               P, pages, _stream()))
    return q, resid_out


def paged_attention_ref(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                        positions: torch.Tensor, token_seq: torch.Tensor, nq: int, nkv: int, d: int,
                        scale: float, window: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q: [T, >= nq*d] (row stride free, heads first in the row); returns [T, nq*d]."""
    _gpu(q, k_cache, v_cache, block_table, positions, token_seq)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < nq * d:
        raise KernelError("q must be [T, >= nq*d] with unit stride along the row")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != q.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(positions, "positions", T)
    _i32(token_seq, "token_seq", T)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block_table must be contiguous int32 [sequences, pages]")
    if out is None:
        out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    elif out.shape != (T, nq * d) or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError("attention: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_paged_attention_ref(_ptr(q), q.stride(0) if T > 1 else q.shape[1], _dt(q), _ptr(k_cache),
                                             _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                             _ptr(positions), _ptr(token_seq), _ptr(out), T, nq, nkv, d, P, window,
                                             c_float(scale), pages, _stream()))
    return out


def sample_workspace(rows: int, device) -> torch.Tensor:
    """What ``sample`` needs beside its output for up to ``rows`` rows (partial results of its chain of launches)."""
    lib = library.core()
    lib.pico_sample_workspace_words.restype = ctypes.c_longlong
    return torch.empty(max(2, int(lib.pico_sample_workspace_words(rows))), dtype=torch.int32, device=device)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor,
           out: Optional[torch.Tensor] = None, work: Optional[torch.Tensor] = None, top_p_rows: bool = True) -> torch.Tensor:
    """One token id per row of float32 logits; per-row temperature (0 = greedy), top_p and
    uniform number.  ``work``: ``sample_workspace`` for at least as many rows (made here if not given).
    ``top_p_rows=False``: the caller knows that no row has top_p < 1, and the launches that look for the
    threshold of such rows are left out (a top_p below 1 is then taken as 1)."""
    _gpu(logits, temperature, top_p, u, work)
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 with unit stride along the vocabulary")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        if t.dtype != torch.float32 or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be contiguous float32 with one entry per row")
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or out.numel() < R or not out.is_contiguous():
        raise KernelError("sample: out must be contiguous int32 with one entry per row")
    lib = library.core()
    if work is None:
        work = sample_workspace(R, logits.device)
    else:
        lib.pico_sample_workspace_words.restype = ctypes.c_longlong
        if work.dtype != torch.int32 or not work.is_contiguous() or work.numel() < int(lib.pico_sample_workspace_words(R)) \
                or work.data_ptr() % 16:
            raise KernelError("sample: the workspace must come from sample_workspace for at least as many rows")
    _check(lib, lib.pico_sample(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(temperature),
                                _ptr(top_p), _ptr(u), _ptr(out), _ptr(work), int(bool(top_p_rows)), _stream()))
    return out


def argmax_workspace(rows: int, device) -> tuple:
    """What ``argmax`` needs beside its output: the maxima of the chunks of every row and where they are."""
    n = rows * int(library.core().pico_argmax_chunks())
    return torch.empty(n, dtype=torch.float32, device=device), torch.empty(n, dtype=torch.int32, device=device)


def argmax(logits: torch.Tensor, out: torch.Tensor, work: tuple) -> torch.Tensor:
    """The index of the first maximum of every row of float32 logits (what ``sample`` gives for
    temperature 0), several workgroups a row."""
    _gpu(logits, out, *work)
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 with unit stride along the vocabulary")
    if out.dtype != torch.int32 or out.numel() < R or not out.is_contiguous():
        raise KernelError("argmax: out must be contiguous int32 with one entry per row")
    lib = library.core()
    need = R * int(lib.pico_argmax_chunks())
    val, idx = work
    if val.dtype != torch.float32 or idx.dtype != torch.int32 or val.numel() < need or idx.numel() < need \
            or not val.is_contiguous() or not idx.is_contiguous():
        raise KernelError("argmax: the workspace must come from argmax_workspace for at least as many rows")
    _check(lib, lib.pico_argmax(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(val), _ptr(idx), _ptr(out), _stream()))
    return out


def add_rows(resid: torch.Tensor, table: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """resid[t] += table[idx[t]] in float32, in place (learned position vectors: idx = positions)."""
    _gpu(resid, table, idx)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != H or not table.is_contiguous():
        raise KernelError(f"add_rows: the table must be contiguous [rows, {H}]")
    _i32(idx, "idx", T)
    lib = library.core()
    _check(lib, lib.pico_add_rows(_ptr(resid), _ptr(table), _dt(table), _ptr(idx), T, H, table.shape[0], _stream()))
    return resid


def relu2(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """max(x, 0)^2 element by element (``out=x``: in place)."""
    _gpu(x, out)
    if not x.is_contiguous():
        raise KernelError("relu2: the input must be contiguous")
    if out is None:
        out = torch.empty_like(x)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise KernelError("relu2: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_relu2(_ptr(x), _ptr(out), _dt(x), c_ll(x.numel()), _stream()))
    return out


def _check_cache2(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, dk: int, dv: int, nv: Optional[int] = None):
    """K pages [pages, nkv, P, dk]; V pages [pages, nv, dv, P] (nv: nkv unless given)."""
    nv = nkv if nv is None else nv
    if k_cache.dim() != 4 or v_cache.dim() != 4 or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("cache tensors must be contiguous and 4-dimensional")
    pages, h, P, dd = k_cache.shape
    if (h, dd) != (nkv, dk) or tuple(v_cache.shape) != (pages, nv, dv, P) or v_cache.dtype != k_cache.dtype:
        raise KernelError(f"cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                          f"{nkv} kv heads with keys of {dk} and {nv} with values of {dv}")
    return pages, P


def kv_mix_store(qkv: torch.Tensor, k_col: int, v_col: int, slots: torch.Tensor, k_cache: torch.Tensor,
                 v_cache: torch.Tensor, nkv: int, dk: int, dv: int, v_first: Optional[torch.Tensor] = None,
                 mix: float = 0.0) -> None:
    """Write the keys (columns k_col ..) and values (columns v_col ..) of every row of ``qkv`` to ``slots`` (page * page
    size + offset; negative: nothing).  With ``v_first`` [T, nkv * dv] (rows may be strided) the value stored is
    (1 - mix) v + mix v_first, computed in float32."""
    _gpu(qkv, slots, k_cache, v_cache, v_first)
    T = qkv.shape[0]
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < max(k_col + nkv * dk, v_col + nkv * dv):
        raise KernelError("kv_mix_store: qkv must be [T, columns] with unit stride along the row and hold keys and values")
    pages, P = _check_cache2(k_cache, v_cache, nkv, dk, dv)
    if k_cache.dtype != qkv.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(slots, "slots", T)
    if v_first is not None and (v_first.dtype != qkv.dtype or v_first.dim() != 2 or v_first.stride(1) != 1
                                or tuple(v_first.shape) != (T, nkv * dv)):
        raise KernelError(f"kv_mix_store: the first values must be [{T}, {nkv * dv}] of the activations' dtype")
    lib = library.core()
    _check(lib, lib.pico_kv_mix_store(_ptr(qkv), _dt(qkv), qkv.stride(0) if T > 1 else qkv.shape[1], k_col, v_col,
                                      _ptr(v_first), 0 if v_first is None else (v_first.stride(0) if T > 1 else nkv * dv),
                                      c_float(mix), _ptr(slots), _ptr(k_cache), _ptr(v_cache), T, nkv, dk, dv, P, pages,
                                      _stream()))


def attn_bias_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    positions: torch.Tensor, token_seq: torch.Tensor, nq: int, nkv: int, dk: int, dv: int, scale: float,
                    window: int = 0, temp_coef: float = 0.0, temp_every: int = 0, slope_span: float = 0.0,
                    out: Optional[torch.Tensor] = None, softcap: float = 0.0, keep_first: int = 0,
                    gate: Optional[torch.Tensor] = None, chunk: int = 0, sink: bool = False, gate_heads: bool = False,
                    v_div: int = 1, out_f32: bool = False) -> torch.Tensor:
    """Attention with a distance penalty slope_h (i - j), slope_h = 2^(-slope_span (h + 1) / nq), and the query
    temperature 1 + temp_coef ln(floor((i + 1) / temp_every) + 1) on the scores.  q: [T, >= nq * dk]; returns [T, nq * dv].
    ``softcap`` > 0: scores <- softcap tanh(scores / softcap).  ``keep_first``: with a window, keys at positions below it
    stay visible.  ``gate`` [T, >= nq * dv] (row stride free): the output is multiplied with sigmoid(gate); with
    ``gate_heads`` the gate is [T, >= nq], one number a head.  ``chunk`` > 0 (instead of a window): key j <= i is seen iff
    floor(i / chunk) == floor(j / chunk).  ``sink``: the softmax's denominator gains a 1.  ``v_div``: kv head g reads value
    head g // v_div (the value pages hold nkv // v_div heads).  ``out_f32``: the output is float32 whatever q's dtype."""
    _gpu(q, k_cache, v_cache, block_table, positions, token_seq, gate)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < nq * dk:
        raise KernelError("q must be [T, >= nq*dk] with unit stride along the row")
    if v_div < 1 or nkv % v_div or chunk < 0 or (chunk and window):
        raise KernelError("attention: kv heads share values in whole groups; chunks or a window, not both")
    pages, P = _check_cache2(k_cache, v_cache, nkv, dk, dv, nkv // v_div)
    if k_cache.dtype != q.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(positions, "positions", T)
    _i32(token_seq, "token_seq", T)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block_table must be contiguous int32 [sequences, pages]")
    odt = torch.float32 if out_f32 else q.dtype
    if out is None:
        out = torch.empty(T, nq * dv, dtype=odt, device=q.device)
    elif out.shape != (T, nq * dv) or out.dtype != odt or not out.is_contiguous():
        raise KernelError("attention: out has the wrong shape or dtype")
    if gate is not None and (gate.dtype != q.dtype or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != T
                             or gate.shape[1] < (nq if gate_heads else nq * dv)):
        raise KernelError(f"attention: the gate must be [T, >= {nq if gate_heads else nq * dv}] of the activations' dtype")
    lib = library.core()
    _check(lib, lib.pico_attn_bias_plain(_ptr(q), q.stride(0) if T > 1 else q.shape[1], _dt(q), _ptr(k_cache), _ptr(v_cache),
                                         _ptr(block_table), block_table.shape[1], _ptr(positions), _ptr(token_seq), _ptr(out),
                                         T, nq, nkv, dk, dv, P, window, c_float(scale), c_float(temp_coef), temp_every,
                                         c_float(slope_span), pages, c_float(softcap), keep_first, _ptr(gate),
                                         0 if gate is None else (gate.stride(0) if T > 1 else gate.shape[1]), chunk,
                                         1 if sink else 0, 1 if gate_heads else 0, v_div, 1 if out_f32 else 0, _stream()))
    return out


def rope_pairs_store(x: torch.Tensor, q_col: int, k_col: int, v_col: int, cos_sin: Optional[torch.Tensor], rotary_dim: int,
                     slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                     nq: int, nkv: int, dk: int, dv: int) -> None:
    """Turn neighbouring pairs (2i, 2i + 1) of the first ``rotary_dim`` entries of every query head (in place, columns
    q_col ..) and key head (columns k_col ..) of ``x`` [T, columns] by the angles of ``cos_sin`` (``rope_table``), and
    write keys and values (columns v_col ..) to ``slots`` of the cache.  Without a cache only the queries are turned."""
    _gpu(x, cos_sin, slots, k_cache, v_cache)
    T = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < q_col + nq * dk:
        raise KernelError("rope_pairs_store: x must be [T, columns] with unit stride along the row and hold the queries")
    pages = P = 0
    if k_cache is not None:
        pages, P = _check_cache2(k_cache, v_cache, nkv, dk, dv)
        if k_cache.dtype != x.dtype:
            raise KernelError("cache and activations differ in dtype")
        if x.shape[1] < max(k_col + nkv * dk, v_col + nkv * dv):
            raise KernelError("rope_pairs_store: the rows do not hold the keys and values")
        _i32(slots, "slots", T)
    if rotary_dim % 2 or not 0 <= rotary_dim <= dk:
        raise KernelError(f"rope_pairs_store: {rotary_dim} rotated entries do not fit a head of {dk}")
    _check_table(cos_sin, T, rotary_dim // 2)
    lib = library.core()
    _check(lib, lib.pico_rope_pairs_store(_ptr(x), _dt(x), x.stride(0) if T > 1 else x.shape[1], q_col, k_col, v_col,
                                          _ptr(cos_sin) if rotary_dim else None, rotary_dim, _ptr(slots), _ptr(k_cache),
                                          _ptr(v_cache), T, nq, nkv, dk, dv, P, pages, _stream()))


def gla_decay(x: torch.Tensor, col: int, a2: torch.Tensor, bias: Optional[torch.Tensor], tau: float) -> torch.Tensor:
    """float32 [T, C]: log(sigmoid(z)) / tau with z = x[:, col : col + R] a2^T + bias; a2 [C, R] of x's dtype, bias float32."""
    _gpu(x, a2, bias)
    T = x.shape[0]
    C, R = a2.shape
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < col + R or a2.dtype != x.dtype or not a2.is_contiguous():
        raise KernelError("gla_decay: x [T, >= col + R] with unit stride along the row and a2 [C, R] of the same dtype")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (C,) or not bias.is_contiguous()):
        raise KernelError(f"gla_decay: bias must be contiguous float32 [{C}]")
    out = torch.empty(T, C, dtype=torch.float32, device=x.device)
    lib = library.core()
    xv = x[:, col:]
    _check(lib, lib.pico_gla_decay(_ptr(xv), x.stride(0) if T > 1 else x.shape[1], _dt(x), _ptr(a2), _ptr(bias), c_float(tau),
                                   _ptr(out), T, C, R, _stream()))
    return out


GLA_MAX_KEY_DIM = 256


def gla_scan(x: torch.Tensor, q_col: int, k_col: int, v_col: int, log_decay: Optional[torch.Tensor], cu_seqlens: torch.Tensor,
             state_slots: torch.Tensor, state: torch.Tensor, num_seqs: int, heads: int, dk: int, dv: int,
             qscale: float, chunk: int = 0, decay_from: Optional[tuple] = None,
             head_decay: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The recurrence S <- diag(exp(log_decay_t)) S + k_t v_t^T, o_t = S^T q_t qscale, for every sequence of the step from
    its state slot (``state`` float32 [slots, heads, dk, dv], updated in place).  Returns o float32 [T, heads * dv].
    ``chunk`` > 0: sequences are cut into chunks of that many tokens that run side by side (every chunk from zero, a walk
    over the chunks' states, every chunk again from its true state): the same sums in another order.
    ``log_decay`` None (whole walks only): the decays are made inside the launch from ``decay_from`` = (column of the
    low-rank activations in x, a2 [heads * dk, R], bias float32 or None, tau), as ``gla_decay`` makes them."""
    _gpu(x, log_decay, cu_seqlens, state_slots, state)
    T = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < max(q_col + heads * dk, k_col + heads * dk, v_col + heads * dv):
        raise KernelError("gla_scan: x must be [T, columns] with unit stride along the row and hold q, k and v")
    a_col, a2, a2_bias, tau, R = 0, None, None, 0.0, 0
    if head_decay is not None:
        # one constant decay a head (float32 [heads], the decays themselves): no logarithms are read or made
        _gpu(head_decay)
        if log_decay is not None or head_decay.dtype != torch.float32 or tuple(head_decay.shape) != (heads,) or not head_decay.is_contiguous():
            raise KernelError(f"gla_scan: a fixed decay is contiguous float32 [{heads}] and comes without logarithms")
    elif log_decay is None:
        if chunk or decay_from is None:
            raise KernelError("gla_scan: without the decays' logarithms the walk runs whole and needs what makes them")
        a_col, a2, a2_bias, tau = decay_from
        _gpu(a2, a2_bias)
        R = a2.shape[1]
        if a2.dtype != x.dtype or tuple(a2.shape) != (heads * dk, R) or not a2.is_contiguous() or x.shape[1] < a_col + R:
            raise KernelError("gla_scan: a2 [heads * dk, R] of x's dtype, and x must hold the R low-rank activations")
        if a2_bias is not None and (a2_bias.dtype != torch.float32 or a2_bias.shape != (heads * dk,) or not a2_bias.is_contiguous()):
            raise KernelError("gla_scan: the decay's bias must be contiguous float32")
    elif log_decay.dtype != torch.float32 or tuple(log_decay.shape) != (T, heads * dk) or not log_decay.is_contiguous():
        raise KernelError(f"gla_scan: the decays' logarithms must be contiguous float32 [{T}, {heads * dk}]")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dk, dv) or not state.is_contiguous():
        raise KernelError(f"gla_scan: the state must be contiguous float32 [slots, {heads}, {dk}, {dv}]")
    if dk > GLA_MAX_KEY_DIM:
        raise KernelError(f"gla_scan: at most {GLA_MAX_KEY_DIM} key channels a head")
    _i32(cu_seqlens, "cu_seqlens", num_seqs + 1)
    _i32(state_slots, "state_slots", num_seqs)
    out = torch.empty(T, heads * dv, dtype=torch.float32, device=x.device)
    ws = ws_decay = None
    max_chunks = 0
    if chunk > 0:
        max_chunks = -(-T // chunk)
        ws = torch.empty(num_seqs * max_chunks, heads, dk, dv, dtype=torch.float32, device=x.device)
        ws_decay = torch.empty(num_seqs * max_chunks, heads, dk, dtype=torch.float32, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_gla_scan(_ptr(x), x.stride(0) if T > 1 else x.shape[1], _dt(x), q_col, k_col, v_col, _ptr(log_decay),
                                  _ptr(cu_seqlens), _ptr(state_slots), _ptr(state), _ptr(out), num_seqs, T, heads, dk, dv,
                                  c_float(qscale), state.shape[0], chunk, max_chunks, _ptr(ws), _ptr(ws_decay), _ptr(a2),
                                  _ptr(a2_bias), a_col, R, c_float(tau), _ptr(head_decay), _stream()))
    return out


def gla_out(o: torch.Tensor, x: torch.Tensor, g_col: int, weight: torch.Tensor, eps: float, heads: int, dv: int,
            sigmoid_gate: bool = False) -> torch.Tensor:
    """[T, heads * dv] of x's dtype: every head of ``o`` (float32) RMS-normed over its dv entries with ``weight`` [dv],
    times silu of the gate (columns g_col .. of x), or with ``sigmoid_gate`` times its sigmoid."""
    _gpu(o, x, weight)
    T = o.shape[0]
    if o.dtype != torch.float32 or tuple(o.shape) != (T, heads * dv) or not o.is_contiguous():
        raise KernelError(f"gla_out: o must be contiguous float32 [T, {heads * dv}]")
    if x.dim() != 2 or x.shape[0] != T or x.stride(1) != 1 or x.shape[1] < g_col + heads * dv:
        raise KernelError("gla_out: the rows do not hold the gate")
    if weight.dtype != torch.float32 or weight.shape != (dv,) or not weight.is_contiguous():
        raise KernelError(f"gla_out: the norm's weight must be contiguous float32 [{dv}]")
    out = torch.empty(T, heads * dv, dtype=x.dtype, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_gla_out(_ptr(o), _ptr(x[:, g_col:]), x.stride(0) if T > 1 else x.shape[1], _dt(x), _ptr(weight),
                                 c_float(eps), _ptr(out), T, heads, dv, 1 if sigmoid_gate else 0, _stream()))
    return out


MOE_MAX_TOP = 16


def moe_route(logits: torch.Tensor, top: int):
    """(experts int32 [T, top], weights float32 [T, top]): every row's ``top`` largest logits (the lowest index among
    equal ones) and their sigmoids."""
    _gpu(logits)
    T, E = logits.shape
    if logits.dtype != torch.float32 or not logits.is_contiguous():
        raise KernelError("moe_route: router logits must be contiguous float32")
    if not 1 <= top <= min(E, MOE_MAX_TOP):
        raise KernelError(f"moe_route: {top} of {E} experts per token (at most {MOE_MAX_TOP})")
    experts = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    lib = library.core()
    _check(lib, lib.pico_moe_route(_ptr(logits), T, E, top, _ptr(experts), _ptr(weights), _stream()))
    return experts, weights


def moe_router(x: torch.Tensor, w_router: torch.Tensor, top: int):
    """Router and choice: z = x w_router^T in float32 (w_router float32 [E, D]; x float32 or bfloat16 with
    unit stride along the row), then as ``moe_route``: (experts int32 [T, top], weights float32 [T, top])."""
    _gpu(x, w_router)
    T, D = x.shape
    E = w_router.shape[0]
    if w_router.dtype != torch.float32 or w_router.dim() != 2 or w_router.shape[1] != D or not w_router.is_contiguous():
        raise KernelError(f"moe_router: the router matrix must be contiguous float32 [experts, {D}]")
    if x.stride(1) != 1:
        raise KernelError("moe_router: activations must have unit stride along the row")
    if not 1 <= top <= min(E, MOE_MAX_TOP):
        raise KernelError(f"moe_router: {top} of {E} experts per token (at most {MOE_MAX_TOP})")
    z = torch.empty(T, E, dtype=torch.float32, device=x.device)
    experts = torch.empty(T, top, dtype=torch.int32, device=x.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_moe_router(_ptr(x), x.stride(0) if T > 1 else D, _dt(x), _ptr(w_router), T, E, D, top,
                                    _ptr(z), _ptr(experts), _ptr(weights), _stream()))
    return experts, weights


def moe_router_softmax(x: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor], top: int, scale: float):
    """Router and choice by softmax scores: z = x w_router^T in float32, s = softmax(z) over all E router outputs; the
    ``top`` largest of s + correction are chosen (the lowest index among equals); weights = the chosen s over their sum
    (+ 1e-20) times ``scale``.  Returns (experts int32 [T, top], weights float32 [T, top])."""
    _gpu(x, w_router, correction)
    T, D = x.shape
    E = w_router.shape[0]
    if w_router.dtype != torch.float32 or w_router.dim() != 2 or w_router.shape[1] != D or not w_router.is_contiguous():
        raise KernelError(f"moe_router_softmax: the router matrix must be contiguous float32 [outputs, {D}]")
    if correction is not None and (correction.dtype != torch.float32 or correction.shape != (E,) or not correction.is_contiguous()):
        raise KernelError(f"moe_router_softmax: the correction must be contiguous float32 [{E}]")
    if x.stride(1) != 1:
        raise KernelError("moe_router_softmax: activations must have unit stride along the row")
    if not 1 <= top <= min(E, MOE_MAX_TOP):
        raise KernelError(f"moe_router_softmax: {top} of {E} experts per token (at most {MOE_MAX_TOP})")
    z = torch.empty(T, E, dtype=torch.float32, device=x.device)
    experts = torch.empty(T, top, dtype=torch.int32, device=x.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_moe_router_softmax(_ptr(x), x.stride(0) if T > 1 else D, _dt(x), _ptr(w_router), _ptr(correction),
                                            T, E, D, top, c_float(scale), _ptr(z), _ptr(experts), _ptr(weights), _stream()))
    return experts, weights


def moe_identity(h: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor, out: torch.Tensor, num_experts: int) -> torch.Tensor:
    """Experts numbered from ``num_experts`` on hand their input on: ``out`` float32 [T, D] += sum of their weights
    times h; or, for a stack [top, T, D] of slabs (one a slot), the slab rows of such slots = weight times h (no
    expert's product writes them)."""
    _gpu(h, experts, weights, out)
    T, D = h.shape
    top = experts.shape[1]
    stacked = out.dim() == 3
    if out.dtype != torch.float32 or not out.is_contiguous() or tuple(out.shape) != ((top, T, D) if stacked else (T, D)):
        raise KernelError("moe_identity: out must be contiguous float32 [T, D] or [top, T, D]")
    if experts.dtype != torch.int32 or weights.dtype != torch.float32 or experts.shape != weights.shape \
            or experts.shape[0] != T or not experts.is_contiguous() or not weights.is_contiguous() or h.stride(1) != 1:
        raise KernelError("moe_identity: experts int32 [T, top], weights float32 [T, top], rows with unit stride")
    lib = library.core()
    _check(lib, lib.pico_moe_identity(_ptr(h), h.stride(0) if T > 1 else D, _dt(h), _ptr(experts), _ptr(weights), _ptr(out),
                                      T, top, num_experts, D, int(stacked), _stream()))
    return out


MOE_CLIPPED, MOE_SWIGLU = 0, 1      # the experts' activation: clipped with the weight on the input; silu(g) u, weight on the output


def _check_experts(h, gate_up, down, experts, weights, who):
    T, D = h.shape
    if gate_up.dim() != 3 or down.dim() != 3 or gate_up.shape[1] % 2:
        raise KernelError(f"{who}: expert matrices are gate_up [E, 2 F, D] and down [E, D, F]")
    E, F = gate_up.shape[0], gate_up.shape[1] // 2
    if gate_up.shape[2] != D or tuple(down.shape) != (E, D, F) or not gate_up.is_contiguous() or not down.is_contiguous():
        raise KernelError(f"{who}: expert matrices do not fit rows of {D}: {tuple(gate_up.shape)} / {tuple(down.shape)}")
    if gate_up.dtype != h.dtype or down.dtype != h.dtype:
        raise KernelError(f"{who}: activations and expert matrices differ in dtype")
    if h.stride(1) != 1:
        raise KernelError(f"{who}: activations must have unit stride along the row")
    if experts.dtype != torch.int32 or weights.dtype != torch.float32 or experts.shape != weights.shape \
            or experts.shape[0] != T or not experts.is_contiguous() or not weights.is_contiguous():
        raise KernelError(f"{who}: experts int32 [T, top] and weights float32 [T, top]")
    return T, D, E, F, experts.shape[1]


def moe_experts_plain(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, experts: torch.Tensor,
                      weights: torch.Tensor, limit: float, alpha: float, mode: int = MOE_CLIPPED) -> torch.Tensor:
    """float32 [T, D]: sum over a token's experts of down_e(act(gate_up_e (w h))), by the plain kernels."""
    _gpu(h, gate_up, down, experts, weights)
    T, D, E, F, top = _check_experts(h, gate_up, down, experts, weights, "moe_experts_plain")
    y = torch.empty(T * top, F, dtype=h.dtype, device=h.device)
    out = torch.empty(T, D, dtype=torch.float32, device=h.device)
    lib = library.core()
    _check(lib, lib.pico_moe_experts_plain(_ptr(h), h.stride(0) if T > 1 else D, _dt(h), _ptr(gate_up), _ptr(down),
                                           _ptr(experts), _ptr(weights), _ptr(y), _ptr(out), T, top, E, F, D,
                                           c_float(limit), c_float(alpha), mode, _stream()))
    return out


MOE_STREAM_ROWS = 32        # up to this many (token, expert) rows every row streams its expert's matrices


def moe_fast_ok(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> bool:
    """Whether the bfloat16 kernels take these operands (sizes in multiples of 8, 16-byte aligned rows)."""
    return (h.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 and down.dtype == torch.bfloat16
            and h.dim() == 2 and h.stride(1) == 1 and h.shape[1] % 8 == 0 and down.shape[2] % 8 == 0
            and (h.stride(0) % 8 == 0 or h.shape[0] == 1) and h.data_ptr() % 16 == 0
            and gate_up.data_ptr() % 16 == 0 and down.data_ptr() % 16 == 0 and gate_up.shape[0] <= 1024)


def moe_grouped_rows(tokens: int, top: int) -> bool:
    """Whether a step of this many tokens sorts its rows by expert and multiplies on the matrix cores (decided from
    the step's size alone)."""
    return tokens * top > MOE_STREAM_ROWS


def moe_experts(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, experts: torch.Tensor,
                weights: torch.Tensor, limit: float, alpha: float, grouped: Optional[bool] = None,
                mode: int = MOE_CLIPPED) -> torch.Tensor:
    """The experts' outputs in bfloat16 storage: float32 [T, D] (few rows: each streams its expert's matrices), or a
    float32 stack [top, T, D] whose sum over the first index it is (many rows: sorted by expert on the device and
    multiplied on the matrix cores)."""
    _gpu(h, gate_up, down, experts, weights)
    T, D, E, F, top = _check_experts(h, gate_up, down, experts, weights, "moe_experts")
    if not moe_fast_ok(h, gate_up, down):
        raise KernelError("moe_experts: bfloat16 operands with sizes in multiples of 8 and 16-byte aligned rows")
    lib = library.core()
    ldh = h.stride(0) if T > 1 else D
    if grouped is None:
        grouped = moe_grouped_rows(T, top)
    if not grouped:
        y = torch.empty(T * top, F, dtype=h.dtype, device=h.device)
        out = torch.empty(T, D, dtype=torch.float32, device=h.device)
        _check(lib, lib.pico_moe_experts_rows(_ptr(h), ldh, _ptr(gate_up), _ptr(down), _ptr(experts), _ptr(weights),
                                              _ptr(y), _ptr(out), T, top, E, F, D, c_float(limit), c_float(alpha), mode, _stream()))
        return out
    bm = lib.pico_moe_tile_rows()
    tiles = (T * top + E * (bm - 1)) // bm
    sorted_rows = torch.empty(tiles * bm, dtype=torch.int32, device=h.device)
    tile_expert = torch.empty(tiles, dtype=torch.int32, device=h.device)
    y = torch.empty(tiles * bm, F, dtype=h.dtype, device=h.device)
    # a slot whose expert has no matrices (a number from E on) is written by no product: with one slot a token the
    # caller adds into the rows, which then start from zero; with several, ``moe_identity`` fills the slabs' rows
    out = (torch.zeros if top == 1 else torch.empty)(top, T, D, dtype=torch.float32, device=h.device)
    _check(lib, lib.pico_moe_experts_grouped(_ptr(h), ldh, _ptr(gate_up), _ptr(down), _ptr(experts), _ptr(weights),
                                             _ptr(sorted_rows), _ptr(tile_expert), tiles, _ptr(y), _ptr(out), T, top, E, F,
                                             D, c_float(limit), c_float(alpha), mode, _stream()))
    return out[0] if top == 1 else out


# ---- layer norm, scaled sums, the embedding of token pairs ---------------------------------------------------------
LN_MAX_SLABS = 16


def _delta_args(resid, delta, who):
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    slabs = 1
    if delta is not None:
        if delta.dim() == 3:
            slabs = delta.shape[0]
            if delta.dtype != torch.float32:
                raise KernelError("a stack of partial sums must be float32")
        if tuple(delta.shape[-2:]) != (T, H) or not delta.is_contiguous():
            raise KernelError(f"{who}: delta must be contiguous and shaped like the residual stream")
    return T, H, slabs


def _vec(t, H, name):
    if t is not None and (t.dtype != torch.float32 or tuple(t.shape) != (H,) or not t.is_contiguous()):
        raise KernelError(f"{name} must be contiguous float32 [{H}]")


def add_layernorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor, eps: float,
                  out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                  delta_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Layer norm (weight and bias, the variance from the deviations) of resid + delta_scale * delta.
    rows is None: resid is updated in place and every row normed; rows given: only those rows, resid left alone.
    delta: [T, H], or a float32 stack [S, T, H] whose slabs are added up first; delta_scale: float32 [H] or None (ones)."""
    _gpu(resid, delta, weight, bias, rows, delta_scale)
    T, H, slabs = _delta_args(resid, delta, "add_layernorm")
    _vec(weight, H, "norm weight"); _vec(bias, H, "norm bias"); _vec(delta_scale, H, "delta scale")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_add_layernorm(_ptr(resid), _ptr(delta), _dt(delta) if delta is not None else F32, slabs, c_ll(T * H),
                                       _ptr(delta_scale), _ptr(weight), _ptr(bias), _ptr(out), _DT[out_dtype], _ptr(rows), n, H,
                                       c_float(eps), _stream()))
    return out


def scaled_add(resid: torch.Tensor, a: Optional[torch.Tensor], b: Optional[torch.Tensor] = None,
               gate: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """resid (float32 [T, H], in place) += scale * (a + sigmoid(gate) * b).  a: [T, H] or a float32 stack [S, T, H];
    b: [T, H]; gate: float32 logits, one a row (a column of a wider float32 matrix will do); scale float32 [H] or None."""
    _gpu(resid, a, b, gate, scale)
    T, H, slabs = _delta_args(resid, a, "scaled_add")
    _vec(scale, H, "scale")
    if b is not None and (tuple(b.shape) != (T, H) or not b.is_contiguous()):
        raise KernelError("scaled_add: b must be contiguous and shaped like the residual stream")
    gs = 0
    if gate is not None:
        if b is None or gate.dtype != torch.float32 or gate.shape[0] != T or gate.dim() > 2 or (gate.dim() == 2 and gate.shape[1] != 1):
            raise KernelError("scaled_add: the gate is float32 [T] or [T, 1] and goes with b")
        gs = gate.stride(0) if T > 1 else 1
    lib = library.core()
    _check(lib, lib.pico_scaled_add(_ptr(resid), _ptr(a), _dt(a) if a is not None else F32, slabs, c_ll(T * H), _ptr(b),
                                    _dt(b) if b is not None else F32, _ptr(gate), gs, _ptr(scale), T, H, _stream()))
    return resid


def pair_embed(resid: torch.Tensor, table: torch.Tensor, ctx, last: torch.Tensor, mul_prev: int, mul_cur: int, buckets: int) -> torch.Tensor:
    """resid[t] += table[(previous token * mul_prev + token * mul_cur) mod buckets], at position 0 table[buckets].
    ``last`` int32 [slots]: every sequence's last token of the step before; updated to this step's."""
    _gpu(resid, table, last)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    if table.dim() != 2 or tuple(table.shape) != (buckets + 1, H) or not table.is_contiguous():
        raise KernelError(f"pair_embed: the table must be contiguous [{buckets + 1}, {H}]")
    if last.dtype != torch.int32 or not last.is_contiguous():
        raise KernelError("pair_embed: the last tokens are contiguous int32, one a state slot")
    B = ctx.num_seqs
    _i32(ctx.token_ids, "token_ids", T); _i32(ctx.positions, "positions", T); _i32(ctx.token_seq, "token_seq", T)
    _i32(ctx.cu_seqlens, "cu_seqlens", B + 1); _i32(ctx.state_slots, "state_slots", B)
    lib = library.core()
    _check(lib, lib.pico_pair_embed(_ptr(resid), _ptr(table), _dt(table), _ptr(ctx.token_ids), _ptr(ctx.positions),
                                    _ptr(ctx.token_seq), _ptr(ctx.cu_seqlens), _ptr(ctx.state_slots), _ptr(last), last.numel(),
                                    c_ll(mul_prev), c_ll(mul_cur), buckets, T, B, H, _stream()))
    return resid


# ---- attention through latents ---------------------------------------------------------------------------------------
def latent_prepare(y: torch.Tensor, q_rank: int, kv_rank: int, rot: int, wq: torch.Tensor, wkv: torch.Tensor, eps: float,
                   cos_sin: Optional[torch.Tensor], slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> torch.Tensor:
    """y [T, q_rank + kv_rank + rot]: returns the normed query latent [T, q_rank]; writes the normed key/value latent and
    the turned rotated key part into the cache (K rows [latent | rotated part], V columns the latent again)."""
    _gpu(y, wq, wkv, cos_sin, slots, k_cache, v_cache)
    T = y.shape[0]
    if y.dim() != 2 or y.stride(1) != 1 or y.shape[1] < q_rank + kv_rank + rot:
        raise KernelError("latent_prepare: the rows do not hold the two latents and the rotated part")
    pages, P = _check_cache2(k_cache, v_cache, 1, kv_rank + rot, kv_rank)
    if k_cache.dtype != y.dtype:
        raise KernelError("cache and activations differ in dtype")
    _vec(wq, q_rank, "the query latent's norm weight"); _vec(wkv, kv_rank, "the key/value latent's norm weight")
    _i32(slots, "slots", T)
    if rot:
        _check_table(cos_sin, T, rot // 2)
    cq = torch.empty(T, q_rank, dtype=y.dtype, device=y.device)
    lib = library.core()
    _check(lib, lib.pico_latent_prepare(_ptr(y), y.stride(0) if T > 1 else y.shape[1], _dt(y), q_rank, kv_rank, rot, _ptr(wq),
                                        _ptr(wkv), c_float(eps), _ptr(cos_sin), _ptr(slots), _ptr(cq), _ptr(k_cache),
                                        _ptr(v_cache), T, P, pages, _stream()))
    return cq


def rope_inplace(x: torch.Tensor, col0: int, heads: int, head_stride: int, rot: int, cos_sin: torch.Tensor, halves: bool) -> torch.Tensor:
    """Turn ``rot`` entries from column col0 + h * head_stride of every row of x, for h < heads, by the angles of
    ``cos_sin`` (``rope_table``): neighbouring pairs, or with ``halves`` entry i with entry i + rot / 2."""
    _gpu(x, cos_sin)
    T = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("rope_inplace: x must be [T, columns] with unit stride along the row")
    if rot:
        _check_table(cos_sin, T, rot // 2)
    lib = library.core()
    _check(lib, lib.pico_rope_inplace(_ptr(x), x.stride(0) if T > 1 else x.shape[1], _dt(x), col0, heads, head_stride, rot,
                                      1 if halves else 0, _ptr(cos_sin), T, _stream()))
    return x


def head_linear(x: torch.Tensor, x_col: int, x_head: int, w: torch.Tensor, heads: int, copy: int = 0,
                out: Optional[torch.Tensor] = None, turn: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A product a head: out[t, h, :n_out] = x[t, x_col + h * x_head : .. + n_in] @ w[h] with w [heads, n_in, n_out];
    the ``copy`` entries behind a head's inputs are handed on behind its outputs, as they are or (``turn``: a table of
    ``rope_table`` for copy / 2 pairs) turned by the token's angles, neighbours in pairs.  Returns [T, heads * (n_out + copy)]."""
    _gpu(x, w, out, turn)
    T = x.shape[0]
    if w.dim() != 3 or w.shape[0] != heads or not w.is_contiguous() or w.dtype != x.dtype:
        raise KernelError("head_linear: w must be contiguous [heads, in, out] of the activations' dtype")
    n_in, n_out = w.shape[1], w.shape[2]
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("head_linear: x must be [T, columns] with unit stride along the row")
    o_head = n_out + copy
    if out is None:
        out = torch.empty(T, heads * o_head, dtype=x.dtype, device=x.device)
    elif tuple(out.shape) != (T, heads * o_head) or out.dtype != x.dtype or not out.is_contiguous():
        raise KernelError("head_linear: out has the wrong shape or dtype")
    if turn is not None:
        if copy % 2 or copy == 0:
            raise KernelError("head_linear: a part that is turned has an even, positive number of entries")
        _check_table(turn, T, copy // 2)
    lib = library.core()
    _check(lib, lib.pico_head_linear(_ptr(x), x.stride(0) if T > 1 else x.shape[1], x_col, x_head, _ptr(w), _ptr(out),
                                     heads * o_head, 0, o_head, _dt(x), T, heads, n_in, n_out, copy, _ptr(turn), _stream()))
    return out


# ---- the selective state-space mixer -----------------------------------------------------------------------------------
SSM_MAX_TAPS, SSM_MAX_STATE = 16, 256


def causal_conv(x: torch.Tensor, channels: int, w: torch.Tensor, bias: torch.Tensor, ctx, state: torch.Tensor, n_state: int,
                single: bool = False) -> torch.Tensor:
    """silu(bias + the causal convolution of the first ``channels`` columns of x with w [taps, channels] (tap by tap,
    the last row the current token's)) for every
    sequence of the step; inputs before a portion come from the slot's history (``state`` float32
    [slots, channels, n_state + taps - 1], its last taps - 1 columns), which is brought up to date.  ``single``: every
    sequence of the step brings one token (one launch makes the convolution and the history)."""
    _gpu(x, w, bias, state)
    T = x.shape[0]
    taps = w.shape[0]
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < channels:
        raise KernelError("causal_conv: the rows do not hold the channels")
    if w.dtype != torch.float32 or tuple(w.shape) != (taps, channels) or not w.is_contiguous() or not 1 <= taps <= SSM_MAX_TAPS:
        raise KernelError(f"causal_conv: the taps are contiguous float32 [1 to {SSM_MAX_TAPS}, {channels}]")
    _vec(bias, channels, "the convolution's bias")          # None: no bias
    if state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (channels, n_state + taps - 1) or not state.is_contiguous():
        raise KernelError(f"causal_conv: the state must be contiguous float32 [slots, {channels}, {n_state + taps - 1}]")
    B = ctx.num_seqs
    _i32(ctx.token_seq, "token_seq", T); _i32(ctx.cu_seqlens, "cu_seqlens", B + 1); _i32(ctx.state_slots, "state_slots", B)
    out = torch.empty(T, channels, dtype=x.dtype, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_causal_conv(_ptr(x), x.stride(0) if T > 1 else x.shape[1], _dt(x), _ptr(w), _ptr(bias), _ptr(ctx.token_seq),
                                     _ptr(ctx.cu_seqlens), _ptr(ctx.state_slots), _ptr(state), state.shape[0], T, B, channels,
                                     n_state, taps, _ptr(out), 1 if single and T == B else 0, _stream()))
    return out


def selective_scan(xc: torch.Tensor, dt_pre: torch.Tensor, dt_bias: torch.Tensor, bc: torch.Tensor, b_col: int, c_col: int,
                   a_log: torch.Tensor, d: torch.Tensor, z: torch.Tensor, ctx, state: torch.Tensor, hist: int,
                   chunk: int = 0) -> torch.Tensor:
    """The recurrence S <- exp(dt A) S + dt x B, y = S . C + D x with dt = softplus(dt_pre + dt_bias), A = -exp(a_log), for
    every sequence of the step from its state slot (``state`` float32 [slots, channels, N + hist], updated in place);
    returns y * silu(z) [T, channels] in xc's dtype.  xc [T, channels]; dt_pre float32 [T, channels]; B and C are
    columns b_col .. and c_col .. of ``bc``; z [T, >= channels] (row stride free).
    ``chunk`` > 0: sequences are cut into chunks of that many tokens that run side by side (every chunk from zero, a walk
    over the chunks' states, every chunk again from its true state): the same sums in another order."""
    _gpu(xc, dt_pre, dt_bias, bc, a_log, d, z, state)
    T, C = xc.shape
    N = a_log.shape[1]
    if not xc.is_contiguous() or dt_pre.dtype != torch.float32 or tuple(dt_pre.shape) != (T, C) or not dt_pre.is_contiguous():
        raise KernelError("selective_scan: xc [T, channels] contiguous and dt_pre float32 of the same shape")
    if a_log.dtype != torch.float32 or tuple(a_log.shape) != (C, N) or not a_log.is_contiguous() or N > SSM_MAX_STATE:
        raise KernelError(f"selective_scan: a_log must be contiguous float32 [{C}, at most {SSM_MAX_STATE}]")
    _vec(dt_bias, C, "dt bias"); _vec(d, C, "D")
    if bc.dtype != xc.dtype or bc.dim() != 2 or bc.shape[0] != T or bc.stride(1) != 1 or bc.shape[1] < max(b_col, c_col) + N:
        raise KernelError("selective_scan: the rows of bc do not hold B and C")
    if z.dtype != xc.dtype or z.dim() != 2 or z.shape[0] != T or z.stride(1) != 1 or z.shape[1] < C:
        raise KernelError("selective_scan: z must be [T, >= channels] of the activations' dtype")
    if state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (C, N + hist) or not state.is_contiguous():
        raise KernelError(f"selective_scan: the state must be contiguous float32 [slots, {C}, {N + hist}]")
    B = ctx.num_seqs
    _i32(ctx.cu_seqlens, "cu_seqlens", B + 1); _i32(ctx.state_slots, "state_slots", B)
    out = torch.empty(T, C, dtype=xc.dtype, device=xc.device)
    ws = ws_dt = None
    max_chunks = 0
    if chunk > 0:
        max_chunks = -(-T // chunk)
        ws = torch.empty(B * max_chunks, C, N, dtype=torch.float32, device=xc.device)
        ws_dt = torch.empty(B * max_chunks, C, dtype=torch.float32, device=xc.device)
    lib = library.core()
    _check(lib, lib.pico_selective_scan(_ptr(xc), _ptr(dt_pre), _ptr(dt_bias), _ptr(bc), bc.stride(0) if T > 1 else bc.shape[1],
                                        b_col, c_col, _ptr(a_log), _ptr(d), _ptr(z), z.stride(0) if T > 1 else z.shape[1], _dt(xc),
                                        _ptr(ctx.cu_seqlens), _ptr(ctx.state_slots), _ptr(state), state.shape[0], B, T, C, N, hist,
                                        _ptr(out), chunk, max_chunks, _ptr(ws), _ptr(ws_dt), _stream()))
    return out


def moe_router_top_softmax(x: torch.Tensor, w_router: torch.Tensor, bias: Optional[torch.Tensor], experts: int, top: int):
    """Router logits z = x w_router^T (+ bias on the first ``experts`` of them) in float32; the ``top`` largest of the
    experts' logits are chosen (the lowest index among equals), weights = softmax over the chosen logits.  Rows of
    w_router behind the experts' give further logits that take no part (returned with the others).
    Returns (experts int32 [T, top], weights float32 [T, top], z float32 [T, rows of w_router])."""
    _gpu(x, w_router, bias)
    T, D = x.shape
    rows = w_router.shape[0]
    if w_router.dtype != torch.float32 or w_router.dim() != 2 or w_router.shape[1] != D or not w_router.is_contiguous() or rows < experts:
        raise KernelError(f"moe_router_top_softmax: the router matrix must be contiguous float32 [>= {experts}, {D}]")
    _vec(bias, experts, "the router's bias")
    if x.stride(1) != 1:
        raise KernelError("moe_router_top_softmax: activations must have unit stride along the row")
    if not 1 <= top <= min(experts, MOE_MAX_TOP):
        raise KernelError(f"moe_router_top_softmax: {top} of {experts} experts per token (at most {MOE_MAX_TOP})")
    z = torch.empty(T, rows, dtype=torch.float32, device=x.device)
    chosen = torch.empty(T, top, dtype=torch.int32, device=x.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_moe_router_top_softmax(_ptr(x), x.stride(0) if T > 1 else D, _dt(x), _ptr(w_router), _ptr(bias), T,
                                                experts, rows - experts, D, top, _ptr(z), _ptr(chosen), _ptr(weights), _stream()))
    return chosen, weights, z


# ---- norms on what a sublayer returns; the stream's own norm ---------------------------------------------------------------
def _delta_like(resid, y, who):
    T, H = resid.shape
    if y.dim() == 3:
        if y.dtype != torch.float32:
            raise KernelError(f"{who}: a stack of partial sums must be float32")
    elif y.dim() != 2:
        raise KernelError(f"{who}: an output is [T, H] or a stack [S, T, H]")
    if tuple(y.shape[-2:]) != (T, H) or not y.is_contiguous():
        raise KernelError(f"{who}: an output must be contiguous and shaped like the residual stream")
    return y.shape[0] if y.dim() == 3 else 1


def norm_add(resid: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, copy_dtype: Optional[torch.dtype] = None,
             y2: Optional[torch.Tensor] = None, weight1: Optional[torch.Tensor] = None,
             weight2: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """resid (float32 [T, H], in place) += rms(y) * weight.  With ``y2``: y and y2 are each RMS-normed with their own
    weights (weight1, weight2), half their sum takes y's place.  y, y2: [T, H], or float32 stacks [S, T, H] whose slabs are
    added up first.  ``copy_dtype``: also returns the new rows in that dtype (what the next sublayer reads)."""
    _gpu(resid, y, weight, y2, weight1, weight2)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    _vec(weight, H, "norm weight")
    s1 = _delta_like(resid, y, "norm_add")
    s2 = 1
    if y2 is not None:
        s2 = _delta_like(resid, y2, "norm_add")
        if weight1 is None or weight2 is None:
            raise KernelError("norm_add: two outputs come with a weight each")
        _vec(weight1, H, "norm weight"); _vec(weight2, H, "norm weight")
    copy = torch.empty(T, H, dtype=copy_dtype, device=resid.device) if copy_dtype is not None else None
    lib = library.core()
    _check(lib, lib.pico_norm_add(_ptr(resid), _ptr(y), _dt(y), s1, _ptr(weight1), _ptr(y2), _dt(y2) if y2 is not None else F32, s2,
                                  _ptr(weight2), c_ll(T * H), _ptr(weight), c_float(eps), _ptr(copy),
                                  _DT[copy_dtype] if copy_dtype is not None else F32, T, H, _stream()))
    return copy


def stream_rmsnorm(resid: torch.Tensor, weight: torch.Tensor, eps: float, copy_dtype: Optional[torch.dtype] = None):
    """resid (float32 [T, H]) <- rms(resid) * weight in place; ``copy_dtype``: also returns the rows in that dtype."""
    _gpu(resid, weight)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    _vec(weight, H, "norm weight")
    copy = torch.empty(T, H, dtype=copy_dtype, device=resid.device) if copy_dtype is not None else None
    lib = library.core()
    _check(lib, lib.pico_stream_rmsnorm(_ptr(resid), _ptr(weight), c_float(eps), _ptr(copy),
                                        _DT[copy_dtype] if copy_dtype is not None else F32, T, H, _stream()))
    return copy


def cast_rows(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """A contiguous float32 tensor in the activations' dtype (float32: itself)."""
    _gpu(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("cast_rows: a contiguous float32 tensor")
    if dtype == torch.float32:
        return x
    out = torch.empty_like(x, dtype=dtype)
    lib = library.core()
    _check(lib, lib.pico_cast_rows(_ptr(x), _ptr(out), _DT[dtype], c_ll(x.numel()), _stream()))
    return out


# ---- what stands between the q/k/v product and an attention that norms its queries and keys --------------------------------
QK_NORM_NONE, QK_NORM_UNIT, QK_NORM_ROW = 0, 1, 2


def qk_norm_store(x: torch.Tensor, q_col: int, k_col: int, v_col: int, nq: int, nk: int, nv: int, dk: int, dv: int, maps: int,
                  norm_mode: int, wq: Optional[torch.Tensor], wk: Optional[torch.Tensor], eps: float,
                  cos_sin: Optional[torch.Tensor], rotary_dim: int, slots: Optional[torch.Tensor],
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor]) -> torch.Tensor:
    """RMS norm of the nq query and nk key units of dk entries in every row of x (QK_NORM_UNIT: every unit by itself,
    weights [dk]; QK_NORM_ROW: all units of a row at once, weights [nq * dk] and [nk * dk]), then the first ``rotary_dim``
    entries of every unit turned (entry i with i + rotary_dim / 2; ``cos_sin`` from ``rope_table``).  Returns the queries
    [T, nq * dk]; with ``maps`` > 1 (a head holds that many units) in the order (kv group, map, head in group).  Keys go
    to ``k_cache`` [pages, nk, P, dk] and columns v_col .. of x, as they are, to ``v_cache`` [pages, nv, dv, P] at
    ``slots`` (negative: nothing); without a cache only the queries are made."""
    _gpu(x, wq, wk, cos_sin, slots, k_cache, v_cache)
    T = x.shape[0]
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("qk_norm_store: x must be [T, columns] with unit stride along the row")
    if maps < 1 or nq % maps or nk % maps or (nq // maps) % (nk // maps):
        raise KernelError("qk_norm_store: query heads are a multiple of kv heads, and both hold whole maps")
    if x.shape[1] < max(q_col + nq * dk, k_col + nk * dk, v_col + nv * dv):
        raise KernelError("qk_norm_store: the rows do not hold q, k and v")
    if norm_mode != QK_NORM_NONE:
        n = dk if norm_mode == QK_NORM_UNIT else None
        _vec(wq, n or nq * dk, "the queries' norm weight"); _vec(wk, n or nk * dk, "the keys' norm weight")
        if wq is None or wk is None:
            raise KernelError("qk_norm_store: a norm needs its weights")
    if rotary_dim % 2 or not 0 <= rotary_dim <= dk:
        raise KernelError(f"qk_norm_store: {rotary_dim} turned entries do not fit a unit of {dk}")
    _check_table(cos_sin, T, rotary_dim // 2)
    pages = P = 0
    if k_cache is not None:
        pages, P = _check_cache2(k_cache, v_cache, nk, dk, dv, nv)
        if k_cache.dtype != x.dtype:
            raise KernelError("cache and activations differ in dtype")
        _i32(slots, "slots", T)
    q_out = torch.empty(T, nq * dk, dtype=x.dtype, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_qk_norm_store(_ptr(x), _dt(x), x.stride(0) if T > 1 else x.shape[1], q_col, k_col, v_col, nq, nk, nv, dk,
                                       dv, maps, norm_mode, _ptr(wq), _ptr(wk), c_float(eps),
                                       _ptr(cos_sin) if rotary_dim else None, rotary_dim, _ptr(slots), _ptr(q_out), _ptr(k_cache),
                                       _ptr(v_cache), T, P, pages, _stream()))
    return q_out


def diff_combine(a: torch.Tensor, lam: float, eps: float, mult: float, heads: int, kv_heads: int, dv: int,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """Two attention maps a head into one output: a float32 [T, 2 * heads * dv] in the order (kv group, map, head in group);
    o = a1 - lam * a2, over its root mean square (eps inside), times ``mult``.  Returns [T, heads * dv] in head order."""
    _gpu(a)
    T = a.shape[0]
    if a.dtype != torch.float32 or tuple(a.shape) != (T, 2 * heads * dv) or not a.is_contiguous() or heads % kv_heads:
        raise KernelError(f"diff_combine: the maps' outputs must be contiguous float32 [T, {2 * heads * dv}]")
    out = torch.empty(T, heads * dv, dtype=out_dtype, device=a.device)
    lib = library.core()
    _check(lib, lib.pico_diff_combine(_ptr(a), c_float(lam), c_float(eps), c_float(mult), _ptr(out), _DT[out_dtype], T, heads,
                                      kv_heads, dv, _stream()))
    return out


# ---- recurrent mixers with a matrix state: the delta rule, state-space duality ---------------------------------------------
DELTA_MAX_KEY_DIM = 512


def delta_prep(x: torch.Tensor, q_col: int, k_col: int, y: torch.Tensor, b_col: int, a_col: int, a2: torch.Tensor,
               dt_bias: torch.Tensor, a_log: torch.Tensor, qscale: float, heads: int, kv_heads: int, dk: int):
    """What enters the delta rule's walk, in float32: unit vectors q (times qscale) and k per q/k head [T, kv_heads * dk]
    from columns q_col .., k_col .. of x; decays g = exp(-exp(a_log_h) softplus(a2 (y[:, a_col : a_col + R]) + dt_bias))
    [T, heads * dk]; beta = sigmoid(y[:, b_col : b_col + heads]) [T, heads]."""
    _gpu(x, y, a2, dt_bias, a_log)
    T = x.shape[0]
    C, R = a2.shape
    if x.dim() != 2 or y.dim() != 2 or x.stride(1) != 1 or y.stride(1) != 1 or y.shape[0] != T or x.dtype != y.dtype:
        raise KernelError("delta_prep: x and y are [T, columns] of one dtype with unit stride along the row")
    if C != heads * dk or a2.dtype != x.dtype or not a2.is_contiguous() or heads % kv_heads:
        raise KernelError(f"delta_prep: a2 must be contiguous [{heads * dk}, R] of the activations' dtype")
    if x.shape[1] < max(q_col, k_col) + kv_heads * dk or y.shape[1] < max(b_col + heads, a_col + R):
        raise KernelError("delta_prep: the rows do not hold what is read")
    _vec(dt_bias, heads * dk, "the decay's bias"); _vec(a_log, heads, "A_log")
    dev = x.device
    qn = torch.empty(T, kv_heads * dk, dtype=torch.float32, device=dev)
    kn = torch.empty(T, kv_heads * dk, dtype=torch.float32, device=dev)
    g = torch.empty(T, heads * dk, dtype=torch.float32, device=dev)
    beta = torch.empty(T, heads, dtype=torch.float32, device=dev)
    lib = library.core()
    _check(lib, lib.pico_delta_prep(_ptr(x), x.stride(0) if T > 1 else x.shape[1], q_col, k_col, _ptr(y),
                                    y.stride(0) if T > 1 else y.shape[1], b_col, a_col, _dt(x), _ptr(a2), _ptr(dt_bias), _ptr(a_log),
                                    c_float(qscale), _ptr(qn), _ptr(kn), _ptr(g), _ptr(beta), T, heads, kv_heads, dk, R, _stream()))
    return qn, kn, g, beta


def ssd_prep(bc: torch.Tensor, b_col: int, c_col: int, n: int, y: torch.Tensor, dt_col: int, dt_bias: torch.Tensor,
             a_log: torch.Tensor, heads: int):
    """What enters a state-space walk, in float32: B and C (n columns each of bc from b_col, c_col) widened;
    dt = softplus(y[:, dt_col : dt_col + heads] + dt_bias) and the decay exp(-exp(a_log) dt), both [T, heads]."""
    _gpu(bc, y, dt_bias, a_log)
    T = bc.shape[0]
    if bc.dim() != 2 or y.dim() != 2 or bc.stride(1) != 1 or y.stride(1) != 1 or y.shape[0] != T or bc.dtype != y.dtype:
        raise KernelError("ssd_prep: bc and y are [T, columns] of one dtype with unit stride along the row")
    if bc.shape[1] < max(b_col, c_col) + n or y.shape[1] < dt_col + heads:
        raise KernelError("ssd_prep: the rows do not hold what is read")
    _vec(dt_bias, heads, "dt bias"); _vec(a_log, heads, "A_log")
    dev = bc.device
    bf = torch.empty(T, n, dtype=torch.float32, device=dev)
    cf = torch.empty(T, n, dtype=torch.float32, device=dev)
    g = torch.empty(T, heads, dtype=torch.float32, device=dev)
    dt = torch.empty(T, heads, dtype=torch.float32, device=dev)
    lib = library.core()
    _check(lib, lib.pico_ssd_prep(_ptr(bc), bc.stride(0) if T > 1 else bc.shape[1], b_col, c_col, n, _ptr(y),
                                  y.stride(0) if T > 1 else y.shape[1], dt_col, _dt(bc), _ptr(dt_bias), _ptr(a_log), _ptr(bf), _ptr(cf),
                                  _ptr(g), _ptr(dt), T, heads, _stream()))
    return bf, cf, g, dt


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, cu_seqlens: torch.Tensor,
               state_slots: torch.Tensor, state: torch.Tensor, num_seqs: int, heads: int, kv_heads: int, dk: int, dv: int,
               delta: bool = True, chunk: int = 0) -> torch.Tensor:
    """The walk S <- diag(g_t) S; u = beta_t (v_t - S^T k_t) (``delta``; else u = beta_t v_t); S <- S + k_t u^T;
    o_t = S^T q_t, for every sequence of the step from its state slot (``state`` float32 [slots, heads, dk, dv], updated in
    place).  q, k float32 [T, kv_heads * dk] (head h reads q/k head h // (heads // kv_heads)); v [T, >= heads * dv] (row
    stride free); g float32 [T, heads * dk] (a decay a key channel) or [T, heads] (one a head); beta float32 [T, heads].
    Returns o float32 [T, heads * dv].
    ``chunk`` > 0: sequences are cut into chunks of that many tokens that run side by side (every chunk from zero, which
    also yields the chunk's map of the state in front of it; a walk over the chunks' states; every chunk again from its
    true state): the same sums in another order."""
    _gpu(q, k, v, g, beta, cu_seqlens, state_slots, state)
    T = q.shape[0]
    for t, name in ((q, "q"), (k, "k")):
        if t.dtype != torch.float32 or tuple(t.shape) != (T, kv_heads * dk) or not t.is_contiguous():
            raise KernelError(f"delta_scan: {name} must be contiguous float32 [T, {kv_heads * dk}]")
    if v.dim() != 2 or v.shape[0] != T or v.stride(1) != 1 or v.shape[1] < heads * dv:
        raise KernelError("delta_scan: the rows do not hold the values")
    if g.dtype != torch.float32 or not g.is_contiguous() or tuple(g.shape) not in ((T, heads * dk), (T, heads)):
        raise KernelError("delta_scan: the decays are contiguous float32, one a key channel or one a head")
    g_channels = tuple(g.shape) == (T, heads * dk)
    if beta.dtype != torch.float32 or tuple(beta.shape) != (T, heads) or not beta.is_contiguous():
        raise KernelError(f"delta_scan: beta must be contiguous float32 [T, {heads}]")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dk, dv) or not state.is_contiguous():
        raise KernelError(f"delta_scan: the state must be contiguous float32 [slots, {heads}, {dk}, {dv}]")
    if dk > DELTA_MAX_KEY_DIM or heads % kv_heads:
        raise KernelError(f"delta_scan: at most {DELTA_MAX_KEY_DIM} key channels a head; heads a multiple of q/k heads")
    _i32(cu_seqlens, "cu_seqlens", num_seqs + 1)
    _i32(state_slots, "state_slots", num_seqs)
    out = torch.empty(T, heads * dv, dtype=torch.float32, device=q.device)
    ws_s = ws_p = None
    max_chunks = 0
    if chunk > 0:
        max_chunks = -(-T // chunk)
        ws_s = torch.empty(num_seqs * max_chunks, heads, dk, dv, dtype=torch.float32, device=q.device)
        ws_p = torch.empty(num_seqs * max_chunks, heads, dk, dk if delta else 1, dtype=torch.float32, device=q.device)
    lib = library.core()
    _check(lib, lib.pico_delta_scan(_ptr(q), _ptr(k), _ptr(v), v.stride(0) if T > 1 else v.shape[1], _dt(v), _ptr(g),
                                    1 if g_channels else 0, _ptr(beta), _ptr(cu_seqlens), _ptr(state_slots), _ptr(state), _ptr(out),
                                    num_seqs, T, heads, kv_heads, dk, dv, state.shape[0], 1 if delta else 0, chunk, max_chunks, _ptr(ws_s),
                                    _ptr(ws_p), _stream()))
    return out


def gated_group_norm(y: torch.Tensor, x: torch.Tensor, z: torch.Tensor, d: torch.Tensor, weight: torch.Tensor, eps: float,
                     heads: int, dv: int, groups: int) -> torch.Tensor:
    """((y + d_h x) * silu(z)) RMS-normed in ``groups`` equal parts of the row, times ``weight``; y float32 [T, heads * dv];
    x, z [T, >= heads * dv] of the activations' dtype (row strides free); returns [T, heads * dv] of that dtype."""
    _gpu(y, x, z, d, weight)
    T, n = y.shape[0], heads * dv
    if y.dtype != torch.float32 or tuple(y.shape) != (T, n) or not y.is_contiguous():
        raise KernelError(f"gated_group_norm: y must be contiguous float32 [T, {n}]")
    for t in (x, z):
        if t.dim() != 2 or t.shape[0] != T or t.stride(1) != 1 or t.shape[1] < n or t.dtype != x.dtype:
            raise KernelError("gated_group_norm: x and z are [T, >= heads * dv] of one dtype with unit stride along the row")
    if groups < 1 or n % groups:
        raise KernelError(f"gated_group_norm: {n} entries are not {groups} equal parts")
    _vec(d, heads, "D"); _vec(weight, n, "norm weight")
    out = torch.empty(T, n, dtype=x.dtype, device=x.device)
    lib = library.core()
    _check(lib, lib.pico_gated_group_norm(_ptr(y), _ptr(x), x.stride(0) if T > 1 else x.shape[1], _ptr(z),
                                          z.stride(0) if T > 1 else z.shape[1], _dt(x), _ptr(d), _ptr(weight), c_float(eps), _ptr(out),
                                          T, heads, dv, groups, _stream()))
    return out
