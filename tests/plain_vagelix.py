"""A plain, slow implementation of the Vagelix decoder: whole sequences, no cache, float64 on the CPU, one function per
mechanism, written from the design's equations and sharing no code with the package.

Notation: T tokens at positions 0 .. T - 1, width D, eps the model's norm constant.  A weight dict maps checkpoint names
('l3.mix.q', 'embed.norm', ..) to tensors; linear weights are [out, in] and applied as x W^T.

  model:   x = rms(E[token]) w_e; per layer x += rms(mixer(x)) w_1, then (if the layer has a feed-forward)
           x += rms(ff(x)) w_2; logits = (rms(x) w_f) E^T.  The sublayers read x itself.
  A layer with weights_of = j runs layer j's tensors (and its own state).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64

# A yardstick for what rounding alone does: with ``forward(..., rounding=f)`` every activation that passes from one part
# to the next (a product's output, a convolution's, an attention's, the stream as a sublayer reads it) goes through f.
_rounding = None


def act(x: torch.Tensor) -> torch.Tensor:
    return x if _rounding is None else _rounding(x)


def stochastic_bfloat16(seed: int):
    """A rounding to bfloat16's 8 significant bits that rounds up or down at random, in proportion (unbiased); draws
    with different seeds are independent."""
    g = torch.Generator().manual_seed(seed)

    def f(x: torch.Tensor) -> torch.Tensor:
        ulp = torch.exp2(torch.floor(torch.log2(x.abs().clamp_min(1e-300))) - 7)
        return torch.floor(x / ulp + torch.rand(x.shape, generator=g, dtype=x.dtype)) * ulp
    return f


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def kv_head_of(h: int, heads: int, kv_heads: int) -> int:
    return h // (heads // kv_heads)


# ---- differential attention ------------------------------------------------------------------------------------------
def query_temperature(p: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((p + 1) // every + 1)


def diff_lambda(lq1, lk1, lq2, lk2, diff: float) -> float:
    return float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + diff)


def differential_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, first_pos: int = 0) -> torch.Tensor:
    """h [T, D] -> [T, D].  q rows are laid out head by head as [map 1 | map 2] (dim each), k likewise per kv head; both
    maps attend over the same values.  Per head and map q and k are RMS-normed over dim with one weight; no rotation;
    q times the temperature of its position; causal softmax; o = a1 - lambda a2, over its root mean square, (1 - diff)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = act(h @ w["q"].T).view(T, H, 2, d)
    k = act(h @ w["k"].T).view(T, G, 2, d)
    v = act(h @ w["v"].T).view(T, G, dv)
    q = act(rms(q, eps) * w["q.norm"])
    k = act(rms(k, eps) * w["k.norm"])
    temp = torch.tensor([query_temperature(first_pos + t, m["q_temp"]["coef"], m["q_temp"]["every"]) if m.get("q_temp") else 1.0
                         for t in range(T)], dtype=h.dtype)
    q = q * temp.view(T, 1, 1, 1)
    lam = diff_lambda(w["lq1"], w["lk1"], w["lq2"], w["lk2"], m["diff"])
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        g = kv_head_of(hh, H, G)
        maps = []
        for mp in range(2):
            s = (q[:, hh, mp] @ k[:, g, mp].T) * m["scale"]
            s = s.masked_fill(~causal, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hh] = rms(o, eps) * (1.0 - m["diff"])
    return act(act(out.reshape(T, H * dv)) @ w["o"].T)


# ---- the parallel mixer's left side: chunked attention with a sink ---------------------------------------------------
def rotate_half(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]: entry i < dims / 2 is paired with entry i + dims / 2 and the pair turned by p base^(-2i / dims)."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype).view(-1, 1, 1) * f
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def chunk_visible(i: int, j: int, size: int) -> bool:
    return j <= i and (size <= 0 or i // size == j // size)


def chunked_sink_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, first_pos: int = 0) -> torch.Tensor:
    """q = Wq h + bq, k = Wk h + bk; the values are k as projected.  q and k are RMS-normed over their whole rows (all
    heads at once) with weights of that size, then the first rot.dims entries of every head are turned.  Position i sees
    j <= i of its own chunk; p_j = exp(s_j) / (1 + sum exp(s)); head outputs times sigmoid(Wg h), one number a head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = act(h @ w["q"].T + w["q.b"])
    k = act(h @ w["k"].T + w["k.b"])
    v = k.view(T, G, d)
    assert dv == d, "the values are the keys: their sizes are one"
    q = (rms(q, eps) * w["q.norm"]).view(T, H, d)
    kn = (rms(k, eps) * w["k.norm"]).view(T, G, d)
    pos = torch.arange(first_pos, first_pos + T)
    rot = m.get("rot") or {}
    q = act(rotate_half(q, pos, rot.get("dims", 0), rot.get("base", 1.0)))
    kn = act(rotate_half(kn, pos, rot.get("dims", 0), rot.get("base", 1.0)))
    size = (m.get("mask") or {}).get("size", 0)
    vis = torch.tensor([[chunk_visible(first_pos + i, first_pos + j, size) for j in range(T)] for i in range(T)])
    gate = torch.sigmoid(act(h @ w["g"].T))                             # [T, H]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hh in range(H):
        g = kv_head_of(hh, H, G)
        s = (q[:, hh] @ kn[:, g].T) * m["scale"]
        e = torch.where(vis, torch.exp(s), torch.zeros_like(s))
        p = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, hh] = (p @ v[:, g]) * gate[:, hh:hh + 1]
    return act(act(out.reshape(T, H * dv)) @ w["o"].T)


# ---- short causal convolution ----------------------------------------------------------------------------------------
def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor] = None,
                history: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, C], taps [C, K] (the last column is the current token's); inputs before the start are zero, or ``history``
    [K - 1, C] (oldest first)."""
    T, C = x.shape
    K = taps.shape[1]
    past = torch.zeros(K - 1, C, dtype=x.dtype) if history is None else history
    xx = torch.cat([past, x], dim=0)
    y = torch.zeros_like(x)
    for j in range(K):
        y += xx[j:j + T] * taps[:, j]
    return y if bias is None else y + bias


# ---- the parallel mixer's right side: the gated delta rule -----------------------------------------------------------
def delta_rule_scan(q, k, v, g, beta, S0=None):
    """q, k [T, H, dk] (already per head), v [T, H, dv], g [T, H, dk] decays, beta [T, H].  Per head, in this order:
    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns (o [T, H, dv], S [H, dk, dv])."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=q.dtype) if S0 is None else S0.clone()
    o = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        S = S * g[t].unsqueeze(-1)
        u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
        S = S + torch.einsum("hk,hv->hkv", k[t], u)
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return o, S


def gated_delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = act(silu(causal_conv(act(h @ w["q"].T), w["q.conv"]))).view(T, G, dk)
    k = act(silu(causal_conv(act(h @ w["k"].T), w["k.conv"]))).view(T, G, dk)
    v = act(silu(causal_conv(act(h @ w["v"].T), w["v.conv"]))).view(T, H, dv)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q = unit(q) * dk ** -0.5
    k = unit(k)
    idx = torch.tensor([kv_head_of(i, H, G) for i in range(H)])
    q, k = q[:, idx], k[:, idx]
    beta = torch.sigmoid(act(h @ w["b"].T))                                               # [T, H]
    step = softplus(act(h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, dk)
    g = torch.exp(-torch.exp(w["A_log"]).view(1, H, 1) * step)
    o, _ = delta_rule_scan(q, k, v, g, beta)
    o = rms(o, eps) * w["norm"]
    o = o * torch.sigmoid(act(act(h @ w["g1"].T) @ w["g2"].T)).view(T, H, dv)
    return act(act(o.reshape(T, H * dv)) @ w["o"].T)


def parallel_mixer(h, w, m, eps, first_pos: int = 0):
    """Both sides read h; half the sum of their outputs, each RMS-normed over the width with its own weight first."""
    sub = lambda side: {n[len(side) + 1:]: t for n, t in w.items() if n.startswith(side + ".")}
    left = chunked_sink_attention(h, sub("left"), m["left"], eps, first_pos)
    right = gated_delta_mixer(h, sub("right"), m["right"], eps)
    return 0.5 * (rms(left, eps) * w["left.out"] + rms(right, eps) * w["right.out"])


# ---- state-space duality mixer -----------------------------------------------------------------------------------------
def ssd_scan(x, B, C, dt, a, D, S0=None):
    """x [T, H, dv], B, C [T, H, N] (already per head), dt [T, H], a [H] = exp(A_log), D [H].
    S_t = exp(-a dt) S_(t-1) + dt B_t x_t^T  (N x dv);  y_t = S_t^T C_t + D x_t."""
    T, H, dv = x.shape
    N = B.shape[-1]
    S = torch.zeros(H, N, dv, dtype=x.dtype) if S0 is None else S0.clone()
    y = torch.zeros_like(x)
    for t in range(T):
        S = S * torch.exp(-a * dt[t]).view(H, 1, 1) + torch.einsum("hn,hv->hnv", B[t] * dt[t].unsqueeze(-1), x[t])
        y[t] = torch.einsum("hnv,hn->hv", S, C[t]) + D.view(H, 1) * x[t]
    return y, S


def mamba2_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, dv, N, G, ng = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * dv
    y = act(h @ w["in"].T)
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    xbc = act(silu(causal_conv(xbc, w["conv"], w["conv.b"])))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    idx = torch.tensor([kv_head_of(i, H, G) for i in range(H)])
    dt = softplus(dt + w["dt_bias"])
    yy, _ = ssd_scan(x, B[:, idx], C[:, idx], dt, torch.exp(w["A_log"]), w["D"])
    yy = yy.reshape(T, inner) * silu(z)
    yy = rms(yy.view(T, ng, inner // ng), eps).reshape(T, inner) * w["norm"]
    return act(act(yy) @ w["o"].T)


# ---- feed-forward, layers, model -------------------------------------------------------------------------------------
def dense_mlp(h, w):
    return act(act(silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T)


def weight_owner(layers: List[dict], i: int) -> int:
    while layers[i].get("weights_of") is not None:
        i = layers[i]["weights_of"]
    return i


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=F64, trace: Optional[list] = None,
            rounding=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  ``trace``: a list that receives the stream after every layer.
    ``rounding``: a function that every activation between the parts goes through (the stream itself stays as it is; what
    a sublayer reads of it is rounded)."""
    global _rounding
    _rounding = rounding
    try:
        return _forward(cfg, weights, tokens, dtype, trace)
    finally:
        _rounding = None


def _forward(cfg, weights, tokens, dtype, trace):
    W = {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in weights.items()}
    eps = cfg["norm"]["eps"]
    x = rms(W["embed"][torch.tensor(tokens)], eps) * W["embed.norm"]
    for i, layer in enumerate(cfg["layers"]):
        j = weight_owner(cfg["layers"], i)
        lw = {n[len(f"l{j}."):]: t for n, t in W.items() if n.startswith(f"l{j}.")}
        mw = {n[4:]: t for n, t in lw.items() if n.startswith("mix.")}
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            y = differential_attention(act(x), mw, m, eps)
        elif kind == "parallel":
            y = parallel_mixer(act(x), mw, m, eps)
        elif kind == "mamba2":
            y = mamba2_mixer(act(x), mw, m, eps)
        else:
            raise ValueError(f"unknown mixer {kind!r}")
        x = x + rms(y, eps) * lw["norm1"]
        if layer.get("mlp"):
            x = x + rms(dense_mlp(act(x), {n[4:]: t for n, t in lw.items() if n.startswith("mlp.")}), eps) * lw["norm2"]
        if trace is not None:
            trace.append(x.clone())
    return act(rms(x, eps) * W["final.norm"]) @ W["embed"].T


# ---- random models -----------------------------------------------------------------------------------------------------
def tensor_shapes(cfg: dict, decay_rank: int = 6, gate_rank: int = 5) -> Dict[str, tuple]:
    """Name -> shape of every tensor a model of this configuration holds (layers with weights_of hold none)."""
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "embed.norm": (D,), "final.norm": (D,)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (D,)
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * 2 * d, D), p + "mix.k": (G * 2 * d, D), p + "mix.v": (G * dv, D), p + "mix.o": (D, H * dv),
                        p + "mix.q.norm": (d,), p + "mix.k.norm": (d,)})
            out.update({p + "mix." + n: (d,) for n in ("lq1", "lk1", "lq2", "lk2")})
        elif layer["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, d = a["heads"], a["kv_heads"], a["dim"]
            q = p + "mix.left."
            out.update({q + "q": (H * d, D), q + "q.b": (H * d,), q + "k": (G * d, D), q + "k.b": (G * d,), q + "q.norm": (H * d,),
                        q + "k.norm": (G * d,), q + "g": (H, D), q + "o": (D, H * d), q + "out": (D,)})
            H, G, d, dv, K = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            q = p + "mix.right."
            out.update({q + "q": (G * d, D), q + "q.conv": (G * d, K), q + "k": (G * d, D), q + "k.conv": (G * d, K),
                        q + "v": (H * dv, D), q + "v.conv": (H * dv, K), q + "b": (H, D), q + "A_log": (H,), q + "norm": (dv,),
                        q + "a1": (decay_rank, D), q + "a2": (H * d, decay_rank), q + "dt_bias": (H * d,),
                        q + "g1": (gate_rank, D), q + "g2": (H * dv, gate_rank), q + "o": (D, H * dv), q + "out": (D,)})
        else:
            H, dv, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, C = H * dv, H * dv + 2 * G * N
            out.update({p + "mix.in": (inner + C + H, D), p + "mix.conv": (C, K), p + "mix.conv.b": (C,), p + "mix.dt_bias": (H,),
                        p + "mix.A_log": (H,), p + "mix.D": (H,), p + "mix.norm": (inner,), p + "mix.o": (D, inner)})
        if layer.get("mlp"):
            F = layer["mlp"]["ff"]
            out.update({p + "norm2": (D,), p + "mlp.gate": (F, D), p + "mlp.up": (F, D), p + "mlp.down": (D, F)})
    return out


def random_model(cfg: dict, seed: int, decay_rank: int = 6, gate_rank: int = 5) -> Dict[str, torch.Tensor]:
    """Random bfloat16 tensors for ``cfg``: matrices N(0, 1 / sqrt(in)), norm weights around 1, what enters a recurrence
    of a size that makes decays and gates neither 0 nor 1."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, decay_rank, gate_rank).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2", "out") or name in ("embed.norm", "final.norm"):
            t = 1.0 + 0.3 * (2 * torch.rand(shape, generator=g) - 1)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif last in ("A_log", "dt_bias", "D", "b") and len(shape) == 1:
            t = 0.7 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16)
    return out
