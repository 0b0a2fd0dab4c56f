"""A plain, slow implementation of the Dikolix decoder: whole sequences, no cache, one function per mechanism,
float64 by default.  It shares no code with the engine; the tests compare the engine with it.

A model is (config, tensors): ``config`` is what config.json holds, ``tensors`` maps checkpoint names to torch
tensors.  Notation: n tokens, width D, heads H.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * weight + bias over the last axis; var is the mean squared deviation."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ---------------------------------------------------------------------------------------------------------------
# embedding
# ---------------------------------------------------------------------------------------------------------------
def pair_rows(tokens: List[int], big: dict) -> List[int]:
    """The row of the pair table for every token: hashed from (previous token, token); the first token has no
    previous one and takes the table's last row."""
    rows = []
    for i, t in enumerate(tokens):
        if i == 0:
            rows.append(big["buckets"])
        else:
            rows.append((tokens[i - 1] * big["mul_prev"] + t * big["mul_cur"]) % big["buckets"])
    return rows


def embed(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype) -> torch.Tensor:
    x = tensors["embed"].to(dtype)[tokens]
    big = (config.get("embedding") or {}).get("bigram")
    if big:
        x = x + tensors["bigram"].to(dtype)[pair_rows(tokens, big)]
    return x


# ---------------------------------------------------------------------------------------------------------------
# rotation
# ---------------------------------------------------------------------------------------------------------------
def rotation_frequencies(rot: dict):
    """(frequencies [dims / 2], factor on cosine and sine)."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    s, L = float(sc["factor"]), float(sc["original"])

    def pair_index(turns: float) -> float:
        return dims * math.log(L / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_index(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / s * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(s) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict, layout: str) -> torch.Tensor:
    """x [n, heads, d]: the first ``dims`` entries of every head are turned by position * f_i, the rest passes.
    layout "pairs": entry 2i goes with 2i + 1;  "halves": entry i goes with i + dims / 2."""
    f, mag = rotation_frequencies(rot)
    dims = rot["dims"]
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    out = x.clone()
    if layout == "pairs":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., 0:dims // 2], x[..., dims // 2:dims]
        out[..., 0:dims // 2] = a * c - b * s
        out[..., dims // 2:dims] = b * c + a * s
    return out


# ---------------------------------------------------------------------------------------------------------------
# mixers
# ---------------------------------------------------------------------------------------------------------------
def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    """Queries and keys/values through low-rank latents; every head's key is [its own unrotated part | one rotated
    part shared by all heads]; causal softmax."""
    n = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = dict(m["rot"], dims=r)
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(n, H, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], positions, rot, "pairs")
    kv = h @ w["dkv"].T
    c = rms_norm(kv[:, :R], w["dkv.norm"], eps)
    k_rot = rotate(kv[:, None, R:], positions, rot, "pairs")[:, 0]            # [n, r]
    k_plain = (c @ w["uk"].T).view(n, H, d)
    v = (c @ w["uv"].T).view(n, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    mask = positions[None, :] <= positions[:, None]
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(n, H * dv)
    return o @ w["o"].T


def causal_conv(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, history: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [n, C]; weight [C, taps], the last column is the current token's; zeros (or ``history`` [taps - 1, C]) before."""
    taps = weight.shape[1]
    pad = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype) if history is None else history
    xp = torch.cat([pad, x], 0)
    out = bias[None, :].expand(x.shape[0], -1).clone()
    for j in range(taps):
        out = out + xp[j:j + x.shape[0]] * weight[:, j][None, :]
    return out


def selective_scan(x, dt, A, B, C, D, state=None):
    """x, dt [n, C]; A [C, N]; B, C [n, N]; D [C].  S <- exp(dt A) S + dt x B;  y = S . C + D x."""
    n, ch = x.shape
    S = torch.zeros(ch, A.shape[1], dtype=x.dtype) if state is None else state.clone()
    ys = []
    for t in range(n):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        ys.append(S @ C[t] + D * x[t])
    return torch.stack(ys), S


def mamba(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ w["in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w["conv"], w["conv.b"]))
    dbc = x @ w["x"].T
    dt = softplus(dbc[:, :R] @ w["dt"].T + w["dt.b"])
    y, _ = selective_scan(x, dt, -torch.exp(w["A_log"]), dbc[:, R:R + N], dbc[:, R + N:R + 2 * N], w["D"])
    return (y * silu(z)) @ w["o"].T


def retention_recurrence(q, k, v, decay, state=None):
    """q, k [n, H, dk], v [n, H, dv], decay [H].  S <- decay S + k v^T;  o = S^T q."""
    n, H, dk = q.shape
    S = torch.zeros(H, dk, v.shape[2], dtype=q.dtype) if state is None else state.clone()
    out = []
    for t in range(n):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hkv,hk->hv", S, q[t]))
    return torch.stack(out), S


def retention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, positions: torch.Tensor,
              margins_out: Optional[List] = None) -> torch.Tensor:
    n = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, dk)
    k = (h @ w["k"].T).view(n, H, dk)
    v = (h @ w["v"].T).view(n, H, dv)
    if m.get("rot"):
        q, k = rotate(q, positions, m["rot"], "halves"), rotate(k, positions, m["rot"], "halves")
    k = k * dk ** -0.5
    o, _ = retention_recurrence(q, k, v, torch.tensor(m["decay"], dtype=h.dtype))
    if margins_out is not None:
        # where a head's output cancels to a small part of what went into it, a rounding decides its direction and the
        # norm behind it blows that up: 4 |o| / (|q| * the largest |k| |v| so far), the least over the heads
        kv = torch.cummax(k.norm(dim=-1) * v.norm(dim=-1), 0).values
        margins_out.append((4.0 * o.norm(dim=-1) / (q.norm(dim=-1) * kv + 1e-300)).min(-1).values)
    o = rms_norm(o, None, eps).reshape(n, H * dv)
    return (o * silu(h @ w["g"].T)) @ w["o"].T


# ---------------------------------------------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------------------------------------------
def gated_mlp(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor, top: int):
    """(experts [n, top], weights [n, top]): the largest logits, softmax over the chosen logits only."""
    z = h @ router.T + bias
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1), z


def route_margin(z: torch.Tensor, top: int) -> torch.Tensor:
    """Per token: how far the last chosen logit lies above the first rejected one, in units of the row's spread
    (infinite where every expert is chosen).  A small margin means that a rounding may choose otherwise."""
    if top >= z.shape[-1]:
        return torch.full((z.shape[0],), float("inf"), dtype=z.dtype)
    val, _ = torch.topk(z, top + 1, dim=-1)
    return (val[:, top - 1] - val[:, top]) / (z.std(-1) + 1e-12)


def moe(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict, margins_out: Optional[List] = None) -> torch.Tensor:
    E, top = f["router"]["experts"], f["router"]["top"]
    idx, wt, z = route(h, w["router"], w["router.b"], top)
    if margins_out is not None:
        margins_out.append(route_margin(z, top))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wt[t, j] * gated_mlp(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if f.get("shared"):
        sh = gated_mlp(h, w["shared.gate"], w["shared.up"], w["shared.down"])
        out = out + sh * torch.sigmoid(h @ w["shared.sg"].T)
    return out


# ---------------------------------------------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------------------------------------------
def sub(tensors: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in tensors.items() if k.startswith(prefix)}


def run_order(config: dict) -> List[tuple]:
    """(layer, whether the embedding output joins in front of it) in the order the layers run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop or loop["times"] <= 1:
        return [(i, False) for i in range(n)]
    out = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        out += [(i, p > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return out + [(i, False) for i in range(loop["stop"], n)]


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, dtype=torch.float64, layers_out: Optional[List] = None,
            margins_out: Optional[List] = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence.  ``layers_out`` gets the residual stream after every layer run,
    ``margins_out`` every routed layer run's margins of the choice (``route_margin``)."""
    tokens = [int(t) for t in tokens]
    eps, mult = config["norm"]["eps"], config.get("residual_mult", 1.0)
    pos = torch.arange(len(tokens))
    x0 = embed(config, tensors, tokens, dtype)
    x = x0.clone()
    for i, rejoin in run_order(config):
        l = config["layers"][i]
        w = sub(tensors, f"l{i}.", dtype)
        if rejoin:
            x = x + x0
        h = layer_norm(x, w["norm1"], w["norm1.b"], eps)
        mw = {k[4:]: v for k, v in w.items() if k.startswith("mix.")}
        if l["type"] == "latent_attention":
            a = latent_attention(h, mw, l["mixer"], eps, pos)
        elif l["type"] == "mamba1":
            a = mamba(h, mw, l["mixer"])
        elif l["type"] == "retention":
            a = retention(h, mw, l["mixer"], eps, pos, margins_out)
        else:
            raise ValueError(l["type"])
        x = x + mult * w["ls1"] * a
        if l.get("mlp"):
            h = layer_norm(x, w["norm2"], w["norm2.b"], eps)
            fw = {k[4:]: v for k, v in w.items() if k.startswith("mlp.")}
            x = x + mult * w["ls2"] * moe(h, fw, l["mlp"], margins_out)
        if layers_out is not None:
            layers_out.append(x.clone())
    h = layer_norm(x, tensors["final.norm"].to(dtype), tensors["final.norm.b"].to(dtype), eps)
    return h @ tensors["embed"].to(dtype).T


# ---------------------------------------------------------------------------------------------------------------
# random models
# ---------------------------------------------------------------------------------------------------------------
def tensor_shapes(config: dict) -> Dict[str, tuple]:
    D, V = config["width"], config["vocab"]
    out = {"embed": (V, D), "final.norm": (D,), "final.norm.b": (D,)}
    big = (config.get("embedding") or {}).get("bigram")
    if big:
        out["bigram"] = (big["buckets"] + 1, D)
    for i, l in enumerate(config["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out.update({p + "norm1": (D,), p + "norm1.b": (D,), p + "ls1": (D,)})
        if l["type"] == "latent_attention":
            H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            out.update({p + "mix.dq": (m["q_rank"], D), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (H * (d + r), m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"] + r, D), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (H * d, m["kv_rank"]), p + "mix.uv": (H * dv, m["kv_rank"]), p + "mix.o": (D, H * dv)})
        elif l["type"] == "mamba1":
            I, N, R = m["inner"], m["state"], m["dt_rank"]
            out.update({p + "mix.in": (2 * I, D), p + "mix.conv": (I, m["conv"]), p + "mix.conv.b": (I,), p + "mix.x": (R + 2 * N, I),
                        p + "mix.dt": (I, R), p + "mix.dt.b": (I,), p + "mix.A_log": (I, N), p + "mix.D": (I,), p + "mix.o": (D, I)})
        else:
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * dk, D), p + "mix.k": (H * dk, D), p + "mix.v": (H * dv, D), p + "mix.g": (H * dv, D),
                        p + "mix.o": (D, H * dv)})
        f = l.get("mlp")
        if f:
            out.update({p + "norm2": (D,), p + "norm2.b": (D,), p + "ls2": (D,)})
            F = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (F, D), p + f"mlp.e{e}.up": (F, D), p + f"mlp.e{e}.down": (D, F)})
            out.update({p + "mlp.router": (f["router"]["experts"], D), p + "mlp.router.b": (f["router"]["experts"],)})
            if f.get("shared"):
                S = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (S, D), p + "mlp.shared.up": (S, D), p + "mlp.shared.down": (D, S),
                            p + "mlp.shared.sg": (1, D)})
    return out


def random_model(config: dict, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of the right shapes, large enough that every mechanism moves the logits."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.split(".")[-1]
        if name.endswith(".b") and "norm" in name:
            t = 0.1 * torch.randn(shape, generator=g)
        elif last in ("norm1", "norm2", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last in ("ls1", "ls2"):
            t = 0.5 + 0.5 * torch.rand(shape, generator=g)
        elif last == "A_log":
            t = torch.log(0.5 + 4.0 * torch.rand(shape, generator=g))
        elif name.endswith("dt.b"):
            t = torch.log(torch.expm1(0.01 + 0.2 * torch.rand(shape, generator=g)))
        elif name.endswith("conv.b") or name.endswith("router.b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = torch.randn(shape, generator=g) * shape[1] ** -0.5
        elif name in ("embed", "bigram"):
            t = torch.randn(shape, generator=g)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=g) * shape[-1] ** -0.5
        else:
            t = 1.5 * torch.randn(shape, generator=g) * shape[-1] ** -0.5
        out[name] = t.to(dtype)
    return out
