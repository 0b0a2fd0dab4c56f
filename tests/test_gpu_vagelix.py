"""The Vagelix decoder in the engine against the plain implementation: each mechanism's kernel alone, then whole
prompts, decoding through the cache and the state, portions down to two tokens, mixed batches in a small pool with few
state slots, keys that stand out at the edges of chunks and far back, long decoding, and greedy generation through the
entry point."""
import math
import random
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_vagelix as P
from gpu_util import DEV, paged_cache
from vagelix_configs import CONFIGS, attention, config, mamba2, model_dir, parallel, tensors_of, write_model

pytestmark = pytest.mark.gpu

# rms of a position's error over its logits (mean taken off), in units of the logits' own rms there
BOUND = {"float32": 3e-5, "bfloat16": 8e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
PAGE = {"a": 16, "b": 8, "c": 32, "d": 16}
F = torch.float64


def row_errors(got, want):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


_plain = {}
YARD_DRAWS = 8


def plain_logits(name, tokens, cfg=None, tensors=None):
    key = (name, tuple(tokens))
    if key not in _plain:
        _plain[key] = P.forward(cfg or CONFIGS[name], tensors or tensors_of(name), tokens).numpy()
    return _plain[key]


def yardstick(name, tokens, dtype, cfg=None, tensors=None):
    """What rounding alone does to every position's logits, in the units of ``row_errors``: the plain implementation
    with the rounding in question against itself in float64.  float32: all of it in float32 (other orders of summation
    than the engine's).  bfloat16: every activation between the parts rounded to 8 bits, up or down at random; the
    largest of a few draws.  Where a norm divides by something small a position's yardstick is many times the usual."""
    key = (name, tuple(tokens), dtype)
    if key not in _plain:
        cfg, tensors, want = cfg or CONFIGS[name], tensors or tensors_of(name), plain_logits(name, tokens, cfg, tensors)
        if dtype == "float32":
            draws = [P.forward(cfg, tensors, tokens, dtype=torch.float32).numpy().astype(np.float64)]
        else:
            draws = [P.forward(cfg, tensors, tokens, rounding=P.stochastic_bfloat16(100 + i)).numpy() for i in range(YARD_DRAWS)]
        _plain[key] = np.max([row_errors(d, want) for d in draws], axis=0)
    return _plain[key]


def replay(model, dtype, steps, max_tokens, page_size=16, max_live=4):
    """Run ``steps`` ([(entries, end)], entries [(id, tokens, want)]) through the engine's trace replayer; returns
    {(id, position): logits row} and the replayer."""
    from pico_vllm_amd.engine.replay import TraceReplayer
    rp = TraceReplayer(model, dtype, max_tokens, page_size, max_live)
    fed, rows = {}, {}
    for k, (entries, end) in enumerate(steps):
        out = rp.run_step({"step": k, "entries": [{"id": r, "tokens": t, "want": list(w)} for r, t, w in entries], "end": list(end)})
        at = 0
        for r, t, w in entries:
            for x in w:
                rows[(r, fed.get(r, 0) + x)] = out[at]
                at += 1
            fed[r] = fed.get(r, 0) + len(t)
        for r in end:
            fed.pop(r, None)
        rp.runner.manager.check()
    return rows, rp


# A position's error may be a few times what rounding alone does there (one float32 run of the plain implementation, or
# the largest of a few bfloat16 draws: themselves random), and never less than the floor is asked of it.  Where a norm
# divides by what is left of a cancellation (the first token's read-out q . k of the delta rule, the difference of the two
# maps) a rounding decides a sign: one draw in ten or twenty then lies at ten times the others, and a handful of draws need
# not show it.  So one position in fifty (at least one a comparison) may lie over its limit, up to CAP; a fault of the
# engine (a wrong key, a lost state) moves whole stretches of positions.
OVER_YARDSTICK = {"float32": 5.0, "bfloat16": 3.0}
CAP = {"float32": 1e-3, "bfloat16": 2.5}


def compare(name, dtype, rows, reqs, bound=None, cfg=None, tensors=None):
    floor = BOUND[dtype] if bound is None else bound
    errs, over, yards = [], [], []
    for (rid, pos), got in rows.items():
        toks = reqs[rid.split("#")[0]]
        e = float(row_errors(got[None], plain_logits(name, toks, cfg, tensors)[pos][None])[0])
        errs.append(e)
        yards.append(float(yardstick(name, toks, dtype, cfg, tensors)[pos]))
        limit = max(floor, OVER_YARDSTICK[dtype] * yards[-1])
        if not e <= limit:
            over.append(f"{rid} position {pos}: {e:.3g} > {limit:.3g}")
            assert e <= CAP[dtype], f"{name} {dtype}: {over[-1]}"
    assert len(over) <= max(1, len(errs) // 50), f"{name} {dtype}: {over}"
    if len(errs) >= 5:
        # the median position: half the floor, or (a model that rounding moves more) what the median yardstick says
        assert np.median(errs) <= max(floor / 2, np.median(yards)), f"{name} {dtype}: median {np.median(errs):.3g}"


def requests(vocab, lengths, seed=0):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def cut(tokens, sizes, tail=0):
    out, at, k = [], 0, 0
    body = len(tokens) - tail
    while at < body:
        n = min(sizes[k % len(sizes)], body - at)
        out.append(n)
        at += n
        k += 1
    return out + [1] * tail


def alone(reqs, portions_of):
    steps = []
    for rid, toks in reqs.items():
        at = 0
        parts = portions_of(toks)
        for i, n in enumerate(parts):
            steps.append(([(rid, toks[at:at + n], range(n))], [rid] if i == len(parts) - 1 else []))
            at += n
    return steps


def roundup(n, m=64):
    return -(-n // m) * m


def step_ctx(new_lens, prefix_lens, slots):
    """The few arrays of a step that the kernels below read."""
    pos, seq, cu = [], [], [0]
    for b, (n, p) in enumerate(zip(new_lens, prefix_lens)):
        pos += list(range(p, p + n))
        seq += [b] * n
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return SimpleNamespace(num_seqs=len(new_lens), num_tokens=len(pos), positions=i32(pos), token_seq=i32(seq), cu_seqlens=i32(cu),
                           state_slots=i32(slots), all_decode=max(new_lens) == 1)


def close(got, want, dtype, scale=1.0):
    tol = (2e-5 if dtype == "float32" else 2e-2) * scale * max(1.0, float(want.abs().max()))
    err = float((got.double().cpu() - want.double().cpu()).abs().max())
    assert err <= tol, (err, tol)


def rounded(t, dtype):
    """What the kernels see of a float64 tensor: its values in the storage type."""
    return t.to(DT[dtype]).to(F)


# ---------------------------------------------------------------------------------------------------------------
# each mechanism's kernels alone
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,slabs", [(5, 72, 1), (33, 128, 3), (2, 44, 1), (7, 4100, 2), (1, 8, 1)])
def test_norm_and_sum_on_a_sublayers_output(dtype, T, H, slabs):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(T + H)
    x, w = torch.randn(T, H, generator=g), 1 + 0.3 * torch.randn(H, generator=g)
    eps = 1e-5
    y = torch.randn(slabs, T, H, generator=g) if slabs > 1 else rounded(torch.randn(T, H, generator=g), dtype).float()
    resid = x.to(DEV)
    yd = y.to(DEV) if slabs > 1 else y.to(DEV, DT[dtype])
    copy = kernels.norm_add(resid, yd, w.to(DEV), eps, DT[dtype])
    ysum = (y.sum(0) if slabs > 1 else y).to(F)
    want = x.to(F) + P.rms(ysum, eps) * w.to(F)
    close(resid, want, "float32")
    close(copy, want, dtype)
    assert copy.dtype == DT[dtype]
    # two outputs with a weight each, normed, averaged and normed again, in one launch; their types may differ
    a, b = torch.randn(T, H, generator=g), rounded(torch.randn(T, H, generator=g), dtype).float()
    wa, wb = 1 + 0.3 * torch.randn(H, generator=g), 1 + 0.3 * torch.randn(H, generator=g)
    if H <= 4096:
        resid = x.to(DEV)
        kernels.norm_add(resid, a.to(DEV), w.to(DEV), eps, None, y2=b.to(DEV, DT[dtype]), weight1=wa.to(DEV), weight2=wb.to(DEV))
        mid = 0.5 * (P.rms(a.to(F), eps) * wa.to(F) + P.rms(b.to(F), eps) * wb.to(F))
        close(resid, x.to(F) + P.rms(mid, eps) * w.to(F), "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_streams_own_norm_and_its_copy(dtype):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(3)
    x, w = 5 * torch.randn(9, 100, generator=g), 1 + 0.3 * torch.randn(100, generator=g)
    resid = x.to(DEV)
    copy = kernels.stream_rmsnorm(resid, w.to(DEV), 1e-6, DT[dtype])
    want = P.rms(x.to(F), 1e-6) * w.to(F)
    close(resid, want, "float32")
    close(copy, want, dtype)
    close(kernels.cast_rows(resid, DT[dtype]), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,dv,maps,mode,rot", [(3, 1, 24, 40, 2, 1, 0), (4, 2, 32, 32, 2, 1, 0), (4, 2, 20, 20, 1, 2, 8),
                                                     (8, 2, 64, 64, 1, 2, 64), (2, 2, 6, 10, 1, 0, 2), (1, 1, 70, 16, 2, 1, 0)])
def test_norm_rotation_and_store_of_queries_and_keys(dtype, H, G, dk, dv, maps, mode, rot):
    """Unit by unit (a unit a map of a head) or over the whole row; the values are columns of the row as they are; the
    queries of heads with two maps leave in the order (group, map, head in group)."""
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(H * dk + rot)
    T, page, pages = 21, 8, 7
    nq, nk, nv = H * maps, G * maps, G
    cols = nq * dk + nk * dk + nv * dv
    v_col = nq * dk + nk * dk if dv != dk or maps > 1 else nq * dk          # values of the keys' size: the keys as projected
    x = rounded(torch.randn(T, cols + 3, generator=g, dtype=F), dtype)
    n = dk if mode == 1 else None
    wq, wk = 1 + 0.3 * torch.randn(n or nq * dk, generator=g), 1 + 0.3 * torch.randn(n or nk * dk, generator=g)
    eps, base = 1e-5, 300.0
    pos = torch.arange(40, 40 + T, dtype=torch.int32)
    slots = torch.tensor([(t * 5) % (page * pages) if t != 4 else -1 for t in range(T)], dtype=torch.int32)
    table = None
    if rot:
        inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32)
        table = kernels.rope_table(pos.to(DEV), inv.to(DEV))
    kc = torch.zeros(pages, nk, page, dk, dtype=DT[dtype], device=DEV)
    vc = torch.zeros(pages, nv, dv, page, dtype=DT[dtype], device=DEV)
    q = kernels.qk_norm_store(x.to(DEV, DT[dtype]), 0, nq * dk, v_col, nq, nk, nv, dk, dv, maps, mode,
                              wq.to(DEV) if mode else None, wk.to(DEV) if mode else None, eps, table, rot, slots.to(DEV), kc, vc)
    xq, xk = x[:, :nq * dk], x[:, nq * dk:nq * dk + nk * dk]
    if mode == 1:
        xq = (P.rms(xq.view(T, nq, dk), eps) * wq.to(F))
        xk = (P.rms(xk.view(T, nk, dk), eps) * wk.to(F))
    elif mode == 2:
        xq, xk = (P.rms(xq, eps) * wq.to(F)).view(T, nq, dk), (P.rms(xk, eps) * wk.to(F)).view(T, nk, dk)
    else:
        xq, xk = xq.view(T, nq, dk), xk.view(T, nk, dk)
    xq, xk = P.rotate_half(xq, pos, rot, base), P.rotate_half(xk, pos, rot, base)
    if maps > 1:
        R = H // G
        xq = xq.view(T, G, R, maps, dk).permute(0, 1, 3, 2, 4).reshape(T, nq, dk)
    close(q.view(T, nq, dk), xq, dtype)
    xv = x[:, v_col:v_col + nv * dv].view(T, nv, dv)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        close(kc[s // page, :, s % page, :], xk[t], dtype)
        assert torch.equal(vc[s // page, :, :, s % page].double().cpu(), xv[t])
    stored = {int(s) for s in slots if s >= 0}
    empty = [s for s in range(page * pages) if s not in stored]
    assert all(float(kc[s // page, :, s % page, :].float().abs().max()) == 0 for s in empty)


def reference_attention(q, k, v, positions, scale, chunk=0, sink=False, gate=None, temp=None):
    """q [n, H, dk] at ``positions`` over keys k [N, G, dk] and values v [N, Gv, dv] of positions 0 .. N - 1, in float64."""
    n, H, dk = q.shape
    G, Gv = k.shape[1], v.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for i, p in enumerate(positions):
        for h in range(H):
            g = h // (H // G)
            s = (k[:p + 1, g] @ q[i, h]) * scale * (temp(p) if temp else 1.0)
            vis = torch.tensor([P.chunk_visible(p, j, chunk) for j in range(p + 1)])
            e = torch.where(vis, torch.exp(s - s[vis].max()), torch.zeros_like(s))
            den = e.sum() + (math.exp(-float(s[vis].max())) if sink else 0.0)
            o = (e / den) @ v[:p + 1, g // (G // Gv)]
            out[i, h] = o * (torch.sigmoid(gate[i, h]) if gate is not None else 1.0)
    return out


def scatter_pages(k_seqs, v_seqs, page, num_pages, dtype, seed):
    """Whole sequences of keys [N, G, dk] and values [N, Gv, dv] into pages in a random physical order, the rest of
    the pool full of large numbers that nothing may read: K [pages, G, page, dk], V [pages, Gv, dv, page], the table."""
    g = torch.Generator().manual_seed(seed)
    (G, dk), (Gv, dv) = k_seqs[0].shape[1:], v_seqs[0].shape[1:]
    K, V = 50 * torch.randn(num_pages, G, page, dk, generator=g), 50 * torch.randn(num_pages, Gv, dv, page, generator=g)
    perm = torch.randperm(num_pages, generator=g).tolist()
    need = [-(-k.shape[0] // page) for k in k_seqs]
    bt = torch.full((len(k_seqs), max(need)), -1, dtype=torch.int32)
    for b, (k, v) in enumerate(zip(k_seqs, v_seqs)):
        for j in range(need[b]):
            pg = perm.pop()
            bt[b, j] = pg
            n = min(page, k.shape[0] - j * page)
            K[pg, :, :n, :] = k[j * page:j * page + n].transpose(0, 1).float()
            V[pg, :, :, :n] = v[j * page:j * page + n].permute(1, 2, 0).float()
    return K.to(DEV, dtype), V.to(DEV, dtype), bt.to(DEV)


ATTENTION_SHAPES = [   # H, G, Gv, dk, dv, chunk, sink, gated, temperature
    (3, 1, 1, 24, 24, 11, True, True, None), (4, 2, 2, 64, 64, 40, True, True, None), (8, 4, 2, 32, 32, 0, False, False, (0.4, 8)),
    (6, 2, 1, 24, 40, 0, False, False, (0.2, 16)), (2, 2, 2, 32, 32, 0, True, True, None), (4, 1, 1, 96, 96, 1, True, True, None),
    (16, 4, 2, 32, 64, 0, False, False, None)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ATTENTION_SHAPES)
def test_attention_in_chunks_with_a_sink_a_gate_a_head_and_shared_values(dtype, shape):
    """Prompts, portions behind a prefix and single tokens in one step, pages in any order; the plain kernel in both
    precisions and, where it takes the sizes, the matrix-core kernel four blocks a workgroup, one block, and in pieces."""
    from pico_vllm_amd.ops import attention_bias_fast, kernels
    H, G, Gv, dk, dv, chunk, sink, gated, temp = shape
    g = torch.Generator().manual_seed(H * 100 + dk)
    page = 8
    new, prefix = [70, 1, 1, 23, 2], [0, 37, 160, 85, 0]
    ks = [rounded(torch.randn(n + p, G, dk, generator=g, dtype=F), dtype) for n, p in zip(new, prefix)]
    vs = [rounded(torch.randn(n + p, Gv, dv, generator=g, dtype=F), dtype) for n, p in zip(new, prefix)]
    qs = [rounded(torch.randn(n, H, dk, generator=g, dtype=F), dtype) for n in new]
    gate = [rounded(torch.randn(n, H, generator=g, dtype=F), dtype) for n in new] if gated else [None] * len(new)
    tf = (lambda p: P.query_temperature(p, *temp)) if temp else None
    want = torch.cat([reference_attention(q, k, v, range(p, p + n), 0.3, chunk, sink, gt, tf)
                      for q, k, v, n, p, gt in zip(qs, ks, vs, new, prefix, gate)]).reshape(sum(new), H * dv)
    num_pages = sum(-(-(n + p) // page) for n, p in zip(new, prefix)) + 3
    K, V, bt = scatter_pages(ks, vs, page, num_pages, DT[dtype], seed=5)
    ctx = step_ctx(new, prefix, [0] * len(new))
    q = torch.cat(qs).reshape(sum(new), H * dk).to(DEV, DT[dtype])
    gt = torch.cat(gate).to(DEV, DT[dtype]) if gated else None
    kw = dict(chunk=chunk, sink=sink, gate_heads=gated, v_div=G // Gv)
    tk = dict(temp_coef=temp[0], temp_every=temp[1]) if temp else {}
    for f32_out in (False, True):
        got = kernels.attn_bias_plain(q, K, V, bt, ctx.positions, ctx.token_seq, H, G, dk, dv, 0.3, gate=gt, out_f32=f32_out, **kw, **tk)
        assert got.dtype == (torch.float32 if f32_out else DT[dtype])
        close(got, want, dtype)
    if dtype == "bfloat16" and attention_bias_fast.supported(dk, dv):
        fast = attention_bias_fast.FastBiasAttention(H, G, dk, dv, 0.3, gated=gated, **kw, **tk)
        for split, chunks in ((False, 1), (True, 1), (True, 2), (True, 5)):
            got = fast.run(q, K, V, bt, ctx.cu_seqlens, ctx.positions, len(new), split=split, chunks=chunks, gate=gt)
            close(got, want, dtype)
        fast32 = attention_bias_fast.FastBiasAttention(H, G, dk, dv, 0.3, gated=gated, out_f32=True, **kw, **tk)
        for split, chunks in ((False, 1), (True, 3)):
            got = fast32.run(q, K, V, bt, ctx.cu_seqlens, ctx.positions, len(new), split=split, chunks=chunks, gate=gt)
            assert got.dtype == torch.float32
            close(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page", [8, 16])
@pytest.mark.parametrize("decoded", [False, True])
def test_one_key_stands_out_just_inside_and_just_outside_the_chunk(dtype, page, decoded):
    """All keys but one are tiny; the query at position p sits on that key if it sees it.  With the key at the first
    position of p's chunk the output is that key's value (less the sink's share); at the position before, it is not."""
    from pico_vllm_amd.ops import attention_bias_fast, kernels
    H, G, d, chunk = 2, 1, 32, 24
    for p, key in ((100, 96), (100, 95), (96, 96), (119, 96), (120, 119), (95, 72), (500, 480), (500, 479), (23, 0), (24, 0)):
        g = torch.Generator().manual_seed(p + key)
        n = p + 1
        k = 0.01 * torch.randn(n, G, d, generator=g, dtype=F)
        v = torch.randn(n, G, d, generator=g, dtype=F)
        qv = torch.randn(1, H, d, generator=g, dtype=F)
        k[key, 0] = 4.0 * qv[0, 0] / qv[0, 0].norm()
        qv[0, 1] = qv[0, 0]
        k, v, qv = rounded(k, dtype), rounded(v, dtype), rounded(qv, dtype)
        new = 1 if decoded else min(n, 30)
        qs = torch.zeros(new, H, d, dtype=F)
        qs[-1] = qv[0]
        K, V, bt = paged_cache([k], [v], page, n // page + 3, DT[dtype], seed=p)
        ctx = step_ctx([new], [n - new], [0])
        q = qs.reshape(new, H * d).to(DEV, DT[dtype])
        want = reference_attention(qv, k, v, [p], 1.0, chunk, True)[0, 0]
        seen = P.chunk_visible(p, key, chunk)
        assert (float((want - v[key, 0]).norm()) < 0.2 * float(v[key, 0].norm())) == seen
        outs = [kernels.attn_bias_plain(q, K, V, bt, ctx.positions, ctx.token_seq, H, G, d, d, 1.0, chunk=chunk, sink=True)]
        if dtype == "bfloat16":
            fast = attention_bias_fast.FastBiasAttention(H, G, d, d, 1.0, chunk=chunk, sink=True)
            outs += [fast.run(q, K, V, bt, ctx.cu_seqlens, ctx.positions, 1, split=s, chunks=c) for s, c in ((False, 1), (True, 1), (True, 4))]
        for got in outs:
            close(got[-1].view(H, d)[0], want, dtype)
            close(got[-1].view(H, d)[1], want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dv", [(3, 1, 40), (4, 2, 32), (1, 1, 16), (8, 2, 100)])
def test_two_maps_into_one_output(dtype, H, G, dv):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(H + dv)
    T, lam, eps, diff = 9, 0.43, 1e-5, 0.3
    a = torch.randn(T, G, 2, H // G, dv, generator=g)
    got = kernels.diff_combine(a.reshape(T, -1).to(DEV), lam, eps, 1 - diff, H, G, dv, DT[dtype])
    a1, a2 = a[:, :, 0].reshape(T, H, dv).to(F), a[:, :, 1].reshape(T, H, dv).to(F)
    close(got.view(T, H, dv), P.rms(a1 - lam * a2, eps) * (1 - diff), dtype)


def run_conv(x, w_t, bias, lens, prefix, slots, state, dtype):
    from pico_vllm_amd.ops import kernels
    ctx = step_ctx(lens, prefix, slots)
    return kernels.causal_conv(x.to(DEV, DT[dtype]), w_t.shape[1], w_t, bias, ctx, state, 0, single=ctx.all_decode)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C,taps", [(44, 2), (256, 4), (36, 1), (40, 5)])
def test_a_convolution_without_bias_whose_state_is_its_last_inputs(dtype, C, taps):
    g = torch.Generator().manual_seed(C)
    T = 29
    x = rounded(torch.randn(T, C + 3, generator=g, dtype=F), dtype)
    w = torch.randn(C, taps, generator=g)
    w_t = w.t().contiguous().to(DEV)
    want = P.silu(P.causal_conv(x[:, :C], w.to(F)))
    for portions in ([T], [2, 13, 1, 1, 12], [1] * T):
        state = torch.full((3, C, taps - 1), 7.0, device=DEV)
        state[1] = 0
        at, outs = 0, []
        for n in portions:
            outs.append(run_conv(x[at:at + n], w_t, None, [n], [at], [1], state, dtype))
            at += n
        close(torch.cat(outs), want, dtype)
        assert float((state[0] - 7).abs().max()) == 0 and float((state[2] - 7).abs().max()) == 0 if taps > 1 else True


DELTA_SHAPES = [(3, 1, 12, 20), (4, 2, 32, 64), (2, 2, 16, 16), (2, 1, 136, 5), (1, 1, 4, 70), (4, 4, 64, 32), (2, 1, 300, 9)]


def delta_inputs(H, G, dk, dv, T, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    unit = lambda t: t / t.norm(dim=-1, keepdim=True)
    q = unit(torch.randn(T, G, dk, generator=g)) * dk ** -0.5
    k = unit(torch.randn(T, G, dk, generator=g))
    v = rounded(torch.randn(T, H, dv, generator=g, dtype=F), dtype)
    decay = torch.sigmoid(2 + torch.randn(T, H, dk, generator=g))
    beta = torch.sigmoid(torch.randn(T, H, generator=g))
    return q, k, v, decay, beta


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,dv", DELTA_SHAPES)
def test_the_delta_rules_walk_whole_in_portions_and_token_by_token(dtype, H, G, dk, dv):
    from pico_vllm_amd.ops import kernels
    T = 50
    q, k, v, decay, beta = delta_inputs(H, G, dk, dv, T, H * dk + dv, dtype)
    idx = torch.tensor([h // (H // G) for h in range(H)])
    want, S_want = P.delta_rule_scan(q.to(F)[:, idx], k.to(F)[:, idx], v, decay.to(F), beta.to(F))
    results = []
    for portions in ([T], [7, 1, 30, 2, 10], [1] * T):
        state = torch.full((4, H, dk, dv), 3.0, device=DEV)
        state[2] = 0
        at, outs = 0, []
        for n in portions:
            sl = slice(at, at + n)
            ctx = step_ctx([n], [at], [2])
            outs.append(kernels.delta_scan(q[sl].reshape(n, -1).to(DEV), k[sl].reshape(n, -1).to(DEV), v[sl].reshape(n, -1).to(DEV, DT[dtype]),
                                           decay[sl].reshape(n, -1).to(DEV), beta[sl].contiguous().to(DEV), ctx.cu_seqlens, ctx.state_slots,
                                           state, 1, H, G, dk, dv, delta=True))
            at += n
        got = torch.cat(outs)
        results.append((got, state.clone()))
        close(got.view(T, H, dv), want, "float32", scale=5)
        close(state[2], S_want, "float32", scale=5)
        assert float((state[[0, 1, 3]] - 3).abs().max()) == 0               # other requests' states are untouched
    for got, st in results[1:]:                                              # the cut changes no bit
        assert torch.equal(got, results[0][0]) and torch.equal(st, results[0][1])
    # chunks side by side: the same sums in another order, from a state that is not zero
    g = torch.Generator().manual_seed(1)
    s0 = 0.3 * torch.randn(H, dk, dv, generator=g)
    want, S_want = P.delta_rule_scan(q.to(F)[:, idx], k.to(F)[:, idx], v, decay.to(F), beta.to(F), s0.to(F))
    for chunk in (4, 16, 64):
        state = torch.full((4, H, dk, dv), 3.0, device=DEV)
        state[2] = s0.to(DEV)
        ctx = step_ctx([T], [9], [2])
        got = kernels.delta_scan(q.reshape(T, -1).to(DEV), k.reshape(T, -1).to(DEV), v.reshape(T, -1).to(DEV, DT[dtype]),
                                 decay.reshape(T, -1).to(DEV), beta.contiguous().to(DEV), ctx.cu_seqlens, ctx.state_slots, state,
                                 1, H, G, dk, dv, delta=True, chunk=chunk)
        close(got.view(T, H, dv), want, "float32", scale=5)
        close(state[2], S_want, "float32", scale=5)
        assert float((state[[0, 1, 3]] - 3).abs().max()) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,N,dv", [(3, 1, 12, 20), (4, 2, 32, 32), (1, 1, 80, 48), (6, 3, 16, 64)])
def test_the_same_walk_without_the_correction_is_the_state_space_layer(dtype, H, G, N, dv):
    """Several sequences side by side, one decay a head, u = dt x."""
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(N + dv)
    lens = [17, 1, 40]
    T = sum(lens)
    x = rounded(torch.randn(T, H, dv, generator=g, dtype=F), dtype)
    B, C = torch.randn(T, G, N, generator=g), torch.randn(T, G, N, generator=g)
    dt = torch.nn.functional.softplus(torch.randn(T, H, generator=g))
    a, D = torch.exp(0.5 * torch.randn(H, generator=g)), torch.randn(H, generator=g)
    idx = torch.tensor([h // (H // G) for h in range(H)])
    ctx = step_ctx(lens, [0, 5, 0], [1, 0, 2])
    state = torch.zeros(3, H, N, dv, device=DEV)
    s0 = torch.randn(H, N, dv, generator=g)
    state[0] = s0.to(DEV)                                                   # the second sequence goes on from a state
    got = kernels.delta_scan(C.reshape(T, -1).to(DEV), B.reshape(T, -1).to(DEV), x.reshape(T, -1).to(DEV, DT[dtype]),
                             torch.exp(-a * dt).contiguous().to(DEV), dt.contiguous().to(DEV), ctx.cu_seqlens, ctx.state_slots, state,
                             3, H, G, N, dv, delta=False)
    def check(got, state):
        at = 0
        for n, S0, slot in zip(lens, (None, s0.to(F), None), (1, 0, 2)):
            sl = slice(at, at + n)
            y, S = P.ssd_scan(x[sl], B.to(F)[sl][:, idx], C.to(F)[sl][:, idx], dt.to(F)[sl], a.to(F), torch.zeros(H, dtype=F), S0)
            close(got[sl].view(n, H, dv), y, "float32", scale=5)
            close(state[slot], S, "float32", scale=5)
            at += n
    check(got, state)
    for chunk in (3, 16):                                                    # chunks side by side, sequences of unequal length
        st = torch.zeros(3, H, N, dv, device=DEV)
        st[0] = s0.to(DEV)
        check(kernels.delta_scan(C.reshape(T, -1).to(DEV), B.reshape(T, -1).to(DEV), x.reshape(T, -1).to(DEV, DT[dtype]),
                                 torch.exp(-a * dt).contiguous().to(DEV), dt.contiguous().to(DEV), ctx.cu_seqlens, ctx.state_slots, st,
                                 3, H, G, N, dv, delta=False, chunk=chunk), st)
    # the gate, the skip and the norm in parts behind it
    from pico_vllm_amd.ops import kernels as K
    z = rounded(torch.randn(T, H * dv + 5, generator=g, dtype=F), dtype)
    w = 1 + 0.3 * torch.randn(H * dv, generator=g)
    for parts in (1, H):
        out = K.gated_group_norm(got, x.reshape(T, -1).to(DEV, DT[dtype]), z.to(DEV, DT[dtype]), D.to(DEV), w.to(DEV), 1e-5, H, dv, parts)
        y = (got.double().cpu().view(T, H, dv) + D.to(F).view(1, H, 1) * x).reshape(T, -1) * P.silu(z[:, :H * dv])
        close(out, P.rms(y.view(T, parts, -1), 1e-5).reshape(T, -1) * w.to(F), dtype)


def test_without_decay_a_first_write_is_read_back_after_hundreds_of_tokens():
    """Keys that are unit vectors of the axes: the first token writes under key 0, the next 600 under other keys; a query
    on key 0 at the end reads the first value; with a decay of 0.99 on that key's channel it reads 0.99^600 of it."""
    from pico_vllm_amd.ops import kernels
    H, dk, dv, T = 1, 8, 6, 601
    k = torch.zeros(T, 1, dk)
    k[0, 0, 0] = 1
    for t in range(1, T):
        k[t, 0, 1 + t % (dk - 1)] = 1
    q = torch.zeros(T, 1, dk)
    q[:, 0, 0] = 1
    g0 = torch.Generator().manual_seed(0)
    v = torch.randn(T, 1, dv, generator=g0)
    beta = torch.ones(T, 1)
    for keep in (1.0, 0.99):
        decay = torch.ones(T, 1, dk)
        decay[1:, 0, 0] = keep
        state = torch.zeros(2, H, dk, dv, device=DEV)
        outs = []
        for lo, hi in ((0, 300), (300, 600), (600, 601)):
            ctx = step_ctx([hi - lo], [lo], [1])
            outs.append(kernels.delta_scan(q[lo:hi].reshape(hi - lo, -1).to(DEV), k[lo:hi].reshape(hi - lo, -1).to(DEV),
                                           v[lo:hi].reshape(hi - lo, -1).to(DEV), decay[lo:hi].reshape(hi - lo, -1).to(DEV),
                                           beta[lo:hi].to(DEV), ctx.cu_seqlens, ctx.state_slots, state, 1, H, 1, dk, dv))
        close(outs[-1][0], (keep ** 600) * v[0, 0].to(F), "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,R", [(3, 1, 12, 6), (4, 2, 32, 5), (2, 1, 136, 9)])
def test_what_enters_the_delta_rules_walk(dtype, H, G, dk, R):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(dk)
    T = 13
    x = rounded(torch.randn(T, 2 * G * dk + 7, generator=g, dtype=F), dtype)
    y = rounded(torch.randn(T, 3 + H + R, generator=g, dtype=F), dtype)
    a2 = rounded(torch.randn(H * dk, R, generator=g, dtype=F), dtype)
    dt_bias, a_log = torch.randn(H * dk, generator=g), 0.5 * torch.randn(H, generator=g)
    qn, kn, dec, beta = kernels.delta_prep(x.to(DEV, DT[dtype]), 0, G * dk, y.to(DEV, DT[dtype]), 3, 3 + H, a2.to(DEV, DT[dtype]),
                                           dt_bias.to(DEV), a_log.to(DEV), dk ** -0.5, H, G, dk)
    unit = lambda t: t / torch.sqrt((t * t).sum(-1, keepdim=True) + 1e-6)
    close(qn.view(T, G, dk), unit(x[:, :G * dk].view(T, G, dk)) * dk ** -0.5, "float32")
    close(kn.view(T, G, dk), unit(x[:, G * dk:2 * G * dk].view(T, G, dk)), "float32")
    close(beta, torch.sigmoid(y[:, 3:3 + H]), "float32")
    step = P.softplus(y[:, 3 + H:] @ a2.T + dt_bias.to(F)).view(T, H, dk)
    close(dec.view(T, H, dk), torch.exp(-torch.exp(a_log.to(F)).view(1, H, 1) * step), "float32")


# ---------------------------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_and_token_by_token_from_the_first_token(name, dtype):
    reqs = requests(CONFIGS[name]["vocab"], [150, 1, 37], seed=1)
    rows, _ = replay(model_dir(name), dtype, alone(reqs, lambda t: [len(t)]), roundup(150), PAGE[name])
    compare(name, dtype, rows, reqs)
    one = {"r2": reqs["r2"]}
    rows1, _ = replay(model_dir(name), dtype, alone(one, lambda t: [1] * len(t)), roundup(37), PAGE[name])
    compare(name, dtype, rows1, one)
    if dtype == "float32":
        for key, row in rows1.items():
            assert np.array_equal(row, rows[key])         # decoded through cache and state: the same bits as the prompt


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_of_many_sizes_down_to_two_tokens_then_decoding(name, dtype):
    reqs = requests(CONFIGS[name]["vocab"], [190], seed=2)
    rows, _ = replay(model_dir(name), dtype, alone(reqs, lambda t: cut(t, [2, 33, 5, 70, 3, 16], tail=60)), roundup(190), PAGE[name])
    compare(name, dtype, rows, reqs)
    if dtype == "float32":
        whole, _ = replay(model_dir(name), dtype, alone(reqs, lambda t: [len(t)]), roundup(190), PAGE[name])
        for key, row in rows.items():
            assert np.array_equal(row, whole[key])


def mixed_steps(reqs, page, seed, max_live=3, tail=12):
    """At most ``max_live`` requests live: portions of changing size of some beside single tokens of others, now and then
    a request left out of a step.  Returns the steps and the most tokens live requests held (rounded up to pages)."""
    rng = random.Random(seed)
    waiting, live, steps = list(reqs), {}, []
    sizes = [17, 2, 40, 6, 29]
    peak = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            toks, at = reqs[rid], live[rid]
            if rng.random() < 0.2 and len(live) > 1:
                continue
            last = len(toks) - at <= tail
            n = 1 if last else min(sizes[rng.randrange(len(sizes))], len(toks) - tail - at)
            entries.append((rid, toks[at:at + n], range(n)))
            live[rid] = at + n
            if live[rid] == len(toks):
                end.append(rid)
        peak = max(peak, sum(roundup(live[r], page) for r in live))
        for rid in end:
            del live[rid]
        if entries:
            steps.append((entries, end))
    return steps, roundup(peak)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_mixed_batches_in_a_pool_that_holds_what_is_live(name, dtype):
    """Seven unequal requests, at most three live, in a pool that holds just the live ones and with three state slots:
    pages and slots are used again; each request against itself alone."""
    lengths = [70, 33, 120, 9, 64, 47, 101]
    reqs = requests(CONFIGS[name]["vocab"], lengths, seed=4)
    steps, peak = mixed_steps(reqs, PAGE[name], seed=7)
    rows, rp = replay(model_dir(name), dtype, steps, peak, PAGE[name], max_live=3)
    compare(name, dtype, rows, reqs)
    m = rp.runner.manager
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.slots.num_free == 3      # all given back
    if dtype == "float32":
        solo, _ = replay(model_dir(name), dtype, alone(reqs, lambda t: [len(t)]), roundup(max(lengths)), PAGE[name])
        for key, row in rows.items():
            assert np.array_equal(row, solo[key])               # what else is in the batch changes no bit


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    reqs = requests(CONFIGS["b"]["vocab"], [330], seed=6)
    rows, _ = replay(model_dir("b"), dtype, alone(reqs, lambda t: cut(t, [30], tail=300)), roundup(330), PAGE["b"])
    compare("b", dtype, rows, reqs)


def test_pages_of_passed_chunks_come_back_while_a_request_runs():
    reqs = requests(CONFIGS["b"]["vocab"], [200], seed=3)
    rows, rp = replay(model_dir("b"), "float32", [([("r0", reqs["r0"][:170], range(170))], [])], roundup(200), 8)
    m = rp.runner.manager
    chunked = [g for g in m.groups if g.spec.chunk][0]
    assert chunked.pool.num_free == chunked.pool.num_pages - 2               # chunks of 40: positions 160 .. 169 are read on
    compare("b", "float32", rows, reqs)


def test_sharp_attention_on_far_keys_and_across_every_chunk_edge():
    """Scales so large that every query's softmax sits on very few keys: in the causal layer many of them hundreds of
    tokens back and on other pages; in the chunked layer a key of the neighbouring chunk would take the place of the sink.
    A key read from a wrong place, or seen across an edge, shows in the logits."""
    cfg = config(64, 64, [(attention(2, 1, 16, 16, diff=0.4, scale=3.0, q_temp=(0.5, 32)), 32),
                          (parallel((2, 1, 16, 13, 8, 1000.0, 3.0), (2, 1, 8, 8, 2)), None)])
    t = P.random_model(cfg, 5)
    d = write_model(cfg, t, "vagelix_far_")
    reqs = requests(64, [400], seed=9)
    for portions in (lambda x: [len(x)], lambda x: cut(x, [2, 61, 8, 130], tail=40)):
        rows, _ = replay(d, "float32", alone(reqs, portions), roundup(400), 8)
        compare("far", "float32", rows, reqs, bound=1e-4, cfg=cfg, tensors=t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(dtype, graphs):
    from pico_vllm_amd import LLM, SamplingParams
    name = "b"
    prompts = [[5, 17, 3, 200, 41], [9] * 19, [77, 2], list(range(60, 130)), [1], [250, 3, 3, 8, 100, 100]]
    llm = LLM(model=model_dir(name), dtype=dtype, block_size=8, num_gpu_blocks=48, max_seq_len=160, max_num_seqs=3,
              max_num_batched_tokens=24, use_cuda_graph=graphs, max_batch_size=4)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.0, ignore_eos=True))
    cfg, t = CONFIGS[name], tensors_of(name)
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 12
        toks = list(p)
        for tok in o.token_ids:
            logits = P.forward(cfg, t, toks)[-1]
            slack = 1e-4 if dtype == "float32" else 0.08 * float(logits.std())
            assert float(logits[tok]) >= float(logits.max()) - slack, (dtype, p, o.token_ids, tok, int(logits.argmax()))
            toks.append(tok)
    llm.engine.runner.manager.check()


def test_the_replay_program_in_a_subprocess():
    import json
    import os
    import subprocess
    import tempfile
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "a"
    reqs = requests(CONFIGS[name]["vocab"], [40, 23, 31], seed=8)
    steps = []
    for rid, toks in reqs.items():
        parts = cut(toks, [9, 2, 14], tail=5)
        at = 0
        for i, n in enumerate(parts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if i == len(parts) - 1 else []})
            at += n
    with tempfile.TemporaryDirectory() as out:
        r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dir(name), "--dtype", "float32", "--out", out,
                            "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
                           text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert r.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
        rows, fed = {}, {}
        for s in steps:
            e = s["entries"][0]
            a = np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(len(e["want"]), -1)
            for w, row in zip(e["want"], a):
                rows[(e["id"], fed.get(e["id"], 0) + w)] = row
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
    compare(name, "float32", rows, reqs)


def test_the_command_line_on_a_model_folder_of_this_design(capsys):
    from pico_vllm_amd import run
    assert run.main(["--model", model_dir("d"), "--prompt-ids", "5,17,3", "--prompt-ids", "9", "--max-new-tokens", "6",
                     "--ignore-eos", "--dtype", "float32", "--num-gpu-blocks", "16", "--max-seq-len", "64"]) == 0
    lines = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")]
    assert len(lines) == 2
    cfg, t = CONFIGS["d"], tensors_of("d")
    for line, prompt in zip(lines, ([5, 17, 3], [9])):
        toks = list(prompt)
        for tok in (int(x) for x in line.split(")")[1].split()):
            logits = P.forward(cfg, t, toks)[-1]
            assert float(logits[tok]) >= float(logits.max()) - 1e-4
            toks.append(tok)


# ---------------------------------------------------------------------------------------------------------------
# configurations drawn at random
# ---------------------------------------------------------------------------------------------------------------
def draw_config(seed, fast=False):
    """Sizes, head counts, order of layers, constants, which layers run another's tensors: all drawn; returns
    (config, page size).  ``fast``: sizes that the matrix-core kernels take."""
    rng = random.Random(2000 + seed)
    width = rng.choice([128, 192, 256] if fast else [40, 64, 72, 96, 128])
    dims = [32, 64] if fast else [6, 10, 16, 24, 40]
    layers = []
    for _ in range(rng.randint(2, 4)):
        kind = rng.choice(["attention", "parallel", "mamba2"])
        ff = rng.choice([None, 24, 64])
        G = rng.choice([1, 2])
        H = G * rng.choice([1, 2, 3])
        if kind == "attention":
            mixer = attention(H, G, rng.choice(dims), rng.choice([16, 32, 48] if fast else [8, 12, 20, 36]), diff=rng.choice([0.2, 0.5, 0.8]),
                              q_temp=rng.choice([None, (0.3, 5), (0.1, 64)]))
        elif kind == "parallel":
            d = rng.choice(dims)
            rot = rng.choice([0, 2, d // 2 * 2, d])
            Gr = rng.choice([1, 2])
            mixer = parallel((H, G, d, rng.choice([0, 1, 7, 16, 33, 100]), rot, rng.choice([100.0, 50000.0]), None),
                             (Gr * rng.choice([1, 2]), Gr, rng.choice([4, 12, 32, 72]), rng.choice([5, 16, 32]), rng.randint(1, 4)))
        else:
            Hm = G * rng.choice([1, 2, 3])
            dv = rng.choice([8, 16, 24])
            mixer = mamba2(Hm, dv, rng.choice([4, 16, 48]), G, rng.choice([1, Hm]), rng.randint(1, 4))
        layers.append((mixer, ff))
    for i in range(len(layers)):
        if rng.random() < 0.3:
            layers.append(i)
    return config(rng.choice([50, 131, 300]), width, layers, eps=rng.choice([1e-5, 1e-6])), rng.choice([8, 16, 32])


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random_in_mixed_batches(seed):
    cfg, page = draw_config(seed, fast=seed >= 8)
    t = P.random_model(cfg, seed, decay_rank=3 + seed % 4, gate_rank=2 + seed % 5)
    d = write_model(cfg, t, f"vagelix_drawn{seed}_")
    lengths = [60, 21, 150, 7, 45] if seed < 8 else [260, 90, 33, 140]
    reqs = requests(cfg["vocab"], lengths, seed=seed)
    steps, peak = mixed_steps(reqs, page, seed=seed)
    for dtype in ("float32", "bfloat16"):
        rows, rp = replay(d, dtype, steps, peak, page, max_live=3)
        compare(f"drawn{seed}", dtype, rows, reqs, cfg=cfg, tensors=t)
