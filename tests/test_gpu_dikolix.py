"""The Dikolix decoder in the engine against the plain implementation: each mechanism's kernel alone, then whole
prompts, decoding through the cache and the state, portions down to two tokens, mixed batches in a small pool with few
state slots, a far key that stands out, long decoding, and greedy generation through the entry point."""
import random
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_dikolix as P
from dikolix_configs import CONFIGS, YARN, config, latent, model_dir, moe, retention, ssm, tensors_of, write_model
from gpu_util import DEV

pytestmark = pytest.mark.gpu

# rms of a position's error over its logits (mean taken off), in units of the logits' own rms there
BOUND = {"float32": 3e-5, "bfloat16": 7e-2}
# In bfloat16 a token whose last chosen and first rejected router logit lie within CLOSE_CALL of the row's spread may get
# the other expert than in the plain run, which is no fault; nor is it one where a retention head's output cancels to a
# small part of what went into it (a rounding then decides its direction in front of the head norm).  What such a token
# changes reaches every later position through the recurrent layers: those positions are only held to TAINTED_BOUND.
# (The margin is counted in units of the router logits' spread over a row; what reaches a router after several layer
# runs in bfloat16 is off by a few percent of its size, and so are the logits.)
CLOSE_CALL, TAINTED_BOUND = 0.4, 2.5
# float32 rounds too: below FLOAT32_FLIP a choice may really turn (then as in bfloat16); below FLOAT32_CLOSE a head norm
# multiplies a rounding of 1e-7 by hundreds
FLOAT32_FLIP, FLOAT32_CLOSE, FLOAT32_LOOSE = 1e-4, 0.01, 1e-3
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
PAGE = {"a": 16, "b": 8, "c": 32, "d": 16}


def row_errors(got, want):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


_plain = {}


def plain_logits(name, tokens, cfg=None, tensors=None):
    key = (name, tuple(tokens))
    if key not in _plain:
        margins = []
        _plain[key] = P.forward(cfg or CONFIGS[name], tensors or tensors_of(name), tokens, margins_out=margins).numpy()
        least = torch.stack(margins).min(0).values if margins else torch.full((len(tokens),), float("inf"), dtype=torch.float64)
        _plain[key + ("margin",)] = torch.cummin(least, 0).values.tolist()
    return _plain[key]


def margin_upto(name, tokens, position):
    return _plain[(name, tuple(tokens), "margin")][position]


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


def compare(name, dtype, rows, reqs, bound=None, cfg=None, tensors=None):
    bound = BOUND[dtype] if bound is None else bound
    errs = []
    for (rid, pos), got in rows.items():
        toks = reqs[rid.split("#")[0]]
        e = float(row_errors(got[None], plain_logits(name, toks, cfg, tensors)[pos][None])[0])
        m = margin_upto(name, toks, pos)
        if not (dtype == "bfloat16" and m < CLOSE_CALL):
            errs.append(e)
        if (dtype == "bfloat16" and m < CLOSE_CALL) or m < FLOAT32_FLIP:
            assert e <= TAINTED_BOUND, f"{name} {dtype}: {rid} position {pos}: {e:.3g}"
        elif dtype == "float32" and m < FLOAT32_CLOSE:
            assert e <= FLOAT32_LOOSE, f"{name} {dtype}: {rid} position {pos}: {e:.3g}"
        else:
            assert e <= bound, f"{name} {dtype}: {rid} position {pos}: {e:.3g} > {bound} (margin {m:.3g})"
    if len(errs) >= 5:
        assert np.median(errs) <= bound / 2, f"{name} {dtype}: median {np.median(errs):.3g}"


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


def step_ctx(new_lens, prefix_lens, slots, tokens=None):
    """The few arrays of a step that the kernels below read."""
    pos, seq, cu = [], [], [0]
    for b, (n, p) in enumerate(zip(new_lens, prefix_lens)):
        pos += list(range(p, p + n))
        seq += [b] * n
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return SimpleNamespace(num_seqs=len(new_lens), num_tokens=len(pos), positions=i32(pos), token_seq=i32(seq), cu_seqlens=i32(cu),
                           state_slots=i32(slots), token_ids=i32(tokens if tokens is not None else [0] * len(pos)))


def close(got, want, dtype, scale=1.0):
    tol = (2e-5 if dtype == "float32" else 2e-2) * scale * max(1.0, float(want.abs().max()))
    err = float((got.double().cpu() - want).abs().max())
    assert err <= tol, (err, tol)


# ---------------------------------------------------------------------------------------------------------------
# each mechanism's kernels alone
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,slabs,scaled", [(5, 72, 1, True), (33, 128, 3, True), (2, 44, 1, False), (7, 4100, 2, True)])
def test_layer_norm_with_a_scaled_sum_in_front(dtype, T, H, slabs, scaled):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(T)
    resid = torch.randn(T, H, generator=g) * 3 + 1.5
    delta = torch.randn(slabs, T, H, generator=g) if slabs > 1 else torch.randn(T, H, generator=g).to(DT[dtype]).float()
    w, b, s = 1 + 0.3 * torch.randn(H, generator=g), 0.2 * torch.randn(H, generator=g), 0.5 + torch.rand(H, generator=g)
    x = resid.double() + (s.double() if scaled else 1.0) * (delta.double().sum(0) if slabs > 1 else delta.double())
    want = P.layer_norm(x, w.double(), b.double(), 1e-5)
    r = resid.to(DEV)
    d = delta.to(DEV) if slabs > 1 else delta.to(DEV, DT[dtype])
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    some = kernels.add_layernorm(r, d, w.to(DEV), b.to(DEV), 1e-5, DT[dtype], rows, s.to(DEV) if scaled else None)
    assert torch.equal(r.cpu(), resid)                              # with rows the stream is left alone
    got = kernels.add_layernorm(r, d, w.to(DEV), b.to(DEV), 1e-5, DT[dtype], None, s.to(DEV) if scaled else None)
    close(got, want, dtype)
    close(some, want[[T - 1, 0]], dtype)
    close(r, x, "float32")
    # a row of equal entries has no deviation: the output is the bias
    flat = torch.full((1, H), 7.0, device=DEV)
    close(kernels.add_layernorm(flat, None, w.to(DEV), b.to(DEV), 1e-5, torch.float32), b.double()[None], "float32")


def test_pair_rows_in_portions_with_the_previous_token_in_the_state():
    from pico_vllm_amd.ops import kernels
    big = {"buckets": 13, "mul_prev": 40000, "mul_cur": 70001}
    H, V = 24, 60000
    table = torch.randn(big["buckets"] + 1, H).to(torch.bfloat16)
    rng = random.Random(3)
    seqs = [[rng.randrange(V) for _ in range(n)] for n in (9, 1, 14)]
    last = torch.full((5,), 7, dtype=torch.int32, device=DEV)        # slots hold what an earlier request left
    got = [[] for _ in seqs]
    fed = [0, 0, 0]
    for portions in ([3, 1, 2], [1, 0, 5], [5, 0, 1], [0, 0, 6]):
        live = [b for b, n in enumerate(portions) if n]
        toks = [t for b in live for t in seqs[b][fed[b]:fed[b] + portions[b]]]
        ctx = step_ctx([portions[b] for b in live], [fed[b] for b in live], [[3, 0, 1][b] for b in live], toks)
        resid = torch.zeros(len(toks), H, device=DEV)
        kernels.pair_embed(resid, table.to(DEV), ctx, last, big["mul_prev"], big["mul_cur"], big["buckets"])
        at = 0
        for b in live:
            got[b].append(resid[at:at + portions[b]].cpu())
            at += portions[b]
            fed[b] += portions[b]
    for b, toks in enumerate(seqs):
        assert torch.equal(torch.cat(got[b]), table.float()[P.pair_rows(toks, big)])
    assert last.tolist()[3] == seqs[0][-1] and last.tolist()[0] == seqs[1][-1] and last.tolist()[1] == seqs[2][-1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("halves", [False, True])
def test_rotation_in_place_in_both_layouts(dtype, halves):
    from pico_vllm_amd.ops import kernels
    from pico_vllm_amd.parts.rotary import scaled_frequencies
    T, heads, stride, rot, col0 = 11, 3, 20, 12, 5
    rotd = {"dims": rot, "base": 300.0, "scaling": YARN}
    x = torch.randn(T, col0 + heads * stride + 3).to(DT[dtype])
    pos = torch.tensor([0, 1, 2, 50, 51, 400, 7, 8, 9, 1000, 3], dtype=torch.int32)
    f, mag = scaled_frequencies(rot, 300.0, (4.0, 64, 8.0, 1.0))
    table = kernels.rope_table(pos.to(DEV), torch.tensor(f, dtype=torch.float64).float().to(DEV), mag)
    got = kernels.rope_inplace(x.to(DEV).clone(), col0, heads, stride, rot, table, halves)
    want = x.double().clone()
    heads_view = want[:, col0:col0 + heads * stride].reshape(T, heads, stride)
    want[:, col0:col0 + heads * stride] = P.rotate(heads_view, pos, rotd, "halves" if halves else "pairs").reshape(T, -1)
    close(got, want, dtype)
    assert torch.equal(got[:, :col0].cpu(), x[:, :col0]) and torch.equal(got[:, col0 + heads * stride:].cpu(), x[:, col0 + heads * stride:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,n_in,n_out,copy", [(3, 3, 24, 56, 8), (70, 4, 32, 96, 32), (1, 1, 64, 64, 0), (5, 2, 6, 28, 10)])
def test_a_product_per_head(dtype, T, H, n_in, n_out, copy):
    from pico_vllm_amd.ops import kernels
    x = torch.randn(T, H * (n_in + copy)).to(DT[dtype])
    w = (torch.randn(H, n_in, n_out) * n_in ** -0.5).to(DT[dtype])
    got = kernels.head_linear(x.to(DEV), 0, n_in + copy, w.to(DEV), H, copy=copy)
    xv = x.double().view(T, H, n_in + copy)
    want = torch.cat([torch.einsum("thi,hio->tho", xv[..., :n_in], w.double()), xv[..., n_in:]], -1).reshape(T, -1)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C,N,taps,R", [(100, 12, 3, 5), (256, 16, 4, 8), (160, 80, 2, 7), (36, 5, 1, 3), (40, 200, 5, 4)])
def test_convolution_and_recurrence_in_portions_and_token_by_token(dtype, C, N, taps, R):
    """Three sequences in slots that were used before (zeroed as the engine does for a new request): whole, in portions
    down to one token beside each other, and cut into chunks that run side by side, against the plain walk."""
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(C + N)
    lens = [37, 5, 18]
    dt_ = DT[dtype]
    mk = lambda *s: torch.randn(*s, generator=g)
    w, cb = mk(C, taps) * taps ** -0.5, 0.3 * mk(C)
    a_log, D, dtb = torch.log(0.5 + 4 * torch.rand(C, N, generator=g)), 1 + 0.3 * mk(C), torch.log(torch.expm1(0.01 + 0.2 * torch.rand(C, generator=g)))
    seqs = []
    for n in lens:
        seqs.append(dict(uz=mk(n, 2 * C).to(dt_), dbc=mk(n, R + 2 * N).to(dt_), dtp=0.5 * mk(n, C)))
    want = []
    for s in seqs:
        u = P.silu(P.causal_conv(s["uz"][:, :C].double(), w.double(), cb.double())).to(dt_).double()      # the engine keeps it in its storage type
        dt = P.softplus(s["dtp"].double() + dtb.double())
        y, _ = P.selective_scan(u, dt, -torch.exp(a_log.double()), s["dbc"][:, R:R + N].double(), s["dbc"][:, R + N:].double(), D.double())
        want.append((u, y * P.silu(s["uz"][:, C:].double())))
    dev = lambda t: t.to(DEV).contiguous()
    plans = [([[37, 5, 18]], 0), ([[2, 1, 7], [30, 3, 1], [1, 1, 9], [4, 0, 1]], 0), ([[1, 1, 1]] * 5 + [[32, 0, 13]], 0)]
    if dtype == "bfloat16":          # chunks that run side by side: of 4 and of 16 tokens, sequences of unequal numbers of chunks
        plans += [([[37, 5, 18]], 4), ([[20, 2, 1], [17, 3, 17]], 16)]
    for portions, chunk in plans:
        state = torch.full((5, C, N + taps - 1), 9.0, device=DEV)
        slots = [4, 0, 2]
        state[slots] = 0
        fed, got_u, got_y = [0, 0, 0], [[], [], []], [[], [], []]
        for step in portions:
            live = [b for b, n in enumerate(step) if n]
            ctx = step_ctx([step[b] for b in live], [fed[b] for b in live], [slots[b] for b in live])
            cat = lambda k: dev(torch.cat([seqs[b][k][fed[b]:fed[b] + step[b]] for b in live]))
            uz, dbc, dtp = cat("uz"), cat("dbc"), cat("dtp")
            u = kernels.causal_conv(uz, C, dev(w.t()), dev(cb), ctx, state, N, single=all(n == 1 for n in step if n))
            y = kernels.selective_scan(u, dtp, dev(dtb), dbc, R, R + N, dev(a_log), dev(D), uz[:, C:], ctx, state, taps - 1, chunk=chunk)
            at = 0
            for b in live:
                got_u[b].append(u[at:at + step[b]])
                got_y[b].append(y[at:at + step[b]])
                at += step[b]
                fed[b] += step[b]
        for b in range(3):
            close(torch.cat(got_u[b]), want[b][0], dtype)
            close(torch.cat(got_y[b]), want[b][1], dtype, scale=2.0)
        assert float(state[1].min()) == 9.0 and float(state[3].max()) == 9.0           # other requests' slots untouched


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,dk,dv,decay", [(2, 24, 40, (0.9, 0.996)), (4, 64, 64, (0.97, 0.99, 0.999, 1.0)), (3, 16, 8, (0.5, 0.9375, 0.99)), (1, 80, 100, (0.999,))])
def test_retention_recurrence_with_fixed_decays(dtype, H, dk, dv, decay):
    """Whole (in bfloat16 long enough to be cut into chunks that run side by side), in portions and token by token."""
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(dk)
    n = 300
    x = torch.randn(n, 2 * H * dk + H * dv, generator=g).to(DT[dtype])
    q, k, v = (x.double()[:, a:b].reshape(n, H, -1) for a, b in ((0, H * dk), (H * dk, 2 * H * dk), (2 * H * dk, 2 * H * dk + H * dv)))
    want, S = P.retention_recurrence(q, k * dk ** -0.5, v, torch.tensor(decay, dtype=torch.float64))
    dec = torch.tensor(decay, dtype=torch.float64).float().to(DEV)
    for portions, chunk in (([300], 0), ([300], 64 if dtype == "bfloat16" else 0), ([2, 129, 1, 1, 60, 7, 100], 0), ([250] + [1] * 50, 0)):
        state = torch.zeros(3, H, dk, dv, device=DEV)
        out, at = [], 0
        for m in portions:
            ctx = step_ctx([m], [at], [1])
            out.append(kernels.gla_scan(x[at:at + m].to(DEV), 0, H * dk, 2 * H * dk, None, ctx.cu_seqlens, ctx.state_slots, state, 1,
                                        H, dk, dv, dk ** -0.5, chunk=chunk if m >= 128 else 0, head_decay=dec))
            at += m
        close(torch.cat(out).view(n, H, dv), want, "float32" if dtype == "float32" else "bfloat16", scale=0.2 if dtype == "bfloat16" else 5.0)
        close(state[1] * dk ** -0.5, S, "float32", scale=20.0)      # the state holds k as it is; the scale sits on the read-out
        assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


def test_a_decay_of_one_keeps_the_first_token_for_good():
    """One key and value at the start, nothing after it: with decay 1 the read-out 2,000 tokens later is what it was."""
    from pico_vllm_amd.ops import kernels
    H, dk, dv, n = 2, 16, 8, 2000
    x = torch.zeros(n, 2 * H * dk + H * dv)
    x[0, H * dk:2 * H * dk] = 1.0
    x[0, 2 * H * dk:] = torch.arange(1, H * dv + 1).float()
    x[:, :H * dk] = 1.0                                                  # every query reads the sum over the key channels
    for portions in ([n], [7, 1500, 493]):
        state = torch.zeros(2, H, dk, dv, device=DEV)
        out, at = [], 0
        for m in portions:
            ctx = step_ctx([m], [at], [0])
            out.append(kernels.gla_scan(x[at:at + m].to(DEV), 0, H * dk, 2 * H * dk, None, ctx.cu_seqlens, ctx.state_slots, state, 1, H, dk,
                                        dv, 1.0, head_decay=torch.tensor([1.0, 0.5], device=DEV)))
            at += m
        o = torch.cat(out).cpu()
        assert torch.equal(o[-1, :dv], dk * torch.arange(1, dv + 1).float()) and float(o[-1, dv:].abs().max()) == 0.0


@pytest.mark.parametrize("E,top,T,D,extra", [(5, 2, 33, 72, 1), (6, 3, 200, 128, 1), (3, 3, 9, 96, 0), (16, 1, 70, 44, 1)])
def test_router_choice_by_logits_and_weights_over_the_chosen(E, top, T, D, extra):
    from pico_vllm_amd.ops import kernels
    g = torch.Generator().manual_seed(E)
    h, wr, b = torch.randn(T, D, generator=g), torch.randn(E + extra, D, generator=g) * D ** -0.5, torch.randn(E, generator=g)
    idx, wt, z = P.route(h.double(), wr[:E].double(), b.double(), top)
    ex, w, zz = kernels.moe_router_top_softmax(h.to(DEV), wr.to(DEV), b.to(DEV), E, top)
    sure = P.route_margin(z, top) > 1e-4
    assert bool(sure.float().mean() > 0.9)
    assert torch.equal(ex.cpu().long()[sure], idx[sure])
    close(w[sure.to(DEV)], wt[sure], "float32")
    close(zz[:, :E], z, "float32")
    if extra:
        close(zz[:, E:], h.double() @ wr[E:].double().T, "float32")       # the rider's logit: no bias, no part in the choice
    assert float(w.sum(-1).sub(1).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_attention_pieces_against_the_heads_spelled_out(dtype):
    """The cache rows [latent | turned part], the queries carried into the latent's space and the attention over one
    key/value head, against keys and values of every head made from the latent."""
    from pico_vllm_amd.ops import kernels
    from pico_vllm_amd.parts.rotary import scaled_frequencies
    H, d, r, dv, Rq, R, n, Pg = 3, 24, 8, 20, 40, 56, 50, 16
    m = {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "q_rank": Rq, "kv_rank": R, "scale": 0.4, "rot": {"dims": r, "base": 100.0, "scaling": YARN}}
    g = torch.Generator().manual_seed(1)
    dt_ = DT[dtype]
    y = torch.randn(n, Rq + R + r, generator=g).to(dt_)
    wq, wkv = 1 + 0.2 * torch.randn(Rq, generator=g), 1 + 0.2 * torch.randn(R, generator=g)
    uq = (torch.randn(H * (d + r), Rq, generator=g) * Rq ** -0.5).to(dt_)
    uk, uv = (torch.randn(H * d, R, generator=g) * R ** -0.5).to(dt_), (torch.randn(H * dv, R, generator=g) * R ** -0.5).to(dt_)
    pos = torch.arange(n)
    f, mag = scaled_frequencies(r, 100.0, (4.0, 64, 8.0, 1.0))
    table = kernels.rope_table(pos.int().to(DEV), torch.tensor(f, dtype=torch.float64).float().to(DEV), mag)
    pages = 6
    kc, vc = torch.zeros(pages, 1, Pg, R + r, dtype=dt_, device=DEV), torch.zeros(pages, 1, R, Pg, dtype=dt_, device=DEV)
    order = [4, 1, 5, 0]
    slots = torch.tensor([order[t // Pg] * Pg + t % Pg for t in range(n)], dtype=torch.int32, device=DEV)
    cq = kernels.latent_prepare(y.to(DEV), Rq, R, r, wq.to(DEV), wkv.to(DEV), 1e-5, table, slots, kc, vc)
    yd = y.double()
    want_cq = P.rms_norm(yd[:, :Rq], wq.double(), 1e-5)
    c = P.rms_norm(yd[:, Rq:Rq + R], wkv.double(), 1e-5)
    kr = P.rotate(yd[:, None, Rq + R:], pos, m["rot"], "pairs")[:, 0]
    close(cq, want_cq, dtype)
    rows = torch.stack([kc[order[t // Pg], 0, t % Pg] for t in range(n)])
    close(rows, torch.cat([c, kr], -1), dtype)
    close(torch.stack([vc[order[t // Pg], 0, :, t % Pg] for t in range(n)]), c, dtype)
    # from here on with what the engine holds (rounded to its storage type)
    cq_s, c_s, kr_s = cq.double().cpu(), rows[:, :R].double().cpu(), rows[:, R:].double().cpu()
    q = (cq_s @ uq.double().T).to(dt_)
    qd = q.double().view(n, H, d + r)
    q_rot = P.rotate(qd[..., d:], pos, m["rot"], "pairs")
    s = (torch.einsum("ihd,jhd->hij", qd[..., :d], (c_s @ uk.double().T).view(n, H, d)) + torch.einsum("ihd,jd->hij", q_rot, kr_s)) * m["scale"]
    s = s.masked_fill(~(pos[None, :] <= pos[:, None])[None], float("-inf"))
    want = torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), (c_s @ uv.double().T).view(n, H, dv)).reshape(n, -1)
    qg = q.to(DEV).clone()
    ql = kernels.head_linear(qg, 0, d + r, uk.to(DEV).view(H, d, R).contiguous(), H, copy=r, turn=table)     # turned on the way
    kernels.rope_inplace(qg, d, H, d + r, r, table, False)
    assert torch.equal(ql, kernels.head_linear(qg, 0, d + r, uk.to(DEV).view(H, d, R).contiguous(), H, copy=r))   # or beforehand
    bt = torch.tensor([order], dtype=torch.int32, device=DEV)
    ol = kernels.attn_bias_plain(ql, kc, vc, bt, pos.int().to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV), H, 1, R + r, R, m["scale"], 0)
    got = kernels.head_linear(ol, 0, R, uv.to(DEV).view(H, dv, R).transpose(1, 2).contiguous(), H)
    close(got, want, dtype, scale=3.0)


# ---------------------------------------------------------------------------------------------------------------
# whole models through the replayer
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


def test_a_far_key_that_stands_out_in_prompts_portions_and_decoding():
    """One latent-attention layer with a scale so large that every query's softmax sits on very few keys, many of them
    hundreds of tokens back and on other pages: a key read from a wrong place shows in the logits."""
    cfg = config(64, 64, [(latent(2, 16, 16, 16, 32, 32, scale=3.0, base=10000.0), moe(2, 1, 16))], bigram=(31, 3, 5))
    t = P.random_model(cfg, 5)
    d = write_model(cfg, t, "dikolix_far_")
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
            margins = []
            logits = P.forward(cfg, t, toks, margins_out=margins)[-1]
            if dtype == "bfloat16" and float(torch.stack(margins).min()) < CLOSE_CALL:
                break                      # a choice of experts that a rounding may turn: from here on no fault
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
def draw_config(seed):
    """Sizes, head counts, order of layers, constants, the loop: all drawn; returns (config, page size)."""
    rng = random.Random(1000 + seed)
    width = rng.choice([40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(2, 4)):
        kind = rng.choice(["latent", "ssm", "retention"])
        if kind == "latent":
            rot = rng.choice([4, 8, 16, 32])
            sc = rng.choice([None, {"factor": rng.choice([2.0, 4.0, 16.0]), "original": rng.choice([16, 64, 256]), "fast": rng.choice([4.0, 32.0]),
                                    "slow": rng.choice([0.5, 1.0])}])
            mx = latent(rng.randint(1, 5), rng.choice([8, 16, 24, 32]), rot, rng.choice([8, 16, 40]), rng.choice([16, 24, 64]),
                        rng.choice([16, 32, 48, 96]), scale=rng.choice([0.1, 0.25, 0.4]), base=rng.choice([100.0, 10000.0, 1e6]), scaling=sc)
        elif kind == "ssm":
            mx = ssm(rng.choice([48, 80, 128, 200]), rng.choice([4, 16, 24, 64, 130]), rng.randint(1, 5), rng.choice([2, 8, 12]))
        else:
            H, dk = rng.randint(1, 4), rng.choice([8, 16, 32, 48])
            mx = retention(H, dk, rng.choice([8, 32, 72]), [rng.choice([0.8, 0.95, 0.99, 0.999, 1.0]) for _ in range(H)],
                           rot_dims=rng.choice([None, dk, dk // 2 // 2 * 2 or 2]), base=rng.choice([100.0, 1e5]))
        E = rng.randint(1, 8)
        ff = None if rng.random() < 0.15 else moe(E, rng.randint(1, min(E, 4)), rng.choice([8, 24, 32]), shared=rng.choice([None, 16, 40]))
        layers.append((mx, ff))
    n = len(layers)
    start = rng.randint(0, n - 1)
    loop = rng.choice([None, (start, rng.randint(start + 1, n), rng.randint(1, 3))])
    big = rng.choice([None, (rng.choice([1, 17, 251]), rng.randint(0, 40), rng.randint(1, 40))])
    return config(rng.choice([33, 100, 256]), width, layers, eps=rng.choice([1e-5, 1e-6]), mult=rng.choice([None, 0.5, 1.2]), bigram=big,
                  loop=loop), rng.choice([8, 16, 32])


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random_in_mixed_batches(seed):
    cfg, page = draw_config(seed)
    t = P.random_model(cfg, seed)
    d = write_model(cfg, t, f"dikolix_draw{seed}_")
    name = f"draw{seed}"
    reqs = requests(cfg["vocab"], [60, 21, 90, 5, 44], seed=seed)
    steps, peak = mixed_steps(reqs, page, seed=seed, tail=8)
    for dtype in ("float32", "bfloat16"):
        rows, _ = replay(d, dtype, steps, peak, page, max_live=3)
        compare(name, dtype, rows, reqs, cfg=cfg, tensors=t)


def draw_larger_config(seed):
    """Sizes the matrix-core kernels take (latents and rotated parts in multiples of 32 and 16, widths of 128 to 384, up
    to 24 experts), every mixer at least once, a loop more often than not."""
    rng = random.Random(5000 + seed)
    width = rng.choice([128, 192, 256, 384])
    kinds = ["latent", "ssm", "retention"] + [rng.choice(["latent", "ssm", "retention"]) for _ in range(rng.randint(0, 2))]
    rng.shuffle(kinds)
    layers = []
    for kind in kinds:
        if kind == "latent":
            rot = rng.choice([32, 64])
            kv = rng.choice([32, 64, 96, 160, 224])
            mx = latent(rng.choice([2, 4, 5, 8, 16]), rng.choice([16, 32, 64]), rot, rng.choice([16, 32, 64]), rng.choice([64, 96, 192]), kv,
                        scale=rng.choice([0.08, 0.15]), base=rng.choice([10000.0, 500000.0]),
                        scaling=rng.choice([None, {"factor": 4.0, "original": 128, "fast": 16.0, "slow": 1.0}]))
        elif kind == "ssm":
            mx = ssm(rng.choice([256, 384, 512]), rng.choice([8, 16, 32, 64]), rng.choice([2, 4]), rng.choice([8, 16, 24]))
        else:
            H, dk = rng.choice([2, 4, 6]), rng.choice([32, 64, 128])
            mx = retention(H, dk, rng.choice([32, 64, 128]), [1.0 - 2.0 ** -rng.randint(3, 11) for _ in range(H)],
                           rot_dims=rng.choice([None, dk, dk // 2]), base=rng.choice([10000.0, 1e6]))
        E = rng.choice([4, 8, 16, 24])
        layers.append((mx, moe(E, rng.randint(1, 4), rng.choice([32, 64, 128]), shared=rng.choice([None, 64, 128]))))
    n = len(layers)
    start = rng.randint(0, n - 2)
    loop = rng.choice([None, (start, rng.randint(start + 1, n), 2), (start, rng.randint(start + 1, n), 3)])
    return config(rng.choice([300, 512]), width, layers, mult=rng.choice([0.5, 0.7, 1.0]), bigram=(rng.choice([509, 4093]), rng.randint(1, 99), rng.randint(1, 99)),
                  loop=loop), rng.choice([16, 32, 64])


@pytest.mark.parametrize("seed", range(4))
def test_larger_configurations_drawn_at_random_with_long_requests(seed):
    """Requests of up to 500 tokens in portions of up to 200 beside one another (steps of more than 128 tokens, whose
    recurrences the bfloat16 engine cuts into chunks that run side by side, several sequences a step) and single tokens."""
    cfg, page = draw_larger_config(seed)
    t = P.random_model(cfg, 100 + seed)
    d = write_model(cfg, t, f"dikolix_large{seed}_")
    name = f"large{seed}"
    reqs = requests(cfg["vocab"], [500, 150, 330, 40], seed=seed)
    rng = random.Random(seed)
    waiting, live, steps, peak = list(reqs), {}, [], 0
    sizes = [130, 7, 64, 200, 2]
    while waiting or live:
        while waiting and len(live) < 3:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            toks, at = reqs[rid], live[rid]
            last = len(toks) - at <= 6
            n = 1 if last else min(sizes[rng.randrange(len(sizes))], len(toks) - 6 - at)
            entries.append((rid, toks[at:at + n], [n - 1] if n > 8 else range(n)))
            live[rid] = at + n
            if live[rid] == len(toks):
                end.append(rid)
        peak = max(peak, sum(roundup(live[r], page) for r in live))
        for rid in end:
            del live[rid]
        steps.append((entries, end))
    for dtype in ("float32", "bfloat16"):
        rows, _ = replay(d, dtype, steps, roundup(peak), page, max_live=3)
        compare(name, dtype, rows, reqs, cfg=cfg, tensors=t)
