"""The plain implementation of Vagelix pinned by cases worked out by hand, and what needs no GPU of the design in the
package: the configuration reader, the model description, the cache needs that reach the cache manager."""
import copy
import math

import pytest
import torch

import plain_vagelix as P
from vagelix_configs import CONFIGS, model_dir, tensors_of

F = torch.float64


def test_rms_has_eps_inside_the_root():
    x = torch.tensor([3.0, 4.0], dtype=F)
    assert torch.allclose(P.rms(x, 0.5), x / math.sqrt(12.5 + 0.5))


def test_visibility_in_chunks_counted_from_position_zero():
    assert P.chunk_visible(5, 5, 3) and P.chunk_visible(5, 3, 3) and not P.chunk_visible(5, 2, 3)
    assert not P.chunk_visible(3, 4, 3) and P.chunk_visible(6, 6, 3) and not P.chunk_visible(6, 5, 3)
    assert P.chunk_visible(100, 0, 0)                                   # no mask: every earlier position
    assert [j for j in range(8) if P.chunk_visible(7, j, 1)] == [7]


def test_temperature_steps_with_the_position():
    assert P.query_temperature(0, 0.3, 4) == 1.0 and P.query_temperature(2, 0.3, 4) == 1.0
    assert P.query_temperature(3, 0.3, 4) == pytest.approx(1 + 0.3 * math.log(2))
    assert P.query_temperature(11, 0.3, 4) == pytest.approx(1 + 0.3 * math.log(4))


def test_rotation_pairs_halves_and_depends_on_the_distance_only():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=F)            # dims 4: pairs (0, 2) and (1, 3); entry 4 passes
    y = P.rotate_half(x, torch.tensor([1]), 4, 100.0)[0, 0]
    a0, a1 = 1.0, 100.0 ** -0.5
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0]
    assert torch.allclose(y, torch.tensor(want, dtype=F))
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=F), torch.randn(1, 1, 8, generator=g, dtype=F)
    dot = lambda i, j: float((P.rotate_half(q, torch.tensor([i]), 6, 50.0) * P.rotate_half(k, torch.tensor([j]), 6, 50.0)).sum())
    assert dot(9, 4) == pytest.approx(dot(105, 100))


def test_a_sink_takes_its_share_of_the_softmax():
    """One head, one key: p = e^s / (1 + e^s) on the key itself; the output is that share of the key as projected."""
    D = 4
    m = {"heads": 1, "kv_heads": 1, "dim": D, "vdim": D, "scale": 0.5}
    w = {"q": torch.eye(D, dtype=F), "k": torch.eye(D, dtype=F), "q.b": torch.zeros(D, dtype=F), "k.b": torch.ones(D, dtype=F),
         "q.norm": torch.ones(D, dtype=F), "k.norm": torch.ones(D, dtype=F), "g": torch.zeros(1, D, dtype=F), "o": torch.eye(D, dtype=F)}
    h = torch.tensor([[1.0, -2.0, 0.5, 3.0]], dtype=F)
    out = P.chunked_sink_attention(h, w, m, 0.0)
    q, k = P.rms(h, 0.0), P.rms(h + 1.0, 0.0)
    s = float((q * k).sum()) * 0.5
    assert torch.allclose(out, math.exp(s) / (1 + math.exp(s)) * (h + 1.0) * 0.5)         # gate sigmoid(0) = 1/2


def test_the_two_maps_are_subtracted_and_the_result_normed():
    """One token: both maps return the value itself, so o = (1 - lambda) v, normed: only its sign and (1 - diff) stay."""
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 3, "scale": 1.0, "diff": 0.25}
    g = torch.Generator().manual_seed(1)
    w = {n: torch.randn(s, generator=g, dtype=F) for n, s in (("q", (4, 5)), ("k", (4, 5)), ("v", (3, 5)))}
    w.update({"q.norm": torch.ones(2, dtype=F), "k.norm": torch.ones(2, dtype=F), "o": torch.eye(3, dtype=F)})
    w.update({n: torch.full((2,), 0.1, dtype=F) for n in ("lq1", "lk1", "lq2", "lk2")})
    h = torch.randn(1, 5, generator=g, dtype=F)
    lam = P.diff_lambda(w["lq1"], w["lk1"], w["lq2"], w["lk2"], 0.25)
    assert lam == pytest.approx(0.25)                                    # the two exponentials cancel
    v = h @ w["v"].T
    assert torch.allclose(P.differential_attention(h, w, m, 0.0), P.rms(v, 0.0) * 0.75)


def test_delta_rule_by_hand_and_through_a_state():
    """First token from zero: S = beta k v^T, o = beta (k . q) v.  A second token with the same unit key and no decay
    replaces the part of the value that the first wrote: u = beta (v2 - beta v1)."""
    k = torch.tensor([[[0.6, 0.8]]], dtype=F).repeat(2, 1, 1)
    q = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=F)
    v = torch.tensor([[[1.0, 2.0, 3.0]], [[-1.0, 0.0, 4.0]]], dtype=F)
    g = torch.ones(2, 1, 2, dtype=F)
    beta = torch.tensor([[0.5], [0.25]], dtype=F)
    o, S = P.delta_rule_scan(q, k, v, g, beta)
    assert torch.allclose(o[0, 0], 0.5 * 0.6 * v[0, 0])
    u2 = 0.25 * (v[1, 0] - 0.5 * v[0, 0])
    assert torch.allclose(S[0], torch.outer(k[0, 0], 0.5 * v[0, 0] + u2))
    assert torch.allclose(o[1, 0], 0.8 * (0.5 * v[0, 0] + u2))
    o1, S1 = P.delta_rule_scan(q[:1], k[:1], v[:1], g[:1], beta[:1])
    o2, S2 = P.delta_rule_scan(q[1:], k[1:], v[1:], g[1:], beta[1:], S1)
    assert torch.allclose(o2[0], o[1]) and torch.allclose(S2, S)
    # a decay acts on the rows of the state that belong to its key channels, before the read
    gd = torch.tensor([[[1.0, 1.0]], [[0.5, 0.0]]], dtype=F)
    _, Sd = P.delta_rule_scan(q, k, v, gd, torch.tensor([[0.5], [0.0]], dtype=F))
    assert torch.allclose(Sd[0], torch.tensor([[0.5], [0.0]], dtype=F) * torch.outer(k[0, 0], 0.5 * v[0, 0]))


def test_state_space_walk_against_its_closed_form():
    T, a, dt = 6, 0.7, 0.3
    x = torch.ones(T, 1, 2, dtype=F)
    B = torch.full((T, 1, 3), 2.0, dtype=F)
    C = torch.ones(T, 1, 3, dtype=F)
    y, S = P.ssd_scan(x, B, C, torch.full((T, 1), dt, dtype=F), torch.tensor([a], dtype=F), torch.tensor([0.5], dtype=F))
    r = math.exp(-a * dt)
    for t in range(T):
        s = dt * 2.0 * sum(r ** j for j in range(t + 1))                 # every state element
        assert y[t, 0, 0].item() == pytest.approx(3 * s + 0.5)
    y1, S1 = P.ssd_scan(x[:2], B[:2], C[:2], torch.full((2, 1), dt, dtype=F), torch.tensor([a], dtype=F), torch.tensor([0.5], dtype=F))
    y2, S2 = P.ssd_scan(x[2:], B[2:], C[2:], torch.full((4, 1), dt, dtype=F), torch.tensor([a], dtype=F), torch.tensor([0.5], dtype=F), S1)
    assert torch.allclose(torch.cat([y1, y2]), y) and torch.allclose(S2, S)


def test_convolution_with_a_history_equals_the_whole():
    g = torch.Generator().manual_seed(2)
    x, taps, b = torch.randn(9, 5, generator=g, dtype=F), torch.randn(5, 4, generator=g, dtype=F), torch.randn(5, generator=g, dtype=F)
    whole = P.causal_conv(x, taps, b)
    assert torch.allclose(whole[0], x[0] * taps[:, 3] + b)               # zeros before the start; the last column is the token's own
    assert torch.allclose(P.causal_conv(x[4:], taps, b, history=x[1:4]), whole[4:])


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_a_prefix_does_not_depend_on_what_follows(name):
    toks = [(7 * i + 3) % CONFIGS[name]["vocab"] for i in range(40)]
    full = P.forward(CONFIGS[name], tensors_of(name), toks)
    part = P.forward(CONFIGS[name], tensors_of(name), toks[:23])
    assert torch.allclose(full[:23], part, atol=1e-9)


def test_a_layer_that_runs_another_layers_tensors():
    cfg = CONFIGS["a"]
    assert P.weight_owner(cfg["layers"], 3) == 1 and not any(n.startswith("l3.") for n in tensors_of("a"))
    other = copy.deepcopy(cfg)
    del other["layers"][3]["weights_of"]                                 # the same tensors under the fourth layer's own names
    t = dict(tensors_of("a"))
    t.update({"l3." + n[3:]: v for n, v in tensors_of("a").items() if n.startswith("l1.")})
    toks = list(range(30))
    assert torch.equal(P.forward(cfg, tensors_of("a"), toks), P.forward(other, t, toks))


# ---- the package's side, without a GPU -----------------------------------------------------------------------------------
def _description(name):
    from pico_vllm_amd.config.registry import load_model_description
    return load_model_description(model_dir(name))


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_model_description_names_exactly_the_checkpoints_tensors(name):
    from pico_vllm_amd.parts.model import model_param_specs
    _, cfg, spec = _description(name)
    want = {p.name: tuple(p.shape) for p in model_param_specs(spec)}
    assert want == {n: tuple(v.shape) for n, v in tensors_of(name).items()}
    layers = CONFIGS[name]["layers"]
    owners = [i for i, l in enumerate(layers) if l.get("weights_of") is None]
    assert [e.layer for e in spec.run_order] == [owners.index(P.weight_owner(layers, i)) for i in range(len(layers))]
    assert all(e.cache_of is None for e in spec.run_order)               # every run has a cache and state of its own


def test_the_low_rank_sizes_come_from_the_checkpoint():
    _, cfg, _ = _description("a")
    assert (cfg.layers[1].mixer.right.decay_rank, cfg.layers[1].mixer.right.gate_rank) == (6, 5)
    from pico_vllm_amd.config.vagelix import VagelixConfig
    raw = copy.deepcopy(CONFIGS["a"])
    shapes = {n: tuple(v.shape) for n, v in P.random_model(raw, 0, decay_rank=9, gate_rank=2).items()}
    right = VagelixConfig.from_dict(raw, shapes).layers[3].mixer.right    # the layer that runs layer 1's tensors
    assert (right.decay_rank, right.gate_rank) == (9, 2)


def test_what_the_configuration_refuses():
    from pico_vllm_amd.config.model_config import ConfigError
    from pico_vllm_amd.config.vagelix import VagelixConfig

    def broken(change):
        raw = copy.deepcopy(CONFIGS["a"])
        change(raw)
        with pytest.raises(ConfigError):
            VagelixConfig.from_dict(raw)
    broken(lambda r: r["layers"][0].update(type="other"))
    broken(lambda r: r["layers"][0]["mixer"].pop("diff"))
    broken(lambda r: r["layers"][1]["mixer"]["left"].update(vdim=24))        # the values are the keys
    broken(lambda r: r["layers"][1]["mixer"]["left"]["rot"].update(dims=7))
    broken(lambda r: r["layers"][2]["mixer"].update(groups=2))               # three heads in two groups
    broken(lambda r: r["layers"][3].update(weights_of=3))
    broken(lambda r: r["layers"][3]["mixer"]["right"].update(conv=3))        # other sizes than the layer whose tensors it runs
    broken(lambda r: r["layers"][0]["mlp"].update(kind="moe"))
    broken(lambda r: r.pop("norm"))
    # what a configuration does not mention does not exist
    cfg = VagelixConfig.from_dict(CONFIGS["c"])
    assert cfg.layers[0].mixer.left.chunk == 0 and cfg.layers[0].mixer.left.rot_dims == 0 and cfg.layers[1].mixer.temp_every == 0
    assert cfg.layers[1].ff == 0


def test_every_mixer_asks_the_cache_manager_for_what_it_keeps():
    import torch as _t
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.parts.model import DecoderModel
    _, _, spec = _description("b")
    model = DecoderModel(spec, _t.float32, "cpu")
    specs = model.cache_specs()
    # runs: duality (state + taps), attention, pair (pages, state + taps), and the attention's tensors twice more
    paged = [k for k, s in specs.items() if s.kind == "paged_kv"]
    states = [k for k, s in specs.items() if s.kind == "state"]
    assert sorted(map(str, paged)) == sorted(map(str, [1, (2, 0), 3, 4])) and len(states) == 4
    m = CacheManager(specs, 8, 64, 3)
    assert len(m.groups) == 2 and sorted(len(g.layers) for g in m.groups) == [1, 3]
    assert {g.spec.chunk for g in m.groups} == {0, 40}


def test_pages_of_passed_chunks_are_given_back():
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.parts.spec import CacheSpec, PageTensor
    spec = CacheSpec("paged_kv", chunk=20, page_tensors=(PageTensor("k", (1, "page", 4)),))
    m = CacheManager({0: spec}, 8, 16, 2)
    assert m.add_request("r") and m.grow("r", 45)
    m.advance("r", 19)
    assert m.num_free_pages() == 10                                       # the next query may still read position 0
    m.advance("r", 20)                                                    # position 20 starts a chunk: pages 0, 1 hold 0 .. 15
    assert m.block_table("r")[:3] == [-1, -1, m.block_table("r")[2]] and m.num_free_pages() == 12
    m.advance("r", 45)                                                    # the chunk of 40 .. 59; page 4 holds 32 .. 39
    assert [p >= 0 for p in m.block_table("r")] == [False] * 5 + [True]
    m.check()
    m.free_request("r")
    assert m.num_free_pages() == 16
