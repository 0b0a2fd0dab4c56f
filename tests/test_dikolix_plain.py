"""The plain Dikolix implementation pinned by cases worked out by hand, and what needs no GPU of the engine's side: the
configuration reader, the run order, the model description against the checkpoint's tensors."""
import math

import pytest
import torch

import plain_dikolix as P
from dikolix_configs import CONFIGS, YARN, config, latent, moe, retention, ssm, tensors_of


def test_pair_rows_by_hand():
    big = {"buckets": 7, "mul_prev": 3, "mul_cur": 5}
    assert P.pair_rows([4, 2, 6], big) == [7, (4 * 3 + 2 * 5) % 7, (2 * 3 + 6 * 5) % 7]
    assert P.pair_rows([0], big) == [7]


def test_run_order_with_and_without_a_loop():
    c = config(10, 8, [(ssm(8, 2, 2, 2), None)] * 4, loop=(1, 3, 3))
    assert P.run_order(c) == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert P.run_order(config(10, 8, [(ssm(8, 2, 2, 2), None)] * 2)) == [(0, False), (1, False)]
    assert P.run_order(config(10, 8, [(ssm(8, 2, 2, 2), None)] * 2, loop=(0, 2, 2))) == [(0, False), (1, False), (0, True), (1, False)]
    assert P.run_order(config(10, 8, [(ssm(8, 2, 2, 2), None)] * 2, loop=(0, 1, 1))) == [(0, False), (1, False)]


def test_layer_norm_by_hand():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=torch.float64)
    y = P.layer_norm(x, torch.tensor([1.0, 1.0, 2.0, 1.0], dtype=torch.float64), torch.tensor([0.0, 0.5, 0.0, 0.0], dtype=torch.float64), 0.5)
    r = 1 / math.sqrt((4 + 1 + 0 + 9) / 4 + 0.5)
    assert torch.allclose(y, torch.tensor([[-2 * r, -r + 0.5, 0.0, 3 * r]], dtype=torch.float64))


def test_rotation_layouts():
    x = torch.arange(1, 9, dtype=torch.float64).view(1, 1, 8)
    rot = {"dims": 4, "base": 100.0}
    a, b = P.rotate(x, torch.tensor([3]), rot, "pairs"), P.rotate(x, torch.tensor([3]), rot, "halves")
    for i, f in enumerate((1.0, 0.1)):
        c, s = math.cos(3 * f), math.sin(3 * f)
        assert float(a[0, 0, 2 * i]) == pytest.approx(x[0, 0, 2 * i] * c - x[0, 0, 2 * i + 1] * s)
        assert float(a[0, 0, 2 * i + 1]) == pytest.approx(x[0, 0, 2 * i + 1] * c + x[0, 0, 2 * i] * s)
        assert float(b[0, 0, i]) == pytest.approx(x[0, 0, i] * c - x[0, 0, i + 2] * s)
        assert float(b[0, 0, i + 2]) == pytest.approx(x[0, 0, i + 2] * c + x[0, 0, i] * s)
    assert torch.equal(a[..., 4:], x[..., 4:]) and torch.equal(b[..., 4:], x[..., 4:])
    f, mag = P.rotation_frequencies({"dims": 16, "base": 10000.0, "scaling": YARN})
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0) and float(f[0]) == 1.0 and float(f[7]) == pytest.approx(10000.0 ** (-14 / 16) / 4)


def test_convolution_and_scan_by_hand():
    x = torch.tensor([[1.0], [2.0], [3.0]], dtype=torch.float64)
    w, b = torch.tensor([[10.0, 1.0]], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64)
    assert P.causal_conv(x, w, b).tolist() == [[1.5], [12.5], [23.5]]
    assert P.causal_conv(x[1:], w, b, history=x[:1]).tolist() == [[12.5], [23.5]]
    dt = torch.tensor([[0.5], [1.0]], dtype=torch.float64)
    A, B, C, D = torch.tensor([[-1.0, -2.0]], dtype=torch.float64), torch.ones(2, 2, dtype=torch.float64), torch.tensor([[1.0, 0.0], [1.0, 1.0]], dtype=torch.float64), torch.tensor([2.0], dtype=torch.float64)
    y, S = P.selective_scan(x[:2], dt, A, B, C, D)
    s0 = [0.5, 0.5]
    s1 = [math.exp(-1) * 0.5 + 2.0, math.exp(-2) * 0.5 + 2.0]
    assert y[0, 0] == pytest.approx(s0[0] + 2.0) and y[1, 0] == pytest.approx(s1[0] + s1[1] + 4.0)
    y2, _ = P.selective_scan(x[1:2], dt[1:], A, B[1:], C[1:], D, state=torch.tensor([s0], dtype=torch.float64))
    assert y2[0, 0] == pytest.approx(float(y[1, 0]))


def test_retention_by_hand_and_the_router():
    q = k = torch.ones(3, 1, 2, dtype=torch.float64)
    v = torch.tensor([[[1.0]], [[10.0]], [[100.0]]], dtype=torch.float64)
    o, S = P.retention_recurrence(q, k, v, torch.tensor([0.5], dtype=torch.float64))
    assert o[:, 0, 0].tolist() == [2.0, 2 * (0.5 + 10), 2 * (0.25 + 5 + 100)]
    o2, _ = P.retention_recurrence(q[2:], k[2:], v[2:], torch.tensor([0.5], dtype=torch.float64), state=torch.full((1, 2, 1), 10.5, dtype=torch.float64))
    assert float(o2[0, 0, 0]) == pytest.approx(float(o[2, 0, 0]))
    h = torch.eye(3, dtype=torch.float64)
    idx, wt, z = P.route(h, torch.tensor([[1.0, 0, 0], [0, 2.0, 0], [0.5, 0, 3.0]], dtype=torch.float64), torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64), 2)
    assert idx.tolist() == [[2, 0], [1, 2], [2, 0]]            # row 0: logits (1, 0, 1.5): the bias takes part in the choice
    assert float(wt[0, 0]) == pytest.approx(math.exp(1.5) / (math.exp(1.5) + math.exp(1.0)))
    assert torch.allclose(wt.sum(-1), torch.ones(3, dtype=torch.float64))


def test_decoding_equals_the_prompt_in_the_plain_implementation():
    """The whole sequence and its prefix give the same logits on the prefix (causality), for every configuration."""
    for name, cfg in CONFIGS.items():
        t = tensors_of(name)
        toks = [(7 * i + 3) % cfg["vocab"] for i in range(21)]
        whole, part = P.forward(cfg, t, toks), P.forward(cfg, t, toks[:9])
        assert torch.allclose(whole[:9], part, atol=1e-9), name


def test_config_reader_spec_and_declared_tensors():
    from pico_vllm_amd.config.dikolix import DikolixConfig, dikolix_run_order, dikolix_spec
    from pico_vllm_amd.config.model_config import ConfigError
    from pico_vllm_amd.parts.model import model_param_specs
    for name, raw in CONFIGS.items():
        cfg = DikolixConfig.from_dict(raw)
        assert dikolix_run_order(cfg) == P.run_order(raw)
        spec = dikolix_spec(cfg)
        want = {p.name: tuple(p.shape) for p in model_param_specs(spec)}
        assert want == P.tensor_shapes(raw), name
        assert [(e.layer, e.add_input) for e in spec.run_order] == P.run_order(raw)
    a = DikolixConfig.from_dict(CONFIGS["a"])
    assert a.residual_mult == 0.6 and a.bigram == (53, 7, 3) and a.loop == (1, 3, 3) and a.layers[1].mlp is None
    c = DikolixConfig.from_dict(CONFIGS["c"])
    assert c.residual_mult == 1.0 and c.bigram is None and c.loop is None and c.layers[2].mixer.rot is None
    bad = dict(CONFIGS["a"], layers=[dict(CONFIGS["a"]["layers"][2], mixer=dict(CONFIGS["a"]["layers"][2]["mixer"], decay=[0.9]))])
    with pytest.raises(ConfigError):
        DikolixConfig.from_dict(bad)
    with pytest.raises(ConfigError):
        DikolixConfig.from_dict(dict(CONFIGS["a"], loop={"start": 2, "stop": 9, "times": 2}))
    with pytest.raises(ConfigError):
        DikolixConfig.from_dict(dict(CONFIGS["a"], layers=[{"type": "other", "mixer": {}, "mlp": None}]))


def test_state_of_parts_around_the_layers_joins_the_cache_manager():
    """The pair embedding keeps a token per request: the model lists it among the states (so a request's slot is
    cleared for it too) and a loop gives every pass a cache of its own."""
    import torch as _t
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.config.dikolix import DikolixConfig, dikolix_spec
    from pico_vllm_amd.parts.model import DecoderModel
    spec = dikolix_spec(DikolixConfig.from_dict(CONFIGS["b"]))
    model = DecoderModel(spec, _t.float32, _t.device("cpu"))
    specs = model.cache_specs()
    assert sorted(specs) == [-1, 0, 1, 2, 3, 4, 5] and specs[-1].kind == "state" and specs[-1].state_dtype == "int32"
    assert specs[1].kind == "paged_kv" and specs[3] == specs[1] and specs[2] == specs[4] and specs[2].kind == "state"
    m = CacheManager(specs, 8, 10, 2)
    assert len(m.groups) == 2 and m.add_request("x") and m.take_fresh_slots() == [m.slot("x")]


def test_a_checkpoint_may_hold_the_unused_second_norm_of_a_layer_without_feed_forward():
    from dikolix_configs import write_model
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.parts.model import model_param_specs
    from pico_vllm_amd.weights.loader import load_checkpoint
    t = dict(tensors_of("a"))
    width = CONFIGS["a"]["width"]
    t["l1.norm2"], t["l1.norm2.b"], t["l1.ls2"] = (torch.ones(width).bfloat16() for _ in range(3))
    d = write_model(CONFIGS["a"], t, "dikolix_extra_")
    _, _, spec = load_model_description(d)
    out = load_checkpoint(d, model_param_specs(spec), torch.float32, optional=spec.ignored_tensors)
    assert "l1.norm2" not in out and "l1.norm1" in out
