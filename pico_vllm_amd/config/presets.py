"""Named configurations for random-weight runs: the sizes of the published Qwen2.5 models and two
tiny ones for quick checks.  Each is what the model's config.json would hold (the keys that
``Qwen2Config.from_dict`` reads); nothing else in the package refers to these sizes."""
from __future__ import annotations

from typing import Dict


def _qwen2(vocab, hidden, layers, heads, kv_heads, inter, tied, eps=1e-6, theta=1e6, max_pos=131072, **more) -> Dict:
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": vocab, "hidden_size": hidden,
           "num_hidden_layers": layers, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
           "intermediate_size": inter, "rms_norm_eps": eps, "rope_theta": theta, "tie_word_embeddings": tied,
           "max_position_embeddings": max_pos, "hidden_act": "silu"}
    cfg.update(more)
    return cfg


PRESETS: Dict[str, Dict] = {
    "tiny-a": _qwen2(256, 64, 2, 4, 1, 172, True, theta=1e4, max_pos=2048, eos_token_id=255),
    "tiny-b": _qwen2(384, 192, 3, 6, 3, 320, False, eps=1e-5, max_pos=4096, eos_token_id=383),
    "1.5b": _qwen2(151936, 1536, 28, 12, 2, 8960, True),
    "7b": _qwen2(152064, 3584, 28, 28, 4, 18944, False),
    "32b": _qwen2(152064, 5120, 64, 40, 8, 27648, False),
}


def _lerazen(vocab, width, layers, heads, kv_heads, dim, dense_ff, experts, top, expert_ff, window=1024, every_global=4,
             max_positions=40960) -> Dict:
    """A Lerazen configuration of a real model's proportions: dense and routed feed-forwards in turn, windowed layers
    with every ``every_global``-th one unwindowed, values mixed with the first layer's."""
    def mixer(i):
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "v_mix": True,
             "q_temp": {"coef": 0.4, "every": 512}}
        if (i + 1) % every_global:
            m["mask"] = {"size": window}
        return m
    dense = {"kind": "dense", "ff": dense_ff}
    routed = {"kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0}, "router": {"experts": experts, "top": top}}
    return {"architecture": "Lerazen", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": 1e-6},
            "layers": [{"type": "attention", "mixer": mixer(i), "mlp": routed if i % 2 else dense} for i in range(layers)]}


# Lerazen at the sizes of the Qwen2.5 shapes above: the same width, heads and layers; a token multiplies as many
# feed-forward weights (two matrices of 1.5 x the intermediate size where it is dense; ``top`` experts of three
# matrices where it is routed).  Kept apart from PRESETS, whose keys are one architecture's.
DESIGN_PRESETS: Dict[str, Dict] = {
    "lerazen-1.5b": _lerazen(151936, 1536, 28, 12, 2, 128, 13440, 16, 2, 4480),
    "lerazen-7b": _lerazen(152064, 3584, 28, 28, 4, 128, 28416, 32, 4, 4736),
}


def _nasedra(vocab, width, layers, heads, kv_heads, dim, dense_ff, experts, top, expert_ff, shared_ff, gla_dim=64,
             window=1024, keep_first=4) -> Dict:
    """A Nasedra configuration of a real model's proportions, in groups of four layers: windowed attention with a dense
    feed-forward, a recurrent layer with a routed one, attention over the first layer's keys and values with a dense
    one, a recurrent layer with a routed one."""
    rot = {"dims": dim, "base": 1000000.0, "scaling": {"factor": 4.0, "original": 8192, "fast": 16.0, "slow": 2.0}}

    def attention(i):
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "softcap": 30.0,
             "mask": {"size": window, "keep_first": keep_first}, "rot": rot}
        if i % 4 == 2:
            m["kv_from"] = i - 2
        return m
    recurrent = {"heads": heads, "dim": gla_dim, "vdim": dim, "tau": 8.0, "rank": 32}
    dense = {"kind": "dense", "ff": dense_ff}
    routed = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "identity": 1, "scale": 2.0},
              "shared": {"ff": shared_ff}}
    return {"architecture": "Nasedra", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"scale": width ** 0.5},
            "layers": [{"type": "gla", "mixer": recurrent, "mlp": routed} if i % 2 else
                       {"type": "attention", "mixer": attention(i), "mlp": dense} for i in range(layers)]}


# Nasedra at the sizes of the Qwen2.5 shapes: the same width, heads and layers, the same dense feed-forward; where it
# is routed a token multiplies as many feed-forward weights (``top`` experts and the shared one).
DESIGN_PRESETS.update({
    "nasedra-1.5b": _nasedra(151936, 1536, 28, 12, 2, 128, 8960, 16, 2, 2240, 4480),
    "nasedra-7b": _nasedra(152064, 3584, 28, 28, 4, 128, 18944, 32, 4, 2368, 9472),
})


def _dikolix(vocab, width, layers, heads, dim, rot_dim, q_rank, kv_rank, experts, top, expert_ff, shared_ff, ret_dim=64,
             buckets=262144) -> Dict:
    """A Dikolix configuration of a real model's proportions, in groups of three layers: attention through latents, a
    selective state-space layer of twice the width, retention; every layer with routed experts and a gated shared one;
    a hashed table of token pairs on the embedding."""
    att = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": dim, "q_rank": q_rank, "kv_rank": kv_rank,
           "scale": (dim + rot_dim) ** -0.5,
           "rot": {"dims": rot_dim, "base": 1000000.0, "scaling": {"factor": 4.0, "original": 8192, "fast": 16.0, "slow": 2.0}}}
    ssm = {"inner": 2 * width, "state": 16, "conv": 4, "dt_rank": width // 16}
    ret = {"heads": heads, "dim": ret_dim, "vdim": dim, "decay": [1.0 - 2.0 ** (-5.0 - 3.0 * h / heads) for h in range(heads)],
           "rot": {"dims": ret_dim, "base": 10000.0}}
    routed = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top}, "shared": {"ff": shared_ff}}
    kinds = (("latent_attention", att), ("mamba1", ssm), ("retention", ret))
    return {"architecture": "Dikolix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": 1000003, "mul_cur": 31}},
            "layers": [{"type": kinds[i % 3][0], "mixer": kinds[i % 3][1], "mlp": routed} for i in range(layers)]}


# Dikolix at the sizes of the Qwen2.5 shapes: the same width, heads and head size; the routed feed-forward of the Nasedra
# presets in every layer; a key/value latent of 256 entries and a rotated part of 64 (the largest value size the
# matrix-core attention of this package takes is 256).
DESIGN_PRESETS.update({
    "dikolix-1.5b": _dikolix(151936, 1536, 27, 12, 128, 64, 768, 256, 16, 2, 2240, 4480),
    "dikolix-7b": _dikolix(152064, 3584, 27, 28, 128, 64, 1536, 256, 32, 4, 2368, 9472),
})


def _vagelix(vocab, width, layers, heads, kv_heads, dim, ff, chunk=1024, delta_dim=64, ssd_dim=64, ssd_state=128,
             ssd_groups=2) -> Dict:
    """A Vagelix configuration of a real model's proportions, in groups of three layers: differential attention (two
    maps of half a head's size each), a chunked attention beside a gated delta rule, a state-space duality layer of twice
    the width; every layer with the dense feed-forward."""
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim // 2, "vdim": dim, "scale": (dim // 2) ** -0.5, "diff": 0.6,
           "q_temp": {"coef": 0.1, "every": 1024}}
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "mask": {"size": chunk},
            "rot": {"dims": dim // 2, "base": 1000000.0}}
    right = {"heads": heads, "kv_heads": kv_heads, "dim": delta_dim, "vdim": dim, "conv": 4, "decay_rank": 32, "gate_rank": 32}
    ssd = {"heads": 2 * width // ssd_dim, "vdim": ssd_dim, "state": ssd_state, "groups": ssd_groups, "norm_groups": ssd_groups, "conv": 4}
    kinds = (("attention", att), ("parallel", {"left": left, "right": right}), ("mamba2", ssd))
    return {"architecture": "Vagelix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6},
            "layers": [{"type": kinds[i % 3][0], "mixer": kinds[i % 3][1], "mlp": {"kind": "dense", "ff": ff}} for i in range(layers)]}


# Vagelix at the sizes of the Qwen2.5 shapes: the same width, heads, head size and dense feed-forward.
DESIGN_PRESETS.update({
    "vagelix-1.5b": _vagelix(151936, 1536, 27, 12, 2, 128, 8960),
    "vagelix-7b": _vagelix(152064, 3584, 27, 28, 4, 128, 18944, ssd_groups=4),
})


def preset(name: str) -> Dict:
    import copy
    key = name.lower()
    if key in PRESETS:
        return dict(PRESETS[key])
    if key in DESIGN_PRESETS:
        return copy.deepcopy(DESIGN_PRESETS[key])
    raise ValueError(f"unknown configuration {name!r}; known: {', '.join(sorted(PRESETS) + sorted(DESIGN_PRESETS))}")
