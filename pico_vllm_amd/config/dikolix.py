"""The Dikolix decoder as a typed configuration and a model description.

config.json gives every size and every constant that differs between models of the design:

  architecture "Dikolix", vocab, width, norm.eps, residual_mult, embedding.bigram.{buckets, mul_prev, mul_cur} (or none),
  loop.{start, stop, times} (or none),
  layers: a list; each entry has type (its mixer), mixer (the mixer's sizes) and mlp (its feed-forward, or null)
    type "latent_attention": heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot.base, rot.scaling.{factor, original, fast, slow}
    type "mamba1":           inner, state, conv, dt_rank
    type "retention":        heads, dim, vdim, decay (one a head), rot.dims / rot.base (or no rot)
    mlp kind "moe": expert.ff, router.experts / top, shared.ff (or no shared)

The model: token row plus the row of a hashed (previous token, token) pair; layers of the pre-norm arrangement with a
constant and a stored vector on every sublayer's output, layer norms with bias; layers loop.start .. loop.stop - 1
run loop.times times in a row with the same weights and a cache or state of their own each time, the embeddings joining
the stream again in front of every pass but the first; a final layer norm; the embedding matrix as output matrix.
Tensor names: embed, bigram, l<i>.norm1(.b), l<i>.norm2(.b), l<i>.ls1, l<i>.ls2, l<i>.mix.*, l<i>.mlp.*, final.norm(.b).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .lerazen import _int, _num
from .model_config import ConfigError
from .nasedra import RotationConfig
from .registry import register_architecture


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    base: float
    scaling: Optional[Tuple[float, float, float, float]]

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LatentAttentionConfig":
        rot_dim = _int(d, "rot_dim", where, least=0)
        base, scaling = 10000.0, None
        if rot_dim:
            if not isinstance(d.get("rot"), dict):
                raise ConfigError(f"{where}: a rotated part needs 'rot'")
            # the rotated vector is the rot_dim part, whatever rot.dims says
            r = RotationConfig.from_dict(dict(d["rot"], dims=rot_dim), where + ".rot", rot_dim)
            base, scaling = r.base, r.scaling
        return cls(heads=_int(d, "heads", where), dim=_int(d, "dim", where), rot_dim=rot_dim, vdim=_int(d, "vdim", where),
                   q_rank=_int(d, "q_rank", where), kv_rank=_int(d, "kv_rank", where), scale=_num(d, "scale", where),
                   base=base, scaling=scaling)


@dataclass(frozen=True)
class StateSpaceConfig:
    inner: int
    state: int
    conv: int
    dt_rank: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "StateSpaceConfig":
        return cls(inner=_int(d, "inner", where), state=_int(d, "state", where), conv=_int(d, "conv", where),
                   dt_rank=_int(d, "dt_rank", where))


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[RotationConfig]

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RetentionConfig":
        heads, dim = _int(d, "heads", where), _int(d, "dim", where)
        decay = d.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(g, (int, float)) and not isinstance(g, bool)
                                                                        and 0 < g <= 1 for g in decay):
            raise ConfigError(f"{where}: 'decay' lists one number in (0, 1] for each of the {heads} heads")
        return cls(heads=heads, dim=dim, vdim=_int(d, "vdim", where), decay=tuple(float(g) for g in decay),
                   rot=RotationConfig.from_dict(d["rot"], where + ".rot", dim) if d.get("rot") else None)


@dataclass(frozen=True)
class ExpertsConfig:
    ff: int
    experts: int
    top: int
    shared_ff: int = 0          # 0: no shared expert

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "ExpertsConfig":
        if d.get("kind") != "moe":
            raise ConfigError(f"{where}: mlp kind {d.get('kind')!r} is not known (moe)")
        ex, ro, sh = d.get("expert") or {}, d.get("router") or {}, d.get("shared") or {}
        cfg = cls(_int(ex, "ff", where + ".expert"), _int(ro, "experts", where + ".router"), _int(ro, "top", where + ".router"),
                  _int(sh, "ff", where + ".shared") if sh else 0)
        if cfg.top > cfg.experts:
            raise ConfigError(f"{where}: top {cfg.top} of {cfg.experts} experts")
        return cfg


@dataclass(frozen=True)
class DikolixLayer:
    type: str
    mixer: Any
    mlp: Optional[ExpertsConfig]


_MIXERS = {"latent_attention": LatentAttentionConfig, "mamba1": StateSpaceConfig, "retention": RetentionConfig}


@dataclass(frozen=True)
class DikolixConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    bigram: Optional[Tuple[int, int, int]]       # buckets, mul_prev, mul_cur
    loop: Optional[Tuple[int, int, int]]         # start, stop, times
    layers: Tuple[DikolixLayer, ...]
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "DikolixConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, l in enumerate(raw_layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or not isinstance(l.get("mixer"), dict):
                raise ConfigError(f"{where} lacks 'mixer'")
            if l.get("type") not in _MIXERS:
                raise ConfigError(f"{where}: mixer type {l.get('type')!r} is not known ({', '.join(sorted(_MIXERS))})")
            mlp = l.get("mlp")
            layers.append(DikolixLayer(l["type"], _MIXERS[l["type"]].from_dict(l["mixer"], where + ".mixer"),
                                       ExpertsConfig.from_dict(mlp, where + ".mlp") if mlp else None))
        eps = _num(d.get("norm") or {}, "eps", "norm")
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        big = (d.get("embedding") or {}).get("bigram")
        bigram = None
        if big:
            bigram = (_int(big, "buckets", "embedding.bigram"), _int(big, "mul_prev", "embedding.bigram", least=0),
                      _int(big, "mul_cur", "embedding.bigram", least=0))
        lp = d.get("loop")
        loop = None
        if lp:
            loop = (_int(lp, "start", "loop", least=0), _int(lp, "stop", "loop", least=0), _int(lp, "times", "loop"))
            if not loop[0] <= loop[1] <= len(layers):
                raise ConfigError(f"loop: layers {loop[0]} .. {loop[1]} - 1 of {len(layers)}")
        eos = d.get("eos_token_id")
        return cls(vocab=_int(d, "vocab", "config.json"), width=_int(d, "width", "config.json"), norm_eps=eps,
                   residual_mult=_num(d, "residual_mult", "config.json") if d.get("residual_mult") is not None else 1.0,
                   bigram=bigram, loop=loop, layers=tuple(layers),
                   eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)


def dikolix_run_order(cfg: DikolixConfig):
    """The layers in the order they run: (layer, whether the embeddings join the stream again in front of it)."""
    n = len(cfg.layers)
    if not cfg.loop or cfg.loop[2] <= 1 or cfg.loop[0] >= cfg.loop[1]:
        return [(i, False) for i in range(n)]
    start, stop, times = cfg.loop
    out = [(i, False) for i in range(start)]
    for p in range(times):
        out += [(i, p > 0 and i == start) for i in range(start, stop)]
    return out + [(i, False) for i in range(stop, n)]


def dikolix_spec(cfg: DikolixConfig) -> ModelSpec:
    norm = PartSpec("layer_norm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_name": "", "bias_name": "b"})
    layers, unused = [], []
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        if l.type == "latent_attention":
            mixer = PartSpec("latent_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
                "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "base": m.base, "scaling": m.scaling,
                "norm_eps": cfg.norm_eps})
        elif l.type == "mamba1":
            mixer = PartSpec("selective_state_space", {
                "hidden_size": cfg.width, "inner": m.inner, "state": m.state, "taps": m.conv, "dt_rank": m.dt_rank})
        else:
            mixer = PartSpec("retention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "decay": m.decay,
                "norm_eps": cfg.norm_eps, "rotary_dim": m.rot.dims if m.rot else 0, "base": m.rot.base if m.rot else 10000.0,
                "scaling": m.rot.scaling if m.rot else None})
        if l.mlp is None:
            # a checkpoint may still hold the second norm and vector of a layer that has no feed-forward to use them
            unused += [f"l{i}.norm2", f"l{i}.norm2.b", f"l{i}.ls2"]
            layers.append(LayerSpec(prefix=f"l{i}", block="prenorm_scaled_mixer_only",
                                    slots={"norm1": ("norm1", norm), "mixer": ("mix", mixer)},
                                    block_params={"size": cfg.width, "mult": cfg.residual_mult}))
            continue
        else:
            ff = PartSpec("top_softmax_routed_experts", {
                "hidden_size": cfg.width, "expert_size": l.mlp.ff, "num_experts": l.mlp.experts, "top": l.mlp.top,
                "shared_size": l.mlp.shared_ff})
        layers.append(LayerSpec(prefix=f"l{i}", block="prenorm_scaled",
                                slots={"norm1": ("norm1", norm), "mixer": ("mix", mixer), "norm2": ("norm2", norm), "ff": ("mlp", ff)},
                                block_params={"size": cfg.width, "mult": cfg.residual_mult}))
    before = ()
    if cfg.bigram:
        before = (("bigram", PartSpec("pair_embedding", {"size": cfg.width, "buckets": cfg.bigram[0], "mul_prev": cfg.bigram[1],
                                                          "mul_cur": cfg.bigram[2], "name": ""})),)
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embed_name="embed", layers=layers,
        run_order=[RunEntry(i, add_input=again) for i, again in dikolix_run_order(cfg)],
        final_norm=norm, final_norm_name="final.norm", head_name=None, eos_token_id=cfg.eos_token_id,
        before_layers=before, ignored_tensors=tuple(unused))


def dikolix_sizes(cfg: DikolixConfig) -> dict:
    """The sizes of a configuration as a flat record (of its first layer of every kind)."""
    out = {"layers": len(cfg.layers), "runs": len(dikolix_run_order(cfg)), "hidden": cfg.width, "vocab": cfg.vocab, "tied": True}
    for l in cfg.layers:
        m = l.mixer
        if l.type == "latent_attention":
            out.setdefault("q_heads", m.heads)
            out.setdefault("kv_heads", 1)
            out.setdefault("head_dim", m.dim + m.rot_dim)
            out.setdefault("value_dim", m.vdim)
            out.setdefault("kv_rank", m.kv_rank)
        elif l.type == "mamba1":
            out.setdefault("ssm_inner", m.inner)
            out.setdefault("ssm_state", m.state)
        else:
            out.setdefault("retention_heads", m.heads)
            out.setdefault("retention_key_dim", m.dim)
            out.setdefault("retention_value_dim", m.vdim)
        if l.mlp is not None:
            out.setdefault("experts", l.mlp.experts)
            out.setdefault("top", l.mlp.top)
            out.setdefault("expert_size", l.mlp.ff)
    return out


def dikolix_with_layers(raw: dict, layers: int) -> dict:
    """The same kinds of layers, ``layers`` of them (the list cut, or repeated from its start), without a loop."""
    have = raw["layers"]
    out = dict(raw, layers=[have[i % len(have)] for i in range(layers)] if have else [])
    out.pop("loop", None)
    return out


register_architecture("Dikolix", DikolixConfig.from_dict, dikolix_spec, dikolix_sizes, dikolix_with_layers)
