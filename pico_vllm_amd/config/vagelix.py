"""The Vagelix decoder as a typed configuration and a model description.

config.json gives every size and every constant that differs between models of the design:

  architecture "Vagelix", vocab, width, norm.eps,
  layers: a list; each entry has type (its mixer), mixer (the mixer's sizes), mlp (its feed-forward, or null) and
  optionally weights_of (the layer whose tensors it runs, with a cache or state of its own)
    type "attention": heads, kv_heads, dim, vdim, scale, diff, q_temp.coef / q_temp.every (or no q_temp)
    type "parallel":  left:  heads, kv_heads, dim, vdim (= dim: the values are the keys), scale, mask.size (or no mask),
                             rot.dims / rot.base (or no rot)
                      right: heads, kv_heads, dim, vdim, conv
    type "mamba2":    heads, vdim, state, groups, norm_groups, conv
    mlp kind "dense": ff

The inner sizes of the recurrent side's two low-rank projections stand in no configuration: they are the shapes of
l<i>.mix.right.a1 and l<i>.mix.right.g1 in the checkpoint.

The model: token rows RMS-normed (embed.norm); layers that norm what a sublayer RETURNS and whose sublayers read the
stream itself, x += norm1(mixer(x)); x += norm2(ff(x)); a final RMS norm; the embedding matrix as output matrix.
Tensor names: embed, embed.norm, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.{gate,up,down}, final.norm.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .lerazen import _int, _num
from .model_config import ConfigError
from .registry import register_architecture

DEFAULT_RANK = 16          # of the low-rank projections, for a model that is yet to be written and names none


@dataclass(frozen=True)
class DiffAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    temp_coef: float
    temp_every: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "DiffAttentionConfig":
        qt = d.get("q_temp") or {}
        cfg = cls(heads=_int(d, "heads", where), kv_heads=_int(d, "kv_heads", where), dim=_int(d, "dim", where),
                  vdim=_int(d, "vdim", where), scale=_num(d, "scale", where), diff=_num(d, "diff", where),
                  temp_coef=_num(qt, "coef", where + ".q_temp") if qt else 0.0,
                  temp_every=_int(qt, "every", where + ".q_temp") if qt else 0)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv heads")
        return cfg


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    chunk: int          # 0: every earlier position is seen
    rot_dims: int       # 0: no rotation
    rot_base: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "ChunkedAttentionConfig":
        mask, rot = d.get("mask") or {}, d.get("rot") or {}
        cfg = cls(heads=_int(d, "heads", where), kv_heads=_int(d, "kv_heads", where), dim=_int(d, "dim", where),
                  scale=_num(d, "scale", where), chunk=_int(mask, "size", where + ".mask") if mask else 0,
                  rot_dims=_int(rot, "dims", where + ".rot", least=0) if rot else 0,
                  rot_base=_num(rot, "base", where + ".rot") if rot else 10000.0)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv heads")
        if d.get("vdim") is not None and _int(d, "vdim", where) != cfg.dim:
            raise ConfigError(f"{where}: the values are the keys as projected, so vdim must equal dim ({cfg.dim})")
        if cfg.rot_dims % 2 or cfg.rot_dims > cfg.dim or (cfg.rot_dims and not cfg.rot_base > 0):
            raise ConfigError(f"{where}.rot: an even number of at most {cfg.dim} turned entries and a positive base")
        return cfg


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, decay_rank: int, gate_rank: int) -> "DeltaRuleConfig":
        cfg = cls(heads=_int(d, "heads", where), kv_heads=_int(d, "kv_heads", where), dim=_int(d, "dim", where),
                  vdim=_int(d, "vdim", where), conv=_int(d, "conv", where), decay_rank=decay_rank, gate_rank=gate_rank)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} query/key heads")
        return cfg


@dataclass(frozen=True)
class PairConfig:
    left: ChunkedAttentionConfig
    right: DeltaRuleConfig


@dataclass(frozen=True)
class DualityConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "DualityConfig":
        cfg = cls(heads=_int(d, "heads", where), vdim=_int(d, "vdim", where), state=_int(d, "state", where),
                  groups=_int(d, "groups", where), norm_groups=_int(d, "norm_groups", where), conv=_int(d, "conv", where))
        if cfg.heads % cfg.groups or (cfg.heads * cfg.vdim) % cfg.norm_groups:
            raise ConfigError(f"{where}: {cfg.heads} heads in {cfg.groups} groups, {cfg.heads * cfg.vdim} entries in "
                              f"{cfg.norm_groups} normed parts: neither divides")
        return cfg


@dataclass(frozen=True)
class VagelixLayer:
    type: str
    mixer: Any
    ff: int                          # 0: no feed-forward
    weights_of: Optional[int]        # the layer whose tensors this one runs (already followed to a layer that owns some)


@dataclass(frozen=True)
class VagelixConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[VagelixLayer, ...]
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], shapes: Optional[Dict[str, tuple]] = None) -> "VagelixConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list):
            raise ConfigError("config.json lacks the list 'layers'")

        def owner(i: int) -> int:
            seen = set()
            while isinstance(raw_layers[i], dict) and raw_layers[i].get("weights_of") is not None:
                j = raw_layers[i]["weights_of"]
                if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(raw_layers) or j in seen or j == i:
                    raise ConfigError(f"layers[{i}]: weights_of must name another layer, got {j!r}")
                seen.add(i)
                i = j
            return i

        def rank(layer: int, name: str, mixer: Dict[str, Any], key: str) -> int:
            full = f"l{layer}.mix.right.{name}"
            if shapes is not None and full in shapes and len(shapes[full]) == 2:
                return int(shapes[full][0])
            if mixer.get(key) is not None:
                return _int(mixer, key, f"layers[{layer}].mixer.right")
            return DEFAULT_RANK

        layers: List[VagelixLayer] = []
        for i, l in enumerate(raw_layers):
            where = f"layers[{i}]"
            if not isinstance(l, dict) or not isinstance(l.get("mixer"), dict):
                raise ConfigError(f"{where} lacks 'mixer'")
            own = owner(i)
            kind, m = l.get("type"), l["mixer"]
            if kind == "attention":
                mixer = DiffAttentionConfig.from_dict(m, where + ".mixer")
            elif kind == "parallel":
                if not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
                    raise ConfigError(f"{where}.mixer lacks 'left' or 'right'")
                mixer = PairConfig(ChunkedAttentionConfig.from_dict(m["left"], where + ".mixer.left"),
                                   DeltaRuleConfig.from_dict(m["right"], where + ".mixer.right",
                                                             rank(own, "a1", m["right"], "decay_rank"), rank(own, "g1", m["right"], "gate_rank")))
            elif kind == "mamba2":
                mixer = DualityConfig.from_dict(m, where + ".mixer")
            else:
                raise ConfigError(f"{where}: mixer type {kind!r} is not known (attention, parallel, mamba2)")
            mlp = l.get("mlp")
            ff = 0
            if mlp:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp: kind {mlp.get('kind')!r} is not known (dense)")
                ff = _int(mlp, "ff", where + ".mlp")
            layers.append(VagelixLayer(kind, mixer, ff, own if own != i else None))
        for i, l in enumerate(layers):
            if l.weights_of is not None:
                o = layers[l.weights_of]
                if (o.type, o.mixer, o.ff) != (l.type, l.mixer, l.ff):
                    raise ConfigError(f"layers[{i}]: it runs layer {l.weights_of}'s tensors, so its sizes must be that layer's")
        eps = _num(d.get("norm") or {}, "eps", "norm")
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        eos = d.get("eos_token_id")
        return cls(vocab=_int(d, "vocab", "config.json"), width=_int(d, "width", "config.json"), norm_eps=eps,
                   layers=tuple(layers), eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)


def _mixer_spec(cfg: VagelixConfig, l: VagelixLayer) -> PartSpec:
    m, D, eps = l.mixer, cfg.width, cfg.norm_eps
    if l.type == "attention":
        return PartSpec("differential_attention", {
            "hidden_size": D, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
            "scale": m.scale, "diff": m.diff, "norm_eps": eps, "temp_coef": m.temp_coef, "temp_every": m.temp_every})
    if l.type == "mamba2":
        return PartSpec("state_space_duality", {
            "hidden_size": D, "num_heads": m.heads, "value_dim": m.vdim, "state": m.state, "groups": m.groups,
            "norm_groups": m.norm_groups, "taps": m.conv, "norm_eps": eps})
    a, r = m.left, m.right
    left = PartSpec("chunked_sink_attention", {
        "hidden_size": D, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "dim": a.dim, "scale": a.scale, "norm_eps": eps,
        "chunk": a.chunk, "rotary_dim": a.rot_dims, "base": a.rot_base})
    right = PartSpec("gated_delta_rule", {
        "hidden_size": D, "num_heads": r.heads, "num_qk_heads": r.kv_heads, "key_dim": r.dim, "value_dim": r.vdim,
        "taps": r.conv, "decay_rank": r.decay_rank, "gate_rank": r.gate_rank, "norm_eps": eps})
    return PartSpec("mixer_pair", {"hidden_size": D, "left": left, "right": right, "norm_eps": eps})


def vagelix_spec(cfg: VagelixConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_name": ""})
    layers, index, order = [], {}, []
    for i, l in enumerate(cfg.layers):
        if l.weights_of is not None:
            continue
        slots = {"norm1": ("norm1", norm), "mixer": ("mix", _mixer_spec(cfg, l))}
        block = "postnorm_mixer_only"
        if l.ff:
            slots["norm2"] = ("norm2", norm)
            slots["ff"] = ("mlp", PartSpec("swiglu_mlp", {"hidden_size": cfg.width, "intermediate_size": l.ff,
                                                           "names": ("gate", "up", "down")}))
            block = "postnorm"
        index[i] = len(layers)
        layers.append(LayerSpec(prefix=f"l{i}", block=block, slots=slots))
    for i, l in enumerate(cfg.layers):
        order.append(RunEntry(index[i if l.weights_of is None else l.weights_of]))
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embed_name="embed", layers=layers, run_order=order,
        final_norm=norm, final_norm_name="final.norm", head_name=None, eos_token_id=cfg.eos_token_id,
        before_layers=(("embed.norm", PartSpec("stream_rms_norm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_name": ""})),))


def vagelix_sizes(cfg: VagelixConfig) -> dict:
    """The sizes of a configuration as a flat record (of its first layer of every kind)."""
    out = {"layers": sum(l.weights_of is None for l in cfg.layers), "runs": len(cfg.layers), "hidden": cfg.width,
           "vocab": cfg.vocab, "tied": True}
    for l in cfg.layers:
        m = l.mixer
        if l.type == "attention":
            out.setdefault("q_heads", m.heads)
            out.setdefault("kv_heads", m.kv_heads)
            out.setdefault("head_dim", m.dim)
            out.setdefault("value_dim", m.vdim)
        elif l.type == "parallel":
            out.setdefault("chunked_heads", m.left.heads)
            out.setdefault("chunked_head_dim", m.left.dim)
            out.setdefault("chunk", m.left.chunk)
            out.setdefault("delta_heads", m.right.heads)
            out.setdefault("delta_key_dim", m.right.dim)
            out.setdefault("delta_value_dim", m.right.vdim)
        else:
            out.setdefault("ssd_heads", m.heads)
            out.setdefault("ssd_value_dim", m.vdim)
            out.setdefault("ssd_state", m.state)
        if l.ff:
            out.setdefault("intermediate", l.ff)
    return out


def vagelix_with_layers(raw: dict, layers: int) -> dict:
    """The same kinds of layers, ``layers`` of them (the list cut, or repeated from its start), each with tensors of its own."""
    have = raw["layers"]
    out = []
    for i in range(layers):
        l = dict(have[i % len(have)]) if have else {}
        seen = 0
        while l.get("weights_of") is not None and seen < len(have):
            l, seen = dict(have[l["weights_of"]]), seen + 1
        l.pop("weights_of", None)
        out.append(l)
    return dict(raw, layers=out)


register_architecture("Vagelix", VagelixConfig.from_dict, vagelix_spec, vagelix_sizes, vagelix_with_layers, reads_shapes=True)
