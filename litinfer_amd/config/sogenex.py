"""Typed configuration of the Sogenex decoder, read from config.json, and the model as data.

config.json: `vocab`, `width`, `norm.eps`, `logit_scale`, `logit_softcap`, and `layers`, a list whose entries have
`type` (the mixer: `mamba2` or `attention`), the mixer's sizes and constants under `mixer`, `mlp` (null, or
{kind: "moe", expert: {ff}, router: {experts, top}, shared: {ff} or null}) and optionally `weights_of`: j, which
says that the layer has no tensors of its own and runs with layer j's (mixer, feed-forward and norms), with a
cache or state of its own.

The model: token embedding plus a sinusoidal position vector; per layer x += mixer(norm1(x)) and, if the layer
has one, x += feed_forward(norm2(x)), with RMS norms whose weights are stored around zero (1 + w); a final norm
of the same kind, a linear head, the logits scaled and then capped by a tanh.
Tensor names: embed, head, final.norm and per layer i with tensors of its own `l<i>.norm1|norm2`, `l<i>.mix.*`,
`l<i>.mlp.*`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .qwen2 import ConfigError
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec
from .tovasun import DEFAULT_MAX_POSITIONS, _number, _pos_int

MIXER_TYPES = ("mamba2", "attention")
SINUSOID_BASE = 10000.0                  # the design fixes the base of its position vector


@dataclass(frozen=True)
class SsmConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class DiffAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: int                          # 0: every earlier position is visible


@dataclass(frozen=True)
class MoeConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int                       # 0: no shared expert


@dataclass(frozen=True)
class SogenexLayer:
    type: str
    mixer: Any                           # SsmConfig | DiffAttentionConfig
    mlp: Optional[MoeConfig]
    weights_of: Optional[int]            # the layer whose tensors this one runs with


def _mixer(kind: str, d: Any, where: str):
    if kind not in MIXER_TYPES:
        raise ConfigError(f"config.json: {where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
    if not isinstance(d, dict):
        raise ConfigError(f"config.json: {where}.mixer must be an object")
    if kind == "mamba2":
        m = SsmConfig(heads=_pos_int(d, "heads", where), vdim=_pos_int(d, "vdim", where), state=_pos_int(d, "state", where),
                      groups=_pos_int(d, "groups", where) if d.get("groups") is not None else 1,
                      conv=_pos_int(d, "conv", where), norm_groups=_pos_int(d, "norm_groups", where) if d.get("norm_groups") is not None else 1)
        if m.heads % m.groups:
            raise ConfigError(f"config.json: {where}: {m.heads} heads are not a multiple of {m.groups} groups")
        if (m.heads * m.vdim) % m.norm_groups:
            raise ConfigError(f"config.json: {where}: {m.heads * m.vdim} columns do not split into {m.norm_groups} norm groups")
        return m
    heads = _pos_int(d, "heads", where)
    kvh = _pos_int(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
    if heads % kvh:
        raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kvh} kv heads")
    dim = _pos_int(d, "dim", where)
    mask = d.get("mask") or {}
    return DiffAttentionConfig(heads=heads, kv_heads=kvh, dim=dim, vdim=_pos_int(d, "vdim", where) if d.get("vdim") is not None else dim,
                               scale=_number(d, "scale", where), diff=_number(d, "diff", where),
                               window=_pos_int(mask, "size", where + ".mask") if mask.get("size") is not None else 0)


def _mlp(d: Any, where: str) -> Optional[MoeConfig]:
    if d is None:
        return None
    if not isinstance(d, dict) or d.get("kind") != "moe":
        raise ConfigError(f"config.json: {where}.mlp.kind {d.get('kind') if isinstance(d, dict) else d!r} is not supported (only 'moe')")
    router, expert, shared = d.get("router") or {}, d.get("expert") or {}, d.get("shared")
    m = MoeConfig(experts=_pos_int(router, "experts", where + ".mlp.router"), top=_pos_int(router, "top", where + ".mlp.router"),
                  ff=_pos_int(expert, "ff", where + ".mlp.expert"),
                  shared_ff=_pos_int(shared, "ff", where + ".mlp.shared") if shared else 0)
    if m.top > m.experts:
        raise ConfigError(f"config.json: {where}.mlp.router: top ({m.top}) exceeds the number of experts ({m.experts})")
    return m


@dataclass(frozen=True)
class SogenexConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    logit_softcap: float
    layers: Tuple[SogenexLayer, ...]
    max_positions: int
    eos_token_ids: Tuple[int, ...]
    raw: Any = None

    architecture = "Sogenex"

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "SogenexConfig":
        vocab, width = _pos_int(cfg, "vocab", "config"), _pos_int(cfg, "width", "config")
        eps = _number(cfg.get("norm") or {}, "eps", "norm")
        if eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        raw_layers = cfg.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, L in enumerate(raw_layers):
            where = f"layers[{i}]"
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            src = L.get("weights_of")
            if src is not None and (isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < len(raw_layers) or src == i):
                raise ConfigError(f"config.json: {where}.weights_of must name another layer, found {src!r}")
            layers.append(SogenexLayer(L.get("type"), _mixer(L.get("type"), L.get("mixer"), where), _mlp(L.get("mlp"), where), src))
        for i, L in enumerate(layers):
            if L.weights_of is not None:
                owner = layers[L.weights_of]
                if owner.weights_of is not None:
                    raise ConfigError(f"config.json: layers[{i}].weights_of names layer {L.weights_of}, which has no tensors of its own")
                if (owner.type, owner.mixer, owner.mlp) != (L.type, L.mixer, L.mlp):
                    raise ConfigError(f"config.json: layers[{i}] runs with the tensors of layer {L.weights_of} but differs from it")
        scale = _number(cfg, "logit_scale", "config") if cfg.get("logit_scale") is not None else 1.0
        cap = _number(cfg, "logit_softcap", "config") if cfg.get("logit_softcap") is not None else 0.0
        if cap < 0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos]))
        maxpos = DEFAULT_MAX_POSITIONS if cfg.get("max_positions") is None else _pos_int(cfg, "max_positions", "config")
        return cls(vocab=vocab, width=width, eps=eps, logit_scale=scale, logit_softcap=cap, layers=tuple(layers),
                   max_positions=maxpos, eos_token_ids=tuple(e for e in eos_ids if e >= 0), raw=cfg)


def _mixer_spec(c: SogenexConfig, L: SogenexLayer, prefix: str) -> PartSpec:
    m = L.mixer
    if L.type == "mamba2":
        return PartSpec("mamba2", prefix, {"hidden_size": c.width, "num_heads": m.heads, "value_dim": m.vdim, "state_size": m.state,
                                           "groups": m.groups, "conv": m.conv, "norm_groups": m.norm_groups, "eps": c.eps})
    return PartSpec("diff_attention", prefix, {"hidden_size": c.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                                               "head_dim": m.dim, "value_dim": m.vdim, "scale": m.scale, "diff": m.diff,
                                               "window": m.window, "eps": c.eps})


def sogenex_model_spec(c: SogenexConfig) -> ModelSpec:
    layers, index = [], {}                       # config layer -> its place among the layers that own tensors
    for i, L in enumerate(c.layers):
        if L.weights_of is not None:
            continue
        p = f"l{i}."

        def norm(name):
            return PartSpec("rmsnorm", p, {"size": c.width, "eps": c.eps, "param": name, "offset": 1.0})
        parts: Dict[str, Optional[PartSpec]] = {"norm1": norm("norm1"), "mixer": _mixer_spec(c, L, p + "mix.")}
        if L.mlp is not None:
            parts["norm2"] = norm("norm2")
            parts["feed_forward"] = PartSpec("routed_relu2", p + "mlp.", {
                "hidden_size": c.width, "experts": L.mlp.experts, "top": L.mlp.top, "intermediate_size": L.mlp.ff,
                "shared_intermediate_size": L.mlp.shared_ff})
        index[i] = len(layers)
        layers.append(LayerSpec(block="prenorm", parts=parts))
    order = tuple(ExecEntry(index[i if L.weights_of is None else L.weights_of]) for i, L in enumerate(c.layers))
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.width, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "embed",
                                                   "sinusoid_base": SINUSOID_BASE}),
        layers=tuple(layers), order=order,
        final_norm=PartSpec("rmsnorm", "final.", {"size": c.width, "eps": c.eps, "param": "norm", "offset": 1.0}),
        head=PartSpec("linear_head", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "head",
                                          "logit_scale": c.logit_scale, "softcap": c.logit_softcap}),
        eos_token_ids=c.eos_token_ids)
