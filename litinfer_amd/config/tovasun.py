"""Typed configuration of the Tovasun decoder, read from config.json, and the model as data.

config.json: `vocab`, `width`, `norm.eps`, `layers` (a list; each entry has `type`, one of the mixers
`attention` and `latent_attention`, the mixer's sizes and constants under `mixer`, and `mlp` = null or
{kind, ff}), optional `loop` {start, stop, times} (layers start..stop-1 are passed `times` times with the
same weights, every pass with a cache of its own) and optional `token_side` {dim} (a per-layer token input).

The model: embedding; per layer an RMS norm before and behind each sublayer (mixer, then the
feed-forward if the layer has one), then the token input; before pass t of the loop the stream takes the
embedding output again (t > 0) and row t of `loop.step`; a final RMS norm and a linear head.
Tensor names: embed, head, final.norm, loop.step, side.embed, and per layer i `l<i>.norm1|norm1b|norm2|norm2b`,
`l<i>.mix.*`, `l<i>.mlp.up|down`, `l<i>.side.gate|proj|norm`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .qwen2 import ConfigError
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("attention", "latent_attention")
DEFAULT_MAX_POSITIONS = 1 << 17          # the design names no longest sequence; the cache's tables need a bound


def _pos_int(d: Dict[str, Any], key: str, where: str, allow_zero: bool = False) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < 0 or (v == 0 and not allow_zero):
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, found {v!r}")
    return v


def _number(d: Dict[str, Any], key: str, where: str) -> float:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}.{key} must be a number, found {v!r}")
    return float(v)


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[Tuple[str, float], ...]]        # sorted (name, value) pairs of factor, original, fast, slow

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RotaryConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: {where} must be an object")
        base, dims = _number(d, "base", where), _pos_int(d, "dims", where)
        if base <= 0 or dims % 2:
            raise ConfigError(f"config.json: {where}: base must be positive and dims even")
        sc = d.get("scaling")
        if sc is not None:
            sc = tuple(sorted((k, _number(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow")))
        return cls(base, dims, sc)

    def scaling_dict(self) -> Optional[Dict[str, float]]:
        return dict(self.scaling) if self.scaling else None


@dataclass(frozen=True)
class MixerConfig:
    type: str
    heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig
    window: int = 0
    keep_first: int = 0
    softcap: float = 0.0
    kv_heads: int = 0            # attention
    rot_dim: int = 0             # latent attention
    kv_rank: int = 0

    @classmethod
    def from_dict(cls, kind: str, d: Dict[str, Any], where: str) -> "MixerConfig":
        if kind not in MIXER_TYPES:
            raise ConfigError(f"config.json: {where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: {where}.mixer must be an object")
        heads, dim = _pos_int(d, "heads", where), _pos_int(d, "dim", where)
        vdim = _pos_int(d, "vdim", where) if d.get("vdim") is not None else dim
        rot = RotaryConfig.from_dict(d.get("rot"), where + ".rot")
        mask = d.get("mask") or {}
        window = _pos_int(mask, "size", where + ".mask") if mask.get("size") is not None else 0
        keep = _pos_int(mask, "keep_first", where + ".mask", allow_zero=True) if mask.get("keep_first") is not None else 0
        softcap = _number(d, "softcap", where) if d.get("softcap") is not None else 0.0
        if softcap < 0:
            raise ConfigError(f"config.json: {where}.softcap must not be negative")
        kw: Dict[str, Any] = {}
        if kind == "attention":
            kvh = _pos_int(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
            if heads % kvh:
                raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kvh} kv heads")
            if rot.dims > dim:
                raise ConfigError(f"config.json: {where}: rot.dims ({rot.dims}) exceeds the head size ({dim})")
            kw = {"kv_heads": kvh}
        else:
            rot_dim, rank = _pos_int(d, "rot_dim", where), _pos_int(d, "kv_rank", where)
            if rot.dims != rot_dim:
                raise ConfigError(f"config.json: {where}: rot.dims ({rot.dims}) must equal rot_dim ({rot_dim})")
            kw = {"rot_dim": rot_dim, "kv_rank": rank}
        return cls(type=kind, heads=heads, dim=dim, vdim=vdim, scale=_number(d, "scale", where), rot=rot,
                   window=window, keep_first=keep, softcap=softcap, **kw)


@dataclass(frozen=True)
class TovasunLayer:
    mixer: MixerConfig
    ff: int                      # 0: the layer has no feed-forward


@dataclass(frozen=True)
class TovasunConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[TovasunLayer, ...]
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    side_dim: int                               # 0: no per-layer token input
    max_positions: int
    eos_token_ids: Tuple[int, ...]
    raw: Any = None

    architecture = "Tovasun"

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "TovasunConfig":
        vocab, width = _pos_int(cfg, "vocab", "config"), _pos_int(cfg, "width", "config")
        norm = cfg.get("norm") or {}
        eps = _number(norm, "eps", "norm")
        if eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        raw_layers = cfg.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, L in enumerate(raw_layers):
            where = f"layers[{i}]"
            mixer = MixerConfig.from_dict(L.get("type"), L.get("mixer"), where)
            mlp = L.get("mlp")
            ff = 0
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind {mlp.get('kind')!r} is not supported (only 'dense')")
                ff = _pos_int(mlp, "ff", where + ".mlp")
            layers.append(TovasunLayer(mixer, ff))
        loop = cfg.get("loop")
        if loop is not None:
            start = _pos_int(loop, "start", "loop", allow_zero=True)
            stop, times = _pos_int(loop, "stop", "loop", allow_zero=True), _pos_int(loop, "times", "loop")
            if not 0 <= start <= stop <= len(layers):
                raise ConfigError(f"config.json: loop {start}..{stop} lies outside the {len(layers)} layers")
            loop = (start, stop, times) if stop > start else None
        side = cfg.get("token_side")
        side_dim = _pos_int(side, "dim", "token_side") if side else 0
        eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos]))
        maxpos = cfg.get("max_positions")
        maxpos = DEFAULT_MAX_POSITIONS if maxpos is None else _pos_int(cfg, "max_positions", "config")
        return cls(vocab=vocab, width=width, eps=eps, layers=tuple(layers), loop=loop, side_dim=side_dim,
                   max_positions=maxpos, eos_token_ids=tuple(e for e in eos_ids if e >= 0), raw=cfg)


def _mixer_spec(c: TovasunConfig, m: MixerConfig, prefix: str) -> PartSpec:
    rot_head = m.dim if m.type == "attention" else m.rot_dim
    position = PartSpec("rope_pairs", "", {"head_dim": rot_head, "rotary_dim": m.rot.dims, "theta": m.rot.base,
                                           "scaling": m.rot.scaling_dict()})
    common = {"hidden_size": c.width, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
              "window": m.window, "keep_first": m.keep_first, "softcap": m.softcap, "scale": m.scale,
              "eps": c.eps, "position": position}
    if m.type == "attention":
        return PartSpec("masked_attention", prefix, {**common, "num_kv_heads": m.kv_heads, "qk_norm": True})
    return PartSpec("latent_attention", prefix, {**common, "rot_dim": m.rot_dim, "kv_rank": m.kv_rank})


def tovasun_model_spec(c: TovasunConfig) -> ModelSpec:
    n = len(c.layers)
    layers = []
    for i, L in enumerate(c.layers):
        p = f"l{i}."

        def norm(name):
            return PartSpec("rmsnorm", p, {"size": c.width, "eps": c.eps, "param": name})
        parts: Dict[str, Optional[PartSpec]] = {"norm1": norm("norm1"), "mixer": _mixer_spec(c, L.mixer, p + "mix."),
                                                "norm1b": norm("norm1b")}
        if L.ff:
            parts.update({"norm2": norm("norm2"), "norm2b": norm("norm2b"),
                          "feed_forward": PartSpec("relu2_mlp", p + "mlp.", {"hidden_size": c.width,
                                                                             "intermediate_size": L.ff})})
        if c.side_dim:
            parts["token_input"] = PartSpec("gated_table_slice", p + "side.", {
                "hidden_size": c.width, "dim": c.side_dim, "offset": i * c.side_dim, "table": "side.embed",
                "vocab_size": c.vocab, "table_width": n * c.side_dim, "eps": c.eps})
        layers.append(LayerSpec(block="sandwich", parts=parts))
    order, injections = [], ()
    if c.loop:
        start, stop, times = c.loop
        injections = (PartSpec("loop_entry", "loop.", {"times": times, "hidden_size": c.width, "param": "step"}),)
        order += [ExecEntry(i) for i in range(start)]
        for t in range(times):
            order += [ExecEntry(i, inject=(0, t) if i == start else None) for i in range(start, stop)]
        order += [ExecEntry(i) for i in range(stop, n)]
    else:
        order = [ExecEntry(i) for i in range(n)]
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.width, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "embed"}),
        layers=tuple(layers), order=tuple(order),
        final_norm=PartSpec("rmsnorm", "final.", {"size": c.width, "eps": c.eps, "param": "norm"}),
        head=PartSpec("linear_head", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "head"}),
        eos_token_ids=c.eos_token_ids, injections=injections)
