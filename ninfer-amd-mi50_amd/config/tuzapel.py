"""Typed configuration of Tuzapel, a decoder-only model whose layers are listed one by one.

config.json keys: `architecture` ("Tuzapel"), `vocab`, `width`, `norm.eps`, `logit_softcap`
(absent or 0: the logits are not capped), and `layers`: a list of objects with `type`
('latent_attention' or 'attention'), `mixer` (the mixer's sizes and constants) and `mlp`
(null, {'kind': 'dense', 'ff', 'limit'} or {'kind': 'moe', 'expert': {'ff', 'limit'},
'router': {'experts', 'top'}}).
A latent_attention mixer has `heads`, `dim`, `rot_dim`, `vdim`, `kv_rank`, `q_rank`, `scale`
and `rot` {`base`, `dims`}; an attention mixer has `heads`, `kv_heads`, `dim`, `vdim`, `scale`,
`conv` (taps of the convolution on its projections; absent or 0: none), `mask.size` (the
window; absent: every earlier position), `rot` {`base`, `dims`, `scaling` {`factor`, `low`,
`high`, `original`}} and optionally `kv_from`, the layer whose keys and values it reads.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class WavelengthScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class RotaryConfig:
    dims: int                 # how many numbers of a head turn (0: none)
    base: float
    scaling: Optional[WavelengthScaling]


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: Optional[int]     # None: queries are projected straight from the layer's input
    scale: float
    rot: RotaryConfig


@dataclass(frozen=True)
class WindowMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    taps: int                 # taps of the convolution on q, k, v (0: none)
    window: Optional[int]
    rot: RotaryConfig
    kv_from: Optional[int]


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                 # 'dense' | 'moe'
    ff: int
    limit: float
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class TuzapelLayer:
    type: str                 # 'latent_attention' | 'attention'
    mixer: Any
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class TuzapelConfig:
    vocab: int
    width: int
    eps: float
    logit_softcap: float
    layers: Tuple[TuzapelLayer, ...]
    architecture: str = "Tuzapel"

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "TuzapelConfig":
        r = KeyReader(raw)
        vocab = r.need_int("vocab", 1)
        width = r.need_int("width", 1)
        eps = _sub(r, "norm").need_float("eps")
        if not eps > 0:
            raise ConfigError(f"config.json: key 'norm.eps' must be > 0, got {eps}")
        cap = r.opt_float("logit_softcap", 0.0)
        if cap < 0:
            raise ConfigError(f"config.json: key 'logit_softcap' must be >= 0, got {cap}")
        entries = r.opt_raw("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = tuple(_layer(x, i) for i, x in enumerate(entries))
        for i, layer in enumerate(layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            where = f"config.json: layers[{i}]: 'mixer.kv_from'"
            if not 0 <= src < i or layers[src].type != "attention" \
                    or layers[src].mixer.kv_from is not None:
                raise ConfigError(f"{where} must name an earlier attention layer with keys and "
                                  f"values of its own, got {src}")
            a, b = layer.mixer, layers[src].mixer
            if (a.kv_heads, a.dim, a.vdim, a.rot) != (b.kv_heads, b.dim, b.vdim, b.rot):
                raise ConfigError(f"{where}: layer {src}'s key/value heads, sizes or rotation "
                                  f"differ from this layer's")
        return TuzapelConfig(vocab, width, eps, cap, layers)


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.opt_raw(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _rot(m: KeyReader, where: str, most: int, default_dims: int) -> RotaryConfig:
    if m.opt_raw("rot") is None:
        return RotaryConfig(0, 10000.0, None)
    rot = _sub(m, "rot")
    dims = rot.opt_int("dims", default_dims, 0)
    if dims % 2 or dims > most:
        raise ConfigError(f"{where}: 'rot.dims' must be even and at most {most}, got {dims}")
    base = rot.need_float("base")
    if not base > 0:
        raise ConfigError(f"{where}: 'rot.base' must be > 0, got {base}")
    scaling = None
    if rot.opt_raw("scaling") is not None:
        s = _sub(rot, "scaling")
        scaling = WavelengthScaling(s.need_float("factor"), s.need_float("low"),
                                    s.need_float("high"), s.need_float("original"))
        if not scaling.factor > 0 or not scaling.high > scaling.low or not scaling.low > 0 \
                or not scaling.original > 0:
            raise ConfigError(f"{where}: 'rot.scaling' needs factor > 0, 0 < low < high, "
                              f"original > 0")
    return RotaryConfig(dims, base, scaling)


def _layer(entry: Any, i: int) -> TuzapelLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(entry, where)
    kind = r.opt_str("type", None)
    m = _sub(r, "mixer")
    if kind == "latent_attention":
        rot_dim = m.need_int("rot_dim", 0)
        mixer = LatentMixerConfig(m.need_int("heads", 1), m.need_int("dim", 1), rot_dim,
                                  m.need_int("vdim", 1), m.need_int("kv_rank", 1),
                                  m.opt_int("q_rank", None, 1), m.need_float("scale"),
                                  _rot(m, where, rot_dim, rot_dim))
    elif kind == "attention":
        heads = m.need_int("heads", 1)
        kv_heads = m.opt_int("kv_heads", heads, 1)
        if heads % kv_heads:
            raise ConfigError(f"{where}: 'mixer.heads' must be a multiple of 'mixer.kv_heads'")
        dim = m.need_int("dim", 1)
        window = None
        if m.opt_raw("mask") is not None:
            window = _sub(m, "mask").opt_int("size", None, 1)
        mixer = WindowMixerConfig(heads, kv_heads, dim, m.need_int("vdim", 1),
                                  m.need_float("scale"), m.opt_int("conv", 0, 0), window,
                                  _rot(m, where, dim, dim), m.opt_int("kv_from", None, 0))
    else:
        raise ConfigError(f"{where}: 'type' must be 'latent_attention' or 'attention', got {kind!r}")
    if not mixer.scale > 0:
        raise ConfigError(f"{where}: 'mixer.scale' must be > 0, got {mixer.scale}")
    mlp = None
    if r.opt_raw("mlp") is not None:
        f = _sub(r, "mlp")
        fk = f.opt_str("kind", "dense")
        if fk == "dense":
            mlp = FeedForwardConfig("dense", f.need_int("ff", 1), f.need_float("limit"))
        elif fk == "moe":
            e, rt = _sub(f, "expert"), _sub(f, "router")
            mlp = FeedForwardConfig("moe", e.need_int("ff", 1), e.need_float("limit"),
                                    rt.need_int("experts", 1), rt.need_int("top", 1))
            if mlp.top > mlp.experts:
                raise ConfigError(f"{where}: 'mlp.router.top' exceeds 'mlp.router.experts'")
        else:
            raise ConfigError(f"{where}: 'mlp.kind' must be 'dense' or 'moe', got {fk!r}")
        if not mlp.limit > 0:
            raise ConfigError(f"{where}: the feed-forward's 'limit' must be > 0, got {mlp.limit}")
    return TuzapelLayer(kind, mixer, mlp)
