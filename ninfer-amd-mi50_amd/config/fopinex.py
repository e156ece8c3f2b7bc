"""Typed configuration of Fopinex, a decoder-only model of gated parallel sublayers.

config.json keys: `architecture` ("Fopinex"), `vocab`, `width`, `norm.eps`, `residual_mult`,
and `layers`: a list of objects with `type` ('attention' or 'gla'), `mixer` (the mixer's sizes
and constants) and `mlp` (null, or {'kind': 'moe', 'expert': {'ff', 'limit'}, 'router':
{'experts', 'top', 'identity', 'groups': {'count', 'keep'}}}).
An attention mixer has `heads`, `kv_heads`, `dim`, `vdim`, `scale`, optionally `mask.size` (the
chunk of positions a row sees) and `kv_from` (the layer whose keys and values it reads); a gla
mixer has `heads`, `dim`, `vdim`, `tau` and optionally `rank` (the inner size of its decay's
two-step projection; without the key the checkpoint's tensors decide).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class SigmoidMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]     # a row sees the keys of its own chunk of so many positions; None: all
    kv_from: Optional[int]   # the layer whose cache holds this layer's keys and values


@dataclass(frozen=True)
class GlaMixerConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int]      # None: whatever the checkpoint's tensors hold


@dataclass(frozen=True)
class MoeConfig:
    ff: int
    limit: float
    experts: int             # experts with weights
    identity: int            # router outputs beyond them whose expert hands its input back
    top: int
    groups: int
    groups_kept: int


@dataclass(frozen=True)
class FopinexLayer:
    type: str                # 'attention' | 'gla'
    mixer: Any               # SigmoidMixerConfig | GlaMixerConfig
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class FopinexConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: Tuple[FopinexLayer, ...]
    architecture: str = "Fopinex"

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "FopinexConfig":
        r = KeyReader(raw)
        vocab = r.need_int("vocab", 1)
        width = r.need_int("width", 1)
        eps = _sub(r, "norm").need_float("eps")
        if not eps > 0:
            raise ConfigError(f"config.json: key 'norm.eps' must be > 0, got {eps}")
        mult = r.need_float("residual_mult")
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
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise ConfigError(f"{where}: layer {src} holds {b.kv_heads} heads of {b.dim} and "
                                  f"{b.vdim} numbers, this layer reads {a.kv_heads} of {a.dim} and "
                                  f"{a.vdim}")
        return FopinexConfig(vocab, width, eps, mult, layers)


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.opt_raw(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _layer(entry: Any, i: int) -> FopinexLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(entry, where)
    kind = r.opt_str("type", None)
    m = _sub(r, "mixer")
    if kind == "attention":
        heads = m.need_int("heads", 1)
        kv_heads = m.opt_int("kv_heads", heads, 1)
        if heads % kv_heads:
            raise ConfigError(f"{where}: 'mixer.heads' must be a multiple of 'mixer.kv_heads'")
        chunk = None
        if m.opt_raw("mask") is not None:
            chunk = _sub(m, "mask").opt_int("size", None, 1)
        mixer = SigmoidMixerConfig(heads, kv_heads, m.need_int("dim", 1), m.need_int("vdim", 1),
                                   m.need_float("scale"), chunk, m.opt_int("kv_from", None, 0))
    elif kind == "gla":
        tau = m.need_float("tau")
        if not tau > 0:
            raise ConfigError(f"{where}: 'mixer.tau' must be > 0, got {tau}")
        mixer = GlaMixerConfig(m.need_int("heads", 1), m.need_int("dim", 1), m.need_int("vdim", 1),
                               tau, m.opt_int("rank", None, 1))
    else:
        raise ConfigError(f"{where}: 'type' must be 'attention' or 'gla', got {kind!r}")
    mlp = None
    if r.opt_raw("mlp") is not None:
        f = _sub(r, "mlp")
        fk = f.opt_str("kind", "moe")
        if fk != "moe":
            raise ConfigError(f"{where}: 'mlp.kind' must be 'moe', got {fk!r}")
        rt = _sub(f, "router")
        experts, top = rt.need_int("experts", 1), rt.need_int("top", 1)
        identity = rt.opt_int("identity", 0, 0)
        groups, kept = 1, 1
        if rt.opt_raw("groups") is not None:
            g = _sub(rt, "groups")
            groups = g.need_int("count", 1)
            kept = g.opt_int("keep", groups, 1)
        total = experts + identity
        if top > total or total % groups or kept > groups or kept * (total // groups) < top:
            raise ConfigError(f"{where}: 'mlp.router' does not fit: {experts} experts and "
                              f"{identity} identity experts, top {top}, {groups} groups of which "
                              f"{kept} are kept")
        e = _sub(f, "expert")
        limit = e.need_float("limit")
        if not limit > 0:
            raise ConfigError(f"{where}: 'mlp.expert.limit' must be > 0, got {limit}")
        mlp = MoeConfig(e.need_int("ff", 1), limit, experts, identity, top, groups, kept)
    return FopinexLayer(kind, mixer, mlp)
