"""Fopinex in plain 64-bit arithmetic: one function per mechanism, whole sequences, no cache.

The oracle of the Fopinex tests. It shares no code with the engine: weights come as a dict
name -> tensor, the configuration as the dict that config.json holds. Notation: h is what a
sublayer reads, n(x) = x / sqrt(mean(x^2) + eps) * gain.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

D = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, gain, eps):
    return rms(x, eps) * gain.to(D)


def lin(w: Dict[str, torch.Tensor], name: str, x: torch.Tensor) -> torch.Tensor:
    return x @ w[name].to(D).T


def chunk_mask(n: int, size: Optional[int]) -> torch.Tensor:
    """[n, n] bool: row i sees column j when j <= i and both lie in the same chunk of `size`
    positions counted from 0 (None: plain causal)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    m = j <= i
    if size is not None:
        m = m & ((i // size) == (j // size))
    return m


def keys_values(w, prefix: str, mixer: dict, h: torch.Tensor):
    """k [G, n, dim], v [G, n, vdim] of the layer that owns the projections."""
    n = h.shape[0]
    g = mixer["kv_heads"]
    k = lin(w, prefix + "k", h).reshape(n, g, mixer["dim"]).transpose(0, 1)
    v = lin(w, prefix + "v", h).reshape(n, g, mixer["vdim"]).transpose(0, 1)
    return k, v


def sigmoid_attention(w, prefix: str, mixer: dict, h: torch.Tensor, kv) -> torch.Tensor:
    """Unnormalised attention: the weight of a visible key is sigmoid(score + bias of the
    head); the heads' weights are mixed by a [H, H] matrix; head a applies its mixed weights
    to the values of its own key/value head. `kv`: keys and values (its own or another
    layer's)."""
    n = h.shape[0]
    hq, g, d, dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = lin(w, prefix + "q", h).reshape(n, hq, d).transpose(0, 1)          # [H, n, d]
    k, v = kv
    per = hq // g
    size = (mixer.get("mask") or {}).get("size")
    vis = chunk_mask(n, size)
    wts = torch.zeros(hq, n, n, dtype=D)
    for a in range(hq):
        s = q[a] @ k[a // per].T * mixer["scale"] + w[prefix + "pb"].to(D)[a]
        wts[a] = torch.where(vis, torch.sigmoid(s), torch.zeros((), dtype=D))
    mixed = torch.einsum("ab,bij->aij", w[prefix + "talk"].to(D), wts)
    out = torch.stack([mixed[a] @ v[a // per] for a in range(hq)], 1)       # [n, H, dv]
    return lin(w, prefix + "o", out.reshape(n, hq * dv))


def gla_decay(w, prefix: str, mixer: dict, h: torch.Tensor) -> torch.Tensor:
    """alpha [n, heads, dim] = sigmoid(z)^(1 / tau), z a low-rank projection plus a bias."""
    z = lin(w, prefix + "a2", lin(w, prefix + "a1", h)) + w[prefix + "a2.b"].to(D)
    return torch.exp(torch.nn.functional.logsigmoid(z) / mixer["tau"]).reshape(
        h.shape[0], mixer["heads"], mixer["dim"])


def gla(w, prefix: str, mixer: dict, h: torch.Tensor, eps: float,
        state: Optional[torch.Tensor] = None):
    """Gated linear attention, token by token: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t;
    every head's o normed over vdim, times silu(W_g h), through W_o. Returns (y, S)."""
    n = h.shape[0]
    hh, d, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = lin(w, prefix + "q", h).reshape(n, hh, d) * d ** -0.5
    k = lin(w, prefix + "k", h).reshape(n, hh, d)
    v = lin(w, prefix + "v", h).reshape(n, hh, dv)
    alpha = gla_decay(w, prefix, mixer, h)
    s = torch.zeros(hh, d, dv, dtype=D) if state is None else state.clone()
    o = torch.zeros(n, hh, dv, dtype=D)
    for t in range(n):
        s = alpha[t][:, :, None] * s + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hd,hdv->hv", q[t], s)
    o = rms(o, eps) * w[prefix + "norm"].to(D)
    gate = lin(w, prefix + "g", h)
    y = o.reshape(n, hh * dv) * (gate * torch.sigmoid(gate))
    return lin(w, prefix + "o", y), s


def route(w, prefix: str, mlp: dict, h: torch.Tensor):
    """(ids [n, top], weights [n, top], margin [n]): softmax over all router outputs; the choice
    adds a correction per output and is limited to the best groups of neighbours (a group's
    score: its largest choice score); weights are the plain scores. margin: how far the
    nearest decision (a group or an expert, in or out) was from going the other way."""
    r = mlp["router"]
    total = r["experts"] + r.get("identity", 0)
    s = torch.softmax(lin(w, prefix + "router", h), -1)
    choice = s + w[prefix + "correction"].to(D)
    n = h.shape[0]
    margin = torch.full((n,), math.inf, dtype=D)
    groups = r.get("groups")
    if groups and groups["count"] > 1:
        per = total // groups["count"]
        best = choice.reshape(n, groups["count"], per).max(-1).values
        order = best.sort(-1, descending=True).values
        keep = groups["keep"]
        if keep < groups["count"]:
            margin = torch.minimum(margin, order[:, keep - 1] - order[:, keep])
        kept = best >= order[:, keep - 1:keep]
        choice = torch.where(kept.repeat_interleave(per, -1), choice,
                             torch.full((), -math.inf, dtype=D))
    order = choice.sort(-1, descending=True)
    top = r["top"]
    if top < total:
        gap = order.values[:, top - 1] - order.values[:, top]
        margin = torch.minimum(margin, torch.where(torch.isfinite(gap), gap,
                                                   torch.full((), math.inf, dtype=D)))
    ids = order.indices[:, :top]
    return ids, s.gather(-1, ids), margin


def expert(w, prefix: str, limit: float, h: torch.Tensor) -> torch.Tensor:
    g = torch.clamp(lin(w, prefix + "gate", h), max=limit)
    u = torch.clamp(lin(w, prefix + "up", h), -limit, limit)
    return lin(w, prefix + "down", g * torch.sigmoid(1.702 * g) * (u + 1))


def moe(w, prefix: str, mlp: dict, h: torch.Tensor, margins: Optional[List[torch.Tensor]] = None):
    """`margins` receives, per call, how clear every row's routing was (see `route`)."""
    ids, wts, margin = route(w, prefix, mlp, h)
    if margins is not None:
        margins.append(margin)
    real = mlp["router"]["experts"]
    out = torch.zeros_like(h)
    for e in range(real + mlp["router"].get("identity", 0)):
        share = torch.where(ids == e, wts, torch.zeros((), dtype=D)).sum(-1)      # [n]
        rows = share.nonzero().flatten()
        if rows.numel() == 0:
            continue
        x = h[rows]
        # an identity expert hands its input back
        y = x if e >= real else expert(w, f"{prefix}e{e}.", mlp["expert"]["limit"], x)
        out[rows] += share[rows, None] * y
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens, margins: Optional[List[torch.Tensor]] = None):
    """(logits [n, vocab], the residual stream after every layer [L, n, width]) of one whole
    sequence from position 0."""
    eps = cfg["norm"]["eps"]
    m = cfg["residual_mult"]
    x = w["embed"].to(D)[torch.as_tensor(tokens, dtype=torch.long)]
    kv_of = {}
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mixer = layer["mixer"]
        h1 = norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            src = mixer.get("kv_from")
            if src is None:
                kv_of[i] = keys_values(w, p + "mix.", mixer, h1)
                src = i
            a = sigmoid_attention(w, p + "mix.", mixer, h1, kv_of[src])
        elif layer["type"] == "gla":
            a, _ = gla(w, p + "mix.", mixer, h1, eps)
        else:
            raise ValueError(layer["type"])
        total = a * torch.sigmoid(lin(w, p + "rg1", h1) + w[p + "rg1.b"].to(D))
        if layer.get("mlp") is not None:
            h2 = norm(x, w[p + "norm2"], eps)
            f = moe(w, p + "mlp.", layer["mlp"], h2, margins)
            total = total + f * torch.sigmoid(lin(w, p + "rg2", h2) + w[p + "rg2.b"].to(D))
        x = x + m * total
        streams.append(x)
    logits = lin(w, "head", norm(x, w["final.norm"], eps))
    return logits, torch.stack(streams)
