"""Tuzapel in plain 64-bit arithmetic: one function per mechanism, whole sequences, no cache.

The oracle of the Tuzapel tests. It shares no code with the engine: weights come as a dict
name -> tensor, the configuration as the dict that config.json holds. Notation: h is what a
sublayer reads; ln(x) = (x - mean) / sqrt(var + eps) * w; rms(x) = x / sqrt(mean(x^2) + eps).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

D = torch.float64
EXPERT_ALPHA = 1.702


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w.to(D)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(D)


def lin(w: Dict[str, torch.Tensor], name: str, x: torch.Tensor) -> torch.Tensor:
    return x @ w[name].to(D).T


def frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` the long wavelengths are slowed
    down by `factor`, the short ones kept, those between blended."""
    dims = rot["dims"]
    f = [rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        out = []
        for x in f:
            wave = 2 * math.pi / x
            if wave < sc["original"] / sc["high"]:
                out.append(x)
            elif wave > sc["original"] / sc["low"]:
                out.append(x / sc["factor"])
            else:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1 - s) * x / sc["factor"] + s * x)
        f = out
    return torch.tensor(f, dtype=D)


def rotate(x: torch.Tensor, pos: torch.Tensor, rot: dict, pairing: str) -> torch.Tensor:
    """x [n, heads, d]: the first rot.dims numbers of every head turn by pos * f_i; pair i is
    (2i, 2i + 1) when `pairing` is 'interleaved', (i, i + dims / 2) when 'half'."""
    dims = (rot or {}).get("dims", 0)
    if not dims:
        return x
    ang = pos.to(D)[:, None] * frequencies(rot)[None, :]          # [n, dims / 2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if pairing == "interleaved":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def short_conv(u: torch.Tensor, w: torch.Tensor, before: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel; u [n, channels], w [channels,
    taps]; `before` [taps - 1, channels]: what came before the first row (None: zeros)."""
    n, ch = u.shape
    taps = w.shape[1]
    pad = torch.zeros(taps - 1, ch, dtype=D) if before is None else before.to(D)
    ext = torch.cat([pad, u], 0)
    y = torch.zeros(n, ch, dtype=D)
    for j in range(taps):
        y += w.to(D)[:, j][None, :] * ext[j:j + n]
    return y


def visible(n: int, window: Optional[int]) -> torch.Tensor:
    """[n, n] bool: row i sees column j when 0 <= i - j (< window, when there is one)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    m = j <= i
    if window is not None:
        m = m & (i - j < window)
    return m


def softmax_rows(s: torch.Tensor, vis: torch.Tensor, sink: bool) -> torch.Tensor:
    """Softmax over the visible columns; with `sink` the denominator has one more term,
    exp(0), that belongs to no column."""
    s = torch.where(vis, s, torch.full((), -math.inf, dtype=D))
    m = s.max(-1, keepdim=True).values
    if sink:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink:
        den = den + torch.exp(-m)
    return e / den


def latent_attention(w, prefix: str, mixer: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, rd, dv, R = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    pos = torch.arange(n)
    if mixer.get("q_rank"):
        cq = rms_norm(lin(w, prefix + "dq", h), w[prefix + "dq.norm"], eps)
        q = lin(w, prefix + "uq", cq).reshape(n, H, d + rd)
    else:
        q = lin(w, prefix + "q", h).reshape(n, H, d + rd)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], pos, mixer.get("rot"), "interleaved")
    ckv = lin(w, prefix + "dkv", h)
    c = rms_norm(ckv[:, :R], w[prefix + "dkv.norm"], eps)
    k_rot = rotate(ckv[:, None, R:], pos, mixer.get("rot"), "interleaved")[:, 0]      # [n, rd]
    k_plain = lin(w, prefix + "uk", c).reshape(n, H, d)
    v = lin(w, prefix + "uv", c).reshape(n, H, dv)
    vis = visible(n, None)
    out = torch.zeros(n, H, dv, dtype=D)
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * mixer["scale"]
        out[:, a] = softmax_rows(s, vis, False) @ v[:, a]
    return lin(w, prefix + "o", out.reshape(n, H * dv))


def window_keys_values(w, prefix: str, mixer: dict, h: torch.Tensor, eps: float):
    """k [n, G, dim] after convolution, norm and rotation; v [n, G, vdim] after convolution."""
    n = h.shape[0]
    G, d, dv = mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    k, v = lin(w, prefix + "k", h), lin(w, prefix + "v", h)
    if mixer.get("conv"):
        k, v = short_conv(k, w[prefix + "k.conv"]), short_conv(v, w[prefix + "v.conv"])
    k, v = k.reshape(n, G, d), v.reshape(n, G, dv)
    k = rms_norm(k, w[prefix + "k.norm"], eps)
    k = rotate(k, torch.arange(n), mixer.get("rot"), "half")
    return k, v


def window_attention(w, prefix: str, mixer: dict, h: torch.Tensor, eps: float, kv) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = lin(w, prefix + "q", h)
    if mixer.get("conv"):
        q = short_conv(q, w[prefix + "q.conv"])
    q = q.reshape(n, H, d)
    q = rotate(rms_norm(q, w[prefix + "q.norm"], eps), torch.arange(n), mixer.get("rot"), "half")
    k, v = kv
    vis = visible(n, (mixer.get("mask") or {}).get("size"))
    per = H // G
    out = torch.zeros(n, H, dv, dtype=D)
    for a in range(H):
        s = q[:, a] @ k[:, a // per].T * mixer["scale"]
        out[:, a] = softmax_rows(s, vis, True) @ v[:, a // per]
    return lin(w, prefix + "o", out.reshape(n, H * dv))


def expert(w, prefix: str, limit: float, h: torch.Tensor) -> torch.Tensor:
    g = torch.clamp(lin(w, prefix + "gate", h), max=limit)
    u = torch.clamp(lin(w, prefix + "up", h), -limit, limit)
    return lin(w, prefix + "down", g * torch.sigmoid(EXPERT_ALPHA * g) * (u + 1))


def route(w, prefix: str, mlp: dict, h: torch.Tensor):
    """(ids [n, top], weights [n, top], margin [n]): the `top` largest logits, softmax over
    them alone; margin: how far the last chosen logit lies above the first that is not."""
    r = mlp["router"]
    z = lin(w, prefix + "router", h) + w[prefix + "router.b"].to(D)
    order = z.sort(-1, descending=True)
    top = r["top"]
    ids = order.indices[:, :top]
    wts = torch.softmax(order.values[:, :top], -1)
    margin = (order.values[:, top - 1] - order.values[:, top]) if top < r["experts"] \
        else torch.full((h.shape[0],), math.inf, dtype=D)
    return ids, wts, margin


def feed_forward(w, prefix: str, mlp: dict, h: torch.Tensor):
    """(y, margin of the routing: inf for a dense layer)."""
    if mlp["kind"] == "dense":
        return expert(w, prefix, mlp["limit"], h), torch.full((h.shape[0],), math.inf, dtype=D)
    ids, wts, margin = route(w, prefix, mlp, h)
    y = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=D)
    for e in range(mlp["router"]["experts"]):
        ye = expert(w, f"{prefix}e{e}.", mlp["expert"]["limit"], h)
        y += ((ids == e).to(D) * wts).sum(-1, keepdim=True) * ye
    return y, margin


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> Tuple[torch.Tensor, List[torch.Tensor], torch.Tensor]:
    """(logits [n, vocab], the stream after every layer, the least routing margin per row)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"].to(D)[torch.as_tensor(tokens, dtype=torch.long)]
    n = x.shape[0]
    streams = []
    margin = torch.full((n,), math.inf, dtype=D)
    kvs = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            y = latent_attention(w, p + "mix.", m, h, eps)
        else:
            src = m.get("kv_from")
            if src is None:
                kvs[i] = window_keys_values(w, p + "mix.", m, h, eps)
                src = i
            y = window_attention(w, p + "mix.", m, h, eps, kvs[src])
        x = x + layer_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = layer_norm(x, w[p + "norm2"], eps)
            y, mg = feed_forward(w, p + "mlp.", layer["mlp"], h)
            margin = torch.minimum(margin, mg)
            x = x + layer_norm(y, w[p + "norm2b"], eps)
        streams.append(x.clone())
    z = lin(w, "embed", layer_norm(x, w["final.norm"], eps))
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return z, streams, margin
