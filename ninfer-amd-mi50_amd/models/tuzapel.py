"""Tuzapel put together from parts, layer by layer from its configuration.

x = embed[token]; every layer has a norm before and after each sublayer,
    x += ln1b(mixer(ln1(x))),   x += ln2b(ff(ln2(x)))      (ln: layer norm with a weight, no bias)
where the mixer is latent attention (queries through a latent of their own, rotated parts in
neighbouring pairs, plain causal softmax) or windowed attention with grouped key/value heads
(a short causal convolution on the projected q, k and v, heads normed before they turn in
half-split pairs at frequencies slowed down by wavelength, a softmax with a sink; a layer may
read the keys and values an earlier layer has cached), and the feed-forward, when the layer has
one, is a clamped gated product, dense or as routed experts (logits with a bias, the largest
chosen, softmax over the chosen). logits = cap tanh(embed ln(x) / cap).
Tensor names: embed, final.norm, and per layer l<i>.{norm1, norm1b, norm2, norm2b, mix.{dq,
dq.norm, uq, dkv, dkv.norm, uk, uv, o} or mix.{q, k, v, o, q.norm, k.norm, q.conv, k.conv,
v.conv}, mlp.{gate, up, down} or mlp.{router, router.b, e<j>.{gate, up, down}}}.
"""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the part factories by kind and name)
from ..config.tuzapel import TuzapelConfig
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import make_part, register_architecture
from .spec import LayerCall, ModelSpec

# fixed by the design: the factor on a gate inside its sigmoid
GATE_ALPHA = 1.702


def _position(rot, pairing: str):
    if not rot.dims:
        return make_part("position", "none")
    s = rot.scaling
    return make_part("position", "rotary", rot_dim=rot.dims, theta=rot.base, pairing=pairing,
                     scaling=None if s is None else {"factor": s.factor, "original": s.original,
                                                     "low": s.low, "high": s.high})


def build_tuzapel(cfg: TuzapelConfig) -> ModelSpec:
    w = cfg.width
    embedding = TokenEmbedding("embed", cfg.vocab, w, leaf="")
    # a cache keeps what the widest window among its own layer and its readers sees
    keep = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type != "attention":
            continue
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        span = layer.mixer.window
        if owner in keep and (keep[owner] is None or span is None):
            keep[owner] = None
        else:
            keep[owner] = span if owner not in keep else max(keep[owner], span)
    blocks, plan = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        if layer.type == "latent_attention":
            mixer = make_part("mixer", "latent_attention", prefix=p + "mix.", hidden=w,
                              heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim,
                              kv_rank=m.kv_rank, scale=m.scale, eps=cfg.eps,
                              position=_position(m.rot, "interleaved"), output_gate=False,
                              q_rank=m.q_rank)
            plan.append(LayerCall(i))
        else:
            own = m.kv_from is None
            mixer = make_part("mixer", "attention", prefix=p + "mix.", hidden=w, heads=m.heads,
                              kv_heads=m.kv_heads, head_dim=m.dim, vdim=m.vdim,
                              position=_position(m.rot, "half"), qkv_bias=False, window=m.window,
                              scale=m.scale, qk_norm_eps=cfg.eps, conv_taps=m.taps, sink=True,
                              own_kv=own, cache_window=keep[i] if own else m.window,
                              names={"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm",
                                     "k_norm": "k.norm", "conv": ".conv"})
            plan.append(LayerCall(i, cache_from=m.kv_from))
        ff = ff_norm = ff_out = None
        f = layer.mlp
        if f is not None:
            if f.kind == "dense":
                ff = make_part("feed_forward", "swiglu", prefix=p + "mlp.", hidden=w, inner=f.ff,
                               act="clamped_swish", act_limit=f.limit, act_alpha=GATE_ALPHA,
                               names=("gate", "up", "down"))
            else:
                ff = make_part(
                    "feed_forward", "sparse_moe", prefix=p + "mlp.", hidden=w, experts=f.experts,
                    top_k=f.top, inner=f.ff, renorm=True, act="clamped_swish", act_limit=f.limit,
                    act_alpha=GATE_ALPHA, router={"score": "softmax", "logit_bias_leaf": "router.b"},
                    names={"router": "", "router_leaf": "router", "experts": "e",
                           "expert_leaves": ("gate", "up", "down")})
            ff_norm = make_part("norm", "layernorm", prefix=p + "norm2", size=w, eps=cfg.eps, leaf="")
            ff_out = make_part("norm", "output_layernorm", tensor=p + "norm2b", size=w, eps=cfg.eps)
        blocks.append(make_part(
            "block", "sandwich",
            mixer_norm=make_part("norm", "layernorm", prefix=p + "norm1", size=w, eps=cfg.eps, leaf=""),
            mixer=mixer,
            mixer_out_norm=make_part("norm", "output_layernorm", tensor=p + "norm1b", size=w, eps=cfg.eps),
            ff_norm=ff_norm, feed_forward=ff, ff_out_norm=ff_out))
    final_norm = make_part("norm", "layernorm", prefix="final.norm", size=w, eps=cfg.eps, leaf="")
    head = LMHead("head", cfg.vocab, w, tied_to=embedding, leaf="", softcap=cfg.logit_softcap)
    return ModelSpec(embedding, blocks, final_norm, head, plan=plan)


register_architecture("Tuzapel", TuzapelConfig.from_dict, build_tuzapel)
