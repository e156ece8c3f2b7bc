"""Fopinex put together from parts, layer by layer from its configuration.

x = embed[token]; every layer is a parallel block with two norms of the same x and gated
sublayers,
    x += m (sigmoid(R1 h1 + r1) * mixer(h1) + sigmoid(R2 h2 + r2) * ff(h2)),
    h1 = norm1(x), h2 = norm2(x), m = residual_mult,
where the mixer is attention without a softmax (sigmoid weights with a bias per head, the
heads' weights mixed by a matrix, a row seeing the keys of its own chunk of positions; a layer
may read the keys and values that an earlier layer has written) or gated linear attention, and
the feed-forward, when the layer has one, is routed experts: softmax scores over the experts
and a few identity experts (which hand their input back), a correction per output that decides
the choice only, the choice limited to the best groups of neighbours, the chosen scores as
weights. logits = head norm(x).
Tensor names: embed, final.norm, head, and per layer l<i>.{norm1, norm2, rg1, rg1.b, rg2,
rg2.b, mix.{q, k, v, o, pb, talk} or mix.{q, k, v, g, o, norm, a1, a2, a2.b}, mlp.{router,
correction, e<j>.{gate, up, down}}}.
"""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the part factories by kind and name)
from ..config.fopinex import FopinexConfig
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import make_part, register_architecture
from .spec import LayerCall, ModelSpec

# fixed by the design: the factor on an expert's gate inside its sigmoid
EXPERT_GATE_ALPHA = 1.702


def build_fopinex(cfg: FopinexConfig) -> ModelSpec:
    w = cfg.width
    embedding = TokenEmbedding("embed", cfg.vocab, w, leaf="")
    blocks, plan = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        if layer.type == "attention":
            mixer = make_part("mixer", "sigmoid_attention", prefix=p + "mix.", hidden=w,
                              heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim,
                              scale=m.scale, chunk=m.chunk, own_kv=m.kv_from is None)
            plan.append(LayerCall(i, cache_from=m.kv_from))
        else:
            mixer = make_part("mixer", "gated_linear_attention", prefix=p + "mix.", hidden=w,
                              heads=m.heads, dim=m.dim, vdim=m.vdim, tau=m.tau, eps=cfg.eps,
                              rank=m.rank)
            plan.append(LayerCall(i))
        ff = None
        f = layer.mlp
        if f is not None:
            ff = make_part(
                "feed_forward", "sparse_moe", prefix=p + "mlp.", hidden=w, experts=f.experts,
                top_k=f.top, inner=f.ff, renorm=False, act="clamped_swish", act_limit=f.limit,
                act_alpha=EXPERT_GATE_ALPHA, identity=f.identity,
                router={"score": "softmax", "choice_bias": True, "choice_bias_leaf": "correction",
                        "n_group": f.groups, "topk_group": f.groups_kept},
                names={"router": "", "router_leaf": "router", "experts": "e",
                       "expert_leaves": ("gate", "up", "down")})
        blocks.append(make_part(
            "block", "parallel",
            norm=make_part("norm", "rmsnorm", prefix=p + "norm1", size=w, eps=cfg.eps, leaf=""),
            ff_norm=make_part("norm", "rmsnorm", prefix=p + "norm2", size=w, eps=cfg.eps, leaf=""),
            mixer=mixer, feed_forward=ff, size=w, mult=cfg.residual_mult, mixer_gate=p + "rg1",
            ff_gate=p + "rg2"))
    final_norm = make_part("norm", "rmsnorm", prefix="final.norm", size=w, eps=cfg.eps, leaf="")
    head = LMHead("head", cfg.vocab, w, leaf="")
    return ModelSpec(embedding, blocks, final_norm, head, plan=plan)


register_architecture("Fopinex", FopinexConfig.from_dict, build_fopinex)
