"""Small Fopinex configurations for the tests: sizes that no fast kernel's tiling suits, sizes
that suit them, and one in which much is 1 or absent (one head, one expert, no groups, no
identity expert, no mask, a layer without a feed-forward, a multiplier of 1)."""
import math
import random


def attention(heads, kv_heads, dim, vdim, chunk=None, kv_from=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if chunk:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def gla(heads, dim, vdim, tau, rank):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}}


def moe(ff, experts, top, identity=0, groups=None, limit=2.0):
    r = {"experts": experts, "top": top, "identity": identity}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config_odd():
    return {"architecture": "Fopinex", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
            "residual_mult": 0.7,
            "layers": [layer(attention(6, 3, 12, 20, chunk=10), moe(24, 7, 3, identity=2, groups=(3, 2))),
                       layer(gla(3, 10, 12, 5.0, 7), None),
                       layer(attention(6, 3, 12, 20, chunk=27, kv_from=0), moe(40, 4, 2, identity=1, limit=0.8)),
                       layer(attention(3, 1, 20, 36), moe(16, 6, 3, identity=3, groups=(3, 1))),
                       layer(gla(2, 24, 20, 2.5, 3), moe(24, 5, 2, identity=1, groups=(2, 2)))]}


def config_even():
    return {"architecture": "Fopinex", "vocab": 384, "width": 128, "norm": {"eps": 1e-6},
            "residual_mult": 0.5,
            "layers": [layer(attention(4, 2, 64, 32, chunk=32), moe(64, 8, 2, identity=0, groups=(4, 2))),
                       layer(attention(4, 2, 64, 32, chunk=48, kv_from=0), moe(32, 12, 4, identity=4, groups=(2, 1))),
                       layer(gla(2, 64, 64, 16.0, 16), moe(64, 6, 2, identity=2)),
                       layer(attention(16, 4, 32, 128, chunk=40), None),
                       layer(gla(4, 128, 32, 8.0, 8), moe(32, 15, 3, identity=1, groups=(4, 3)))]}


def config_ones():
    return {"architecture": "Fopinex", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
            "residual_mult": 1.0,
            "layers": [layer(attention(1, 1, 16, 16), moe(16, 1, 1)),
                       layer(gla(1, 16, 16, 1.0, 1), moe(24, 1, 1, identity=1, groups=(2, 1))),
                       layer(attention(2, 2, 8, 24, chunk=1), None),
                       layer(attention(2, 2, 8, 24, chunk=64, kv_from=2), moe(16, 3, 3, identity=1, groups=(1, 1)))]}


CASES = {"odd": (config_odd, 11), "even": (config_even, 12), "ones": (config_ones, 13)}


def random_config(seed: int) -> dict:
    """A seeded random configuration: sizes, head counts, kinds and order of layers, chunks,
    what is absent."""
    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 136])
    layers = []
    owners = []
    for i in range(rng.randint(2, 5)):
        if rng.random() < 0.3:
            mixer = gla(rng.choice([1, 2, 3]), rng.choice([8, 12, 16, 32, 40]), rng.choice([8, 16, 20, 48]),
                        rng.choice([1.0, 4.0, 16.0]), rng.choice([1, 4, 9]))
        else:
            chunk = rng.choice([None, 3, 16, 31, 32, 50])
            if owners and rng.random() < 0.4:
                src = rng.choice(owners)
                m = layers[src]["mixer"]
                per = rng.choice([1, 2, 3])
                mixer = attention(m["kv_heads"] * per, m["kv_heads"], m["dim"], m["vdim"], chunk, kv_from=src)
            else:
                kv = rng.choice([1, 2, 3])
                mixer = attention(kv * rng.choice([1, 2, 4]), kv, rng.choice([8, 16, 24, 64]),
                                  rng.choice([8, 16, 40, 64]), chunk)
                owners.append(i)
        mlp = None
        if rng.random() < 0.8:
            count = rng.choice([1, 2, 3])
            per = rng.choice([1, 2, 4])
            total = count * per
            identity = rng.randint(0, total - 1)
            keep = rng.randint(1, count)
            mlp = moe(rng.choice([16, 24, 40]), total - identity, rng.randint(1, keep * per), identity,
                      (count, keep) if rng.random() < 0.8 else None, limit=rng.choice([0.5, 2.0, 7.0]))
            if mlp["router"].get("groups") is None:
                mlp["router"]["top"] = rng.randint(1, total)
        layers.append(layer(mixer, mlp))
    return {"architecture": "Fopinex", "vocab": rng.choice([97, 256, 333]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5])}, "residual_mult": rng.choice([0.3, 0.5, 1.0]),
            "layers": layers}
