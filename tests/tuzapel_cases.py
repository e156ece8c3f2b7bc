"""Small Tuzapel configurations for the tests: sizes that no fast kernel's tiling suits, sizes
that suit them, and one in which much is 1 or absent (one head, one tap, a window of one
position, one expert, no cap on the logits, no query latent, a layer without a feed-forward,
a layer without a window)."""
import math
import random


def rot(dims, base=10000.0, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim),
         "rot": rot(rot_dim, base)}
    if q_rank:
        m["q_rank"] = q_rank
    return {"type": "latent_attention", "mixer": m}


def attention(heads, kv_heads, dim, vdim, window=None, taps=0, rot_dims=None, base=10000.0,
              scaling=None, kv_from=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim),
         "rot": rot(dim if rot_dims is None else rot_dims, base, scaling)}
    if taps:
        m["conv"] = taps
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def dense(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config_odd():
    sc = (3.0, 1.0, 6.0, 48)
    return {"architecture": "Tuzapel", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
            "logit_softcap": 20.0,
            "layers": [layer(attention(6, 3, 20, 12, window=10, taps=4, rot_dims=10, scaling=sc), moe(24, 7, 3)),
                       layer(latent(3, 12, 6, 20, 40, q_rank=24), dense(40, limit=0.7)),
                       layer(attention(6, 3, 20, 12, window=27, taps=2, rot_dims=10, scaling=sc, kv_from=0), None),
                       layer(attention(3, 1, 36, 28, window=33, taps=3, rot_dims=36, base=500.0), moe(16, 5, 2, limit=0.9)),
                       layer(attention(6, 3, 20, 12, window=5, taps=4, rot_dims=10, scaling=sc, kv_from=0), dense(56))]}


def config_even():
    sc = (4.0, 1.0, 4.0, 64)
    return {"architecture": "Tuzapel", "vocab": 384, "width": 128, "norm": {"eps": 1e-6},
            "logit_softcap": 12.0,
            "layers": [layer(latent(4, 32, 16, 32, 64, q_rank=48, base=3000.0), moe(64, 12, 4)),
                       layer(attention(8, 2, 64, 32, window=32, taps=3, rot_dims=32, scaling=sc), dense(128)),
                       layer(attention(4, 4, 32, 96, window=48, taps=2, rot_dims=32, base=100000.0, scaling=sc), moe(32, 6, 2)),
                       layer(attention(8, 2, 64, 32, window=70, taps=3, rot_dims=32, scaling=sc, kv_from=1), moe(64, 8, 1)),
                       layer(latent(2, 64, 32, 64, 128, q_rank=32), dense(64, limit=3.0)),
                       layer(attention(16, 2, 64, 32, window=16, taps=3, rot_dims=64), None)]}


def config_ones():
    return {"architecture": "Tuzapel", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
            "layers": [layer(attention(1, 1, 16, 16, window=1, taps=1, rot_dims=2), moe(16, 1, 1)),
                       layer(latent(1, 16, 2, 8, 16), None),
                       layer(attention(2, 2, 8, 24, taps=0, rot_dims=0), dense(16)),
                       layer(attention(2, 2, 8, 24, window=2, taps=5, rot_dims=0, kv_from=2), moe(24, 3, 3))]}


CASES = {"odd": (config_odd, 21), "even": (config_even, 22), "ones": (config_ones, 23)}


def random_config(seed: int) -> dict:
    """A seeded random configuration: sizes, head counts, kinds and order of layers, windows,
    taps, what is absent."""
    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 136])
    layers, owners = [], []
    for i in range(rng.randint(2, 5)):
        if rng.random() < 0.3:
            rd = rng.choice([2, 8, 16])
            mixer = latent(rng.choice([1, 2, 4]), rng.choice([8, 16, 24]), rd, rng.choice([8, 16, 40]),
                           rng.choice([16, 32, 48]), q_rank=rng.choice([None, 8, 24]),
                           base=rng.choice([100.0, 10000.0]))
        else:
            window = rng.choice([None, 1, 3, 16, 31, 32, 50])
            taps = rng.choice([0, 1, 2, 3, 4])
            if owners and rng.random() < 0.4:
                src = rng.choice(owners)
                m = layers[src]["mixer"]
                mixer = attention(m["heads"], m["kv_heads"], m["dim"], m["vdim"], window=window, taps=taps,
                                  rot_dims=m["rot"]["dims"], base=m["rot"]["base"], kv_from=src,
                                  scale=rng.choice([None, 0.3]))
                if "scaling" in m["rot"]:
                    mixer["mixer"]["rot"]["scaling"] = dict(m["rot"]["scaling"])
            else:
                kv = rng.choice([1, 2, 3])
                dim = rng.choice([8, 12, 16, 32, 40, 64])
                mixer = attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([8, 16, 20, 48]),
                                  window=window, taps=taps, rot_dims=rng.choice([0, dim // 2 // 2 * 2, dim]),
                                  base=rng.choice([50.0, 10000.0]),
                                  scaling=rng.choice([None, (2.0, 1.0, 3.0, 24), (8.0, 0.5, 16.0, 100)]))
                owners.append(i)
        kind = rng.random()
        mlp = None if kind < 0.15 else dense(rng.choice([16, 40, 64]), rng.choice([0.5, 1.0, 4.0])) if kind < 0.5 \
            else moe(rng.choice([16, 24, 64]), *rng.choice([(1, 1), (4, 2), (5, 5), (9, 3), (16, 4)]),
                     limit=rng.choice([0.5, 1.0, 4.0]))
        layers.append(layer(mixer, mlp))
    cfg = {"architecture": "Tuzapel", "vocab": rng.choice([64, 130, 300]), "width": width,
           "norm": {"eps": rng.choice([1e-5, 1e-6])}, "layers": layers}
    if rng.random() < 0.6:
        cfg["logit_softcap"] = rng.choice([5.0, 30.0])
    return cfg
