"""Small Mirorax configurations for the tests (config.json dicts). Sizes are deliberately
unequal to one another (dim != vdim != rot_dim, kv_heads 1 / < heads / == heads, rotary dims
< rot_dim and == rot_dim), include values that are not multiples of the kernels' vector and
tile widths, windows short enough that prompts of a few dozen tokens cross their edge many
times, loops of one pass and of several, at the start, in the middle and over the whole stack."""


def attn(heads=4, kv_heads=2, dim=24, vdim=40, scale=0.21):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}


def latent(heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=32, size=9, scale=0.19, rot_dims=None, base=10000.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "mask": {"size": size},
            "scale": scale, "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}}


def dense(ff=72, limit=1.25):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=6, top=2, ff=40, shared=24):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def config(layers, width=96, vocab=211, eps=1e-5, loop=None):
    c = {"architecture": "Mirorax", "norm": {"eps": eps}, "vocab": vocab, "width": width,
         "layers": [{"type": t, "mixer": m, "mlp": f} for t, m, f in layers]}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


A, L = "attention", "latent_attention"

# one mechanism at a time (no feed-forward; no loop)
ONLY_ATTN = config([(A, attn(), None)])
ONLY_LATENT = config([(L, latent(), None)])
ONLY_DENSE = config([(A, attn(heads=1, kv_heads=1, dim=8, vdim=8), dense())])
ONLY_MOE = config([(A, attn(heads=1, kv_heads=1, dim=8, vdim=8), moe())])
# the loop alone: one layer walked three times; a loop of one pass (its vector still joins)
ONLY_LOOP = config([(A, attn(heads=2, kv_heads=1, dim=16, vdim=16), dense(ff=32))], loop=(0, 1, 3))
LOOP_ONCE = config([(L, latent(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=16, size=5), dense(ff=32)),
                    (A, attn(heads=2, kv_heads=2, dim=16, vdim=8), None)], loop=(0, 2, 1))
# everything, different sizes per layer, a layer without feed-forward, a loop in the middle,
# a window of 1 (a position sees itself and the sink only), rotary dims < rot_dim, top 1, no
# shared expert, kv_heads == heads and == 1
MIXED = config([
    (A, attn(), dense()),
    (L, latent(), moe()),
    (A, attn(heads=6, kv_heads=6, dim=16, vdim=16, scale=0.3), moe(experts=4, top=1, ff=24, shared=0)),
    (L, latent(heads=4, dim=16, rot_dim=16, vdim=24, kv_rank=24, size=1, scale=0.3, rot_dims=8, base=500.0), None),
    (L, latent(heads=2, dim=40, rot_dim=4, vdim=16, kv_rank=48, size=33, scale=0.15), dense(ff=56, limit=0.75)),
    (A, attn(heads=3, kv_heads=1, dim=32, vdim=24, scale=0.17), moe(experts=5, top=5, ff=16, shared=40)),
], loop=(1, 4, 2))
# sizes that defeat every vector path: odd width, odd head sizes, odd ranks and feed-forward sizes
ODD = config([
    (L, latent(heads=3, dim=7, rot_dim=6, vdim=9, kv_rank=11, size=5, scale=0.4), dense(ff=19)),
    (A, attn(heads=5, kv_heads=5, dim=10, vdim=3, scale=0.35), moe(experts=3, top=2, ff=7, shared=5)),
    (L, latent(heads=2, dim=5, rot_dim=2, vdim=11, kv_rank=13, size=13, scale=0.5), None),
    (A, attn(heads=2, kv_heads=1, dim=9, vdim=7, scale=0.5), dense(ff=13, limit=2.0)),
], width=50, vocab=37, eps=1e-4, loop=(2, 4, 2))
# wider sizes: several tiles per product, key rows of more than 64 entries, many heads, a window
# longer than a key tile and one longer than most prompts, the whole stack looped
WIDE = config([
    (L, latent(heads=8, dim=64, rot_dim=32, vdim=64, kv_rank=128, size=70, scale=0.1), dense(ff=320)),
    (A, attn(heads=8, kv_heads=2, dim=96, vdim=80, scale=0.1), moe(experts=8, top=3, ff=64, shared=96)),
    (L, latent(heads=12, dim=32, rot_dim=16, vdim=48, kv_rank=64, size=150, scale=0.15), moe(experts=16, top=4, ff=48, shared=0)),
    (A, attn(heads=2, kv_heads=2, dim=128, vdim=128, scale=0.09), dense(ff=200, limit=3.0)),
], width=256, vocab=1000, loop=(0, 4, 2))
# dense feed-forwards only: no router whose near-ties a rounding could flip (bf16 comparisons)
DENSE_ONLY = config([
    (L, latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, size=20, scale=0.15), dense(ff=128)),
    (A, attn(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.15), dense(ff=96)),
    (L, latent(heads=2, dim=48, rot_dim=8, vdim=64, kv_rank=40, size=64, scale=0.12), dense(ff=160, limit=2.5)),
], width=128, vocab=300, loop=(0, 2, 2))

ALL = {"only_attn": ONLY_ATTN, "only_latent": ONLY_LATENT, "only_dense": ONLY_DENSE, "only_moe": ONLY_MOE,
       "only_loop": ONLY_LOOP, "loop_once": LOOP_ONCE, "mixed": MIXED, "odd": ODD, "wide": WIDE, "dense_only": DENSE_ONLY}


def tokens(cfg, n, seed=0):
    import numpy as np

    return np.random.default_rng(2000 + seed).integers(0, cfg["vocab"], n).tolist()
