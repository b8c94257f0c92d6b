"""Small Lifenex configurations for the tests (config.json dicts, plus the three sizes the design
leaves to the tensors' shapes). Sizes are deliberately unequal to one another (dim != vdim, state
!= vdim, kv_heads 1 / < heads / == heads on both sides of a pair, groups != norm_groups, taps 1..4),
include values that are not multiples of the kernels' vector and tile widths, temperature blocks
and distance tables short enough that prompts of a few dozen tokens cross their edges many times,
routers with one group, with groups of one expert, top 1 and top = experts."""


def ssm(heads=3, vdim=16, state=24, groups=1, norm_groups=3, conv=4):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def attn(heads=4, kv_heads=2, dim=24, vdim=40, scale=0.21, bias_max=60, coef=0.4, every=16):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max,
            "q_temp": {"coef": coef, "every": every}}


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def pair(left=None, right=None):
    return {"left": left or attn(), "right": right or delta()}


def dense(ff=72):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=40, shared=24, count=3, keep=2):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top,
                                                          "groups": {"count": count, "keep": keep}}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def config(layers, width=96, vocab=211, eps=1e-5, logit_scale=0.5, sizes=None):
    """sizes: rel_rows / decay_rank / gate_rank of the model's tensors (not part of config.json)."""
    c = {"architecture": "Lifenex", "norm": {"eps": eps}, "vocab": vocab, "width": width, "logit_scale": logit_scale,
         "layers": [{"type": t, "mixer": m, "mlp": f} for t, m, f in layers]}
    SIZES[id(c)] = dict({"rel_rows": 12, "decay_rank": 10, "gate_rank": 6}, **(sizes or {}))
    return c


SIZES = {}  # id(config) -> the tensor sizes it was made with


def sizes(cfg):
    return SIZES.get(id(cfg), {"rel_rows": 12, "decay_rank": 10, "gate_rank": 6})


S, P = "mamba2", "parallel"
TINY = ssm(heads=1, vdim=8, state=8, norm_groups=1, conv=2)

# one mechanism at a time
ONLY_SSM = config([(S, ssm(), None)])
ONLY_PAIR = config([(P, pair(), None)])
ONLY_DENSE = config([(S, TINY, dense())])
ONLY_MOE = config([(S, TINY, moe())])
# everything, different sizes per layer: groups == heads and 1, norm_groups 1 and == heads, a layer
# without feed-forward, kv_heads == heads and == 1 on either side, a temperature block of one
# position and one longer than the prompts, a distance table that saturates after a few tokens and
# one that never does, one router group, groups of one expert, top 1, top == experts, no shared expert
MIXED = config([
    (S, ssm(), dense()),
    (P, pair(), moe()),
    (P, pair(attn(heads=6, kv_heads=6, dim=16, vdim=16, scale=0.3, bias_max=9, every=1),
             delta(heads=2, kv_heads=2, dim=24, vdim=8, conv=4)), moe(experts=4, top=1, ff=24, shared=0, count=1, keep=1)),
    (S, ssm(heads=4, vdim=8, state=16, groups=4, norm_groups=1, conv=3), None),
    (P, pair(attn(heads=3, kv_heads=1, dim=32, vdim=24, scale=0.17, bias_max=500, every=1000),
             delta(heads=6, kv_heads=1, dim=8, vdim=16, conv=2)), moe(experts=5, top=5, ff=16, shared=40, count=5, keep=5)),
    (S, ssm(heads=2, vdim=24, state=40, groups=2, norm_groups=2, conv=1), moe(experts=8, top=3, ff=16, shared=8, count=4, keep=2)),
], sizes={"rel_rows": 8, "decay_rank": 5, "gate_rank": 12})
# sizes that defeat every vector path: odd width, odd head sizes, odd ranks and feed-forward sizes
ODD = config([
    (S, ssm(heads=3, vdim=7, state=9, groups=3, norm_groups=1, conv=3), dense(ff=19)),
    (P, pair(attn(heads=5, kv_heads=5, dim=10, vdim=3, scale=0.35, bias_max=21, every=7),
             delta(heads=3, kv_heads=1, dim=5, vdim=11, conv=4)), moe(experts=3, top=2, ff=7, shared=5, count=1, keep=1)),
    (P, pair(attn(heads=2, kv_heads=1, dim=9, vdim=7, scale=0.5, bias_max=33, every=5),
             delta(heads=2, kv_heads=2, dim=7, vdim=5, conv=1)), None),
    (S, ssm(heads=1, vdim=13, state=11, groups=1, norm_groups=1, conv=2), moe(experts=6, top=2, ff=9, shared=0, count=2, keep=1)),
], width=50, vocab=37, eps=1e-4, logit_scale=1.7, sizes={"rel_rows": 7, "decay_rank": 3, "gate_rank": 1})
# wider sizes: several tiles per product, key rows and states of more than 64 entries, many heads
WIDE = config([
    (S, ssm(heads=8, vdim=64, state=128, groups=2, norm_groups=4, conv=4), dense(ff=320)),
    (P, pair(attn(heads=8, kv_heads=2, dim=96, vdim=80, scale=0.1, bias_max=100, every=64),
             delta(heads=4, kv_heads=2, dim=128, vdim=64, conv=4)), moe(experts=8, top=3, ff=64, shared=96, count=4, keep=2)),
    (P, pair(attn(heads=12, kv_heads=4, dim=32, vdim=48, scale=0.15, bias_max=300, every=50),
             delta(heads=8, kv_heads=8, dim=64, vdim=32, conv=2)), moe(experts=16, top=4, ff=48, shared=0, count=4, keep=3)),
    (S, ssm(heads=4, vdim=96, state=64, groups=1, norm_groups=1, conv=3), dense(ff=200)),
], width=256, vocab=1000, logit_scale=0.3, sizes={"rel_rows": 32, "decay_rank": 16, "gate_rank": 24})
# dense feed-forwards only: no router whose near-ties a rounding could flip (bf16 comparisons)
DENSE_ONLY = config([
    (S, ssm(heads=4, vdim=32, state=32, groups=2, norm_groups=4, conv=4), dense(ff=128)),
    (P, pair(attn(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.15, bias_max=80, every=32),
             delta(heads=4, kv_heads=2, dim=32, vdim=16, conv=3)), dense(ff=96)),
    (P, pair(attn(heads=2, kv_heads=1, dim=48, vdim=64, scale=0.12, bias_max=200, every=100),
             delta(heads=2, kv_heads=1, dim=64, vdim=48, conv=4)), dense(ff=160)),
], width=128, vocab=300, sizes={"rel_rows": 16, "decay_rank": 8, "gate_rank": 8})

ALL = {"only_ssm": ONLY_SSM, "only_pair": ONLY_PAIR, "only_dense": ONLY_DENSE, "only_moe": ONLY_MOE, "mixed": MIXED,
       "odd": ODD, "wide": WIDE, "dense_only": DENSE_ONLY}


def tokens(cfg, n, seed=0):
    import numpy as np

    return np.random.default_rng(3000 + seed).integers(0, cfg["vocab"], n).tolist()
