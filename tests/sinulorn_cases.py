"""Small Sinulorn configurations for the tests (config.json dicts) and helpers that build
random checkpoints for them. Sizes are deliberately unequal to one another (dim != vdim,
kv_rank != dim, recurrence width != model width, ...) and include values that are not
multiples of the kernels' vector and tile widths."""
import numpy as np


def moe(ff=24, limit=1.5, experts=8, top=2, groups=4, keep=2, scale=1.75, shared=(40, 0.75)):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def dense(ff=72):
    return {"kind": "dense", "ff": ff}


def latent(heads=3, dim=16, vdim=24, kv_rank=40, q_rank=56, scale=0.3, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def rglru(width=80, blocks=5, conv=3):
    return {"width": width, "blocks": blocks, "conv": conv}


def delta(heads=4, kv_heads=2, dim=24, vdim=40, conv=4):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def config(layers, width=96, vocab=211, scale=7.0, eps=1e-5):
    return {"architecture": "Sinulorn", "embedding": {"scale": scale}, "norm": {"eps": eps}, "vocab": vocab,
            "width": width, "layers": [{"type": t, "mixer": m, "mlp": f} for t, m, f in layers]}


# one mechanism at a time
ONLY_LATENT = config([("latent_attention", latent(), None)])
ONLY_RGLRU = config([("rglru", rglru(), None)])
ONLY_DELTA = config([("delta", delta(), None)])
ONLY_DENSE = config([("rglru", rglru(width=32, blocks=1, conv=1), dense())])
ONLY_MOE = config([("rglru", rglru(width=32, blocks=2, conv=2), moe())])
# every branch in one stack: shared latent cache, a layer without feed-forward, experts with
# and without a shared expert, one group / every group kept, top 1, kv_heads == heads
MIXED = config([
    ("delta", delta(), dense()),
    ("latent_attention", latent(), moe()),
    ("rglru", rglru(), None),
    ("latent_attention", latent(heads=2, dim=24, vdim=16, q_rank=32, scale=0.2, kv_from=1), dense(ff=40)),
    ("delta", delta(heads=2, kv_heads=2, dim=40, vdim=24, conv=2), moe(ff=16, experts=6, top=1, groups=1, keep=1, shared=None)),
    ("rglru", rglru(width=64, blocks=1, conv=4), moe(ff=32, experts=6, top=3, groups=3, keep=3, scale=0.5)),
], width=96, vocab=211)
# the same mixers with dense feed-forwards only (no routing decisions to flip under bf16)
MIXED_DENSE = config([(t, m, dense(ff=56) if f else None) for t, m, f in
                      [(l["type"], l["mixer"], l["mlp"]) for l in MIXED["layers"]]], width=96, vocab=211)
# sizes that defeat every vector path: odd width, odd ranks and feed-forward sizes
ODD = config([
    ("latent_attention", latent(heads=2, dim=7, vdim=9, kv_rank=13, q_rank=11, scale=0.4), dense(ff=19)),
    ("delta", delta(heads=3, kv_heads=1, dim=9, vdim=5, conv=3), moe(ff=7, experts=4, top=2, groups=2, keep=1, shared=(5, 1.0))),
    ("rglru", rglru(width=15, blocks=3, conv=2), dense(ff=10)),
], width=50, vocab=37, scale=3.0, eps=1e-4)
# wider sizes: several tiles per GEMM, a latent rank above 64, a key dim above 64
WIDE = config([
    ("latent_attention", latent(heads=4, dim=32, vdim=32, kv_rank=96, q_rank=64, scale=0.18), dense(ff=320)),
    ("delta", delta(heads=2, kv_heads=1, dim=72, vdim=64, conv=4), None),
    ("rglru", rglru(width=192, blocks=3, conv=4), moe(ff=48, experts=16, top=4, groups=4, keep=2)),
], width=160, vocab=300)


# sizes that are multiples of the large-tile GEMM's tiles (N % 128, K % 64): long portions of
# this model run their plain products there when the whole library is loaded
TILED = config([
    ("rglru", rglru(width=256, blocks=4, conv=4), dense(ff=512)),
    ("latent_attention", latent(heads=2, dim=64, vdim=64, kv_rank=64, q_rank=128, scale=0.11), dense(ff=384)),
    ("delta", delta(heads=2, kv_heads=1, dim=64, vdim=64, conv=3), None),
], width=256, vocab=384)


# one routed layer whose shared expert's gated pair is tile-aligned (the routed experts' row
# lists stay on the general kernel); last layer, so a flipped routing tie touches one position
TILED_MOE = config([("rglru", rglru(width=128, blocks=2, conv=2), moe(ff=64, limit=1.25, experts=8, top=2, groups=2,
                                                                     keep=2, shared=(128, 0.9)))], width=256, vocab=256)


def tokens(cfg, n, seed=0):
    return np.random.default_rng(1000 + seed).integers(0, cfg["vocab"], n).tolist()
