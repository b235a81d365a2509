"""Small Lenuzen configurations for the tests (config.json dicts). Sizes are deliberately
unequal to one another (dim != vdim, rotary dims < dim and == dim, kv_heads 1 / < heads /
== heads), include values that are not multiples of the kernels' vector and tile widths,
and windows / chunks short enough that prompts of a few dozen tokens cross several edges."""
import numpy as np


def rot(dims, base=10000.0, factor=2.0, original=64, fast=8.0, slow=2.0):
    r = {"dims": dims, "base": base}
    if factor:
        r["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return r


def window(heads=4, kv_heads=2, dim=24, vdim=40, size=9, scale=0.21, rot_dims=16, **kw):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "scale": scale,
            "rot": rot(rot_dims, **kw)}


def chunk(heads=3, kv_heads=1, dim=32, vdim=16, size=7, scale=0.17, rot_dims=32, **kw):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "scale": scale,
            "rot": rot(rot_dims, **kw)}


def dense(ff=72):
    return {"kind": "dense", "ff": ff}


def config(layers, width=96, vocab=211, scale=5.0, eps=1e-5, logit_scale=0.75):
    return {"architecture": "Lenuzen", "embedding": {"scale": scale}, "norm": {"eps": eps}, "vocab": vocab,
            "width": width, "logit_scale": logit_scale,
            "layers": [{"type": t, "mixer": m, "mlp": f} for t, m, f in layers]}


# one mechanism at a time
ONLY_WINDOW = config([("attention", window(), None)])
ONLY_CHUNK = config([("attention_2", chunk(), None)])
ONLY_DENSE = config([("attention", window(heads=1, kv_heads=1, dim=8, vdim=8, size=3, rot_dims=4), dense())])
# both mixers, different sizes per layer, a layer without feed-forward, kv_heads == heads,
# a window of 1 (a position sees itself only), a chunk of 1, no rotary rescaling, rot dims 0 < dims < dim
MIXED = config([
    ("attention_2", chunk(), dense()),
    ("attention", window(), dense(ff=40)),
    ("attention_2", chunk(heads=4, kv_heads=4, dim=16, vdim=24, size=12, rot_dims=8, factor=0), None),
    ("attention", window(heads=2, kv_heads=1, dim=40, vdim=24, size=1, scale=0.3, rot_dims=40, base=500.0), dense(ff=56)),
    ("attention_2", chunk(heads=2, kv_heads=2, dim=24, vdim=24, size=1, rot_dims=2), dense(ff=24)),
    ("attention", window(heads=6, kv_heads=3, dim=16, vdim=16, size=33, rot_dims=16, factor=8.0, original=16), dense(ff=88)),
], width=96, vocab=211)
# sizes that defeat every vector path: odd width, odd head sizes, odd feed-forward sizes
ODD = config([
    ("attention", window(heads=3, kv_heads=1, dim=7, vdim=9, size=5, rot_dims=6, scale=0.4), dense(ff=19)),
    ("attention_2", chunk(heads=5, kv_heads=5, dim=10, vdim=3, size=4, rot_dims=10, scale=0.35), dense(ff=7)),
    ("attention_2", chunk(heads=2, kv_heads=1, dim=6, vdim=11, size=13, rot_dims=2, scale=0.5), None),
], width=50, vocab=37, scale=3.0, eps=1e-4, logit_scale=1.5)
# wider sizes: several tiles per product, heads of more than 64 entries, many heads, windows
# and chunks longer than a key tile
WIDE = config([
    ("attention", window(heads=8, kv_heads=2, dim=96, vdim=80, size=70, rot_dims=64, scale=0.1, original=128), dense(ff=320)),
    ("attention_2", chunk(heads=12, kv_heads=4, dim=32, vdim=48, size=100, rot_dims=16, scale=0.18), dense(ff=200)),
    ("attention", window(heads=2, kv_heads=2, dim=128, vdim=128, size=150, rot_dims=128, scale=0.09), None),
], width=160, vocab=300)
# sizes that are multiples of the large-tile GEMM's tiles (N % 128, K % 64), and of the MFMA
# attention's (heads of 64 and 128)
TILED = config([
    ("attention", window(heads=4, kv_heads=2, dim=64, vdim=64, size=192, rot_dims=48, scale=0.11, original=256), dense(ff=512)),
    ("attention_2", chunk(heads=4, kv_heads=1, dim=128, vdim=64, size=160, rot_dims=64, scale=0.09, original=256), dense(ff=384)),
], width=256, vocab=384)


def tokens(cfg, n, seed=0):
    return np.random.default_rng(1000 + seed).integers(0, cfg["vocab"], n).tolist()
