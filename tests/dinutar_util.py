"""Small Dinutar configurations and weights made for testing.

The configurations differ from each other in every size, in the order of their layers and in what the design
allows to be absent or equal (a layer without a feed-forward, a rotation that covers only part of a head, no
stretching of the rotation, a layer that reads another layer's cache, one head, a decay of exactly 1, sizes
that are no multiples of 16). Weights are drawn so that every path matters: norm weights and the per-channel
scales are far from one, the pair table is as large as the embedding.
"""
from __future__ import annotations

import math

import torch

from kanavik_util import Driver, row_error, write_folder  # noqa: F401  (the same driver of the package's step function)


def latent(heads, dim, rot_dim, vdim, rank, scale, base=10000.0, scaling=None, kv_from=None, ff=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def retention(heads, dim, vdim, decay, rot_dims, base=10000.0, scaling=None, ff=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": rot},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width, vocab, alpha, scale, buckets, mul_prev, mul_cur, eps=1e-5):
    return {"architecture": "Dinutar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
            "embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}},
            "layers": layers}


# sizes that are no multiples of 16 or 8, a stretched rotation, a retention layer whose rotation covers part of a
# head, a layer that reads the first layer's cache with other head counts and sizes, layers without feed-forward
CONFIG_ODD = config([latent(3, 24, 8, 40, 48, 0.3, base=100.0, scaling=(4.0, 24, 6.0, 0.5), ff=136),
                     retention(3, 40, 24, [0.9, 0.97, 0.996], 16, base=500.0),
                     latent(5, 12, 8, 20, 48, 0.4, base=100.0, scaling=(4.0, 24, 6.0, 0.5), kv_from=0, ff=64),
                     retention(2, 20, 36, [0.5, 0.99], 20, base=50.0, scaling=(2.0, 16, 4.0, 1.0), ff=72)],
                    width=96, vocab=211, alpha=1.5, scale=1.7, buckets=53, mul_prev=5, mul_cur=3)
# retention first, one head with a decay of exactly 1 and values in two column slices; two latent layers with
# caches of their own that differ in size (two cache groups) and two readers; no stretching; multipliers whose
# products pass 2^31 for large ids
CONFIG_WIDE = config([retention(1, 64, 128, [1.0], 64, base=1e6, ff=192),
                      latent(8, 32, 32, 64, 96, 0.11, base=1e4, ff=200),
                      latent(2, 64, 16, 16, 32, 0.2, base=300.0),
                      latent(12, 16, 32, 32, 96, 0.18, base=1e4, kv_from=1),
                      retention(4, 16, 16, [0.8, 0.9, 0.95, 0.999], 8, base=200.0),
                      latent(1, 48, 16, 80, 32, 0.15, base=300.0, kv_from=2, ff=96)],
                     width=128, vocab=300, alpha=1.0, scale=1.0, buckets=4093, mul_prev=1000003, mul_cur=999983, eps=1e-6)
# one latent layer and nothing else; a multiplier of zero (the pair row depends on the token alone)
CONFIG_ONE = config([latent(2, 16, 16, 32, 16, 0.25, base=20.0, scaling=(8.0, 8, 2.0, 1.0))],
                    width=48, vocab=97, alpha=2.5, scale=0.3, buckets=7, mul_prev=0, mul_cur=11)

# a latent too large for the one-head kernel of one-token sequences (latent + rotated part over 256 elements): every
# sequence then goes the prompt portions' way; read by a second layer
CONFIG_DEEP = config([latent(2, 16, 16, 24, 272, 0.2, base=1000.0, ff=80),
                      retention(2, 16, 16, [0.9, 0.99], 16),
                      latent(3, 8, 16, 16, 272, 0.3, base=1000.0, kv_from=0)],
                     width=64, vocab=120, alpha=1.2, scale=0.9, buckets=31, mul_prev=3, mul_cur=5)

CONFIGS = {"odd": CONFIG_ODD, "wide": CONFIG_WIDE, "one": CONFIG_ONE, "deep": CONFIG_DEEP}


def tensor_shapes(c):
    C = c["width"]
    shapes = {"embed": (c["vocab"], C), "bigram": (c["embedding"]["bigram"]["buckets"] + 1, C), "embed.norm": (C,),
              "final.norm": (C,)}
    for i, lay in enumerate(c["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        H, D, E = m["heads"], m["dim"], m["vdim"]
        shapes.update({p + "norm1": (C,), p + "ls1": (C,), p + "mix.o": (C, H * E)})
        if lay["type"] == "latent_attention":
            R, L = m["rot_dim"], m["kv_rank"]
            shapes.update({p + "mix.q": (H * (D + R), C), p + "mix.uk": (H * D, L), p + "mix.uv": (H * E, L)})
            if "kv_from" not in m:
                shapes.update({p + "mix.dkv": (L + R, C), p + "mix.dkv.norm": (L,)})
        else:
            shapes.update({p + "mix.q": (H * D, C), p + "mix.k": (H * D, C), p + "mix.v": (H * E, C), p + "mix.g": (H * E, C)})
        if lay["mlp"]:
            F = lay["mlp"]["ff"]
            shapes.update({p + "norm2": (C,), p + "ls2": (C,), p + "mlp.up": (F, C), p + "mlp.down": (C, F)})
    return shapes


def make_weights(c, seed, sharp=1.0):
    """{name: bfloat16 tensor}: what a checkpoint of configuration C holds. SHARP multiplies every query matrix: above
    one, a softmax concentrates on its best key, wherever that lies."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(c).items():
        leaf = name.split(".")[-1]
        normal = torch.randn(shape, generator=g)
        if name in ("embed", "bigram"):
            t = normal
        elif leaf in ("norm1", "norm2", "norm"):
            t = 1.0 + 0.3 * normal
        elif leaf in ("ls1", "ls2"):
            t = 0.8 + 0.5 * normal
        else:                                             # linear maps [out, in]
            t = normal / math.sqrt(shape[-1])
            if leaf == "q":
                t = t * sharp
        out[name] = t.to(torch.bfloat16)
    return out
