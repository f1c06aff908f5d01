"""Small Gimozen configurations for the tests: sizes that differ from each other in every way the design allows."""

import math


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, coef=0.25, every=8, ff=48, scale=None):
    return {"type": "attention", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or 1.0 / math.sqrt(dim),
                      "q_temp": {"coef": coef, "every": every}}}


def latent_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, ff=48, kv_from=None, rot_dims=None, scaling="yarn", base=10000.0, scale=None):
    rot = {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}
    if scaling == "yarn":
        rot["scaling"] = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot,
             "scale": scale or 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mlp": None if ff is None else {"kind": "dense", "ff": ff}, "mixer": mixer}


def model(layers, width=64, vocab=97, scale=4.0, alpha=1.5, eps=1e-5):
    return {"architecture": "Gimozen", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps}, "postln_alpha": alpha,
            "vocab": vocab, "width": width}


CASES = {
    # a latent layer first, borrowed twice; grouped heads; value heads wider than key heads
    "mixed": model([latent_layer(), attention_layer(), latent_layer(kv_from=0), attention_layer(dim=16, vdim=32, kv_heads=1, ff=None),
                    latent_layer(kv_from=0, ff=None)]),
    # attention only: heads of 24 (no power of two), one head a group, a temperature that changes at every position
    "attention": model([attention_layer(heads=3, kv_heads=3, dim=24, vdim=24, every=1, coef=0.5), attention_layer(heads=2, kv_heads=1, dim=32, vdim=8)],
                       width=48, vocab=61, alpha=1.0, scale=1.0),
    # latent only: one head; rotation of a part of the rotated elements, without scaling; an odd latent; two latents of different sizes
    "latent": model([latent_layer(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=21, rot_dims=8, scaling=None),
                     latent_layer(heads=5, dim=24, rot_dim=4, vdim=16, kv_rank=64, base=500.0),
                     latent_layer(heads=2, dim=24, rot_dim=4, vdim=40, kv_rank=64, base=500.0, kv_from=1)], width=80, vocab=130, alpha=2.0),
    # sizes that are no multiples of anything a kernel would like: rows of 200 bytes, heads of 20 and 12, a latent of 30 + 6
    "odd": model([attention_layer(heads=5, kv_heads=1, dim=20, vdim=12, ff=90, every=3),
                  latent_layer(heads=5, dim=20, rot_dim=6, vdim=12, kv_rank=30, ff=None, base=777.0),
                  latent_layer(heads=7, dim=12, rot_dim=6, vdim=20, kv_rank=30, ff=90, base=777.0, kv_from=1)], width=100, vocab=77, alpha=0.7, eps=1e-6),
}
