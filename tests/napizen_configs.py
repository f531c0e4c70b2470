"""Small Napizen configurations of the tests' own, differing from each other in every size, constant and layer order."""

from __future__ import annotations

from tests.nobodra_configs import write_folder  # noqa: F401  (folders are written the same way)


def latent(heads, dim, rot_dim, vdim, rank, scale, base, scaling=None, mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def experts(ff, count, top, scale, groups=None):
    router = {"experts": count, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def model(vocab, width, eps, alpha, layers, embedding=1.0, cap=None):
    raw = {"architecture": "Napizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha, "embedding": {"scale": embedding},
           "layers": layers}
    if cap is not None:
        raw["logit_softcap"] = cap
    return raw


# groups of three experts of which two groups are kept, a layer without feed-forward in the middle, stretched rotations
# whose blend begins and ends inside the pairs, three heads, all five sizes of a head different
MIXED = model(211, 64, 1e-5, 1.7, [
    latent(3, 16, 8, 24, 40, 0.2, 10000.0, (8.0, 64, 16.0, 2.0), dense(96)),
    latent(2, 24, 4, 8, 20, 0.31, 500.0, None, experts(32, 6, 2, 1.5, (2, 1))),
    latent(4, 8, 12, 16, 32, 0.25, 2e5, (5.0, 256, 20.0, 1.0), None),
    latent(3, 16, 8, 24, 40, 0.2, 10000.0, (8.0, 64, 16.0, 2.0), experts(24, 9, 3, 2.5, (3, 2))),
], embedding=6.0, cap=9.0)
# values that coincide or are 1: one head, groups of one expert, every group kept, one choice, alpha 1, no cap, a rotated part
# of one pair, dim = vdim = rank, every expert chosen, more experts than a wave has lanes
PLAIN = model(157, 48, 3e-6, 1.0, [
    latent(1, 16, 2, 16, 16, 0.4, 100.0, None, experts(16, 4, 1, 1.0, (4, 4))),
    latent(2, 8, 8, 8, 8, 0.3, 2000.0, (2.0, 32, 4.0, 1.0), experts(8, 3, 3, 1.0)),
    latent(1, 4, 6, 30, 12, 1.0, 30.0, None, experts(8, 70, 2, 0.5, (70, 5))),
    latent(5, 8, 2, 4, 24, 0.2, 1e4, None, dense(40)),
])
# sizes the matrix-core kernels take: rows of 128 and 160 kept values, heads of 64 and 128, eight and sixteen heads
CORES = model(300, 128, 1e-6, 2.0, [
    latent(8, 64, 32, 64, 96, 0.1, 3e5, (6.0, 128, 24.0, 1.5), dense(256)),
    latent(16, 32, 16, 32, 64, 0.14, 1e4, None, experts(64, 8, 3, 1.5, (4, 2))),
    latent(4, 128, 32, 128, 128, 0.08, 1e5, (16.0, 64, 8.0, 2.0), experts(128, 4, 4, 1.0)),
], embedding=11.0, cap=25.0)
# wide enough that prompts go through the products for many rows
WIDE = model(1000, 512, 1e-6, 3.0, [
    latent(8, 64, 32, 64, 128, 0.1, 5e5, (3.0, 512, 28.0, 1.0), experts(256, 8, 2, 1.25, (4, 2))),
    latent(8, 64, 64, 128, 192, 0.09, 1e4, None, dense(1024)),
], embedding=22.0, cap=28.0)
