"""Small Mafalorn configurations for the tests: every size differs between
them where it can (retention with a rotation of all, of a part and of none of
a head's channels, decays from 0.5 to 1; softmax heads 2:1, 3:1 and 1:1 with
scaled and plain frequencies; delta-rule heads 2:1, 1:1 and 4:2 with 2 to 5
taps and values narrower and wider than the keys; latents narrower and wider
than a head, windows shorter and longer than a page and none; routers that
choose 1 to 3 of 3 to 12 outputs with 0 to 4 identity outputs in 1 to 4 groups
of which 1 to 3 are kept; layers without a feed-forward; every mixer first)."""


def rotation(dims, base, scaling=None):
    out = {"dims": dims, "base": base}
    if scaling:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def retention(heads, dim, vdim, decay, rot=None):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        out["rot"] = rotation(*rot)
    return out


def softmax(heads, kv_heads, dim, scale=0.2, rot=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot:
        out["rot"] = rotation(*rot)
    return out


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(left, right, left_scale=1.0, right_scale=1.0):
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale=0.2, base=1e4, window=None):
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
           "rot": {"dims": rot_dim, "base": base}}
    if window:
        out["mask"] = {"size": window}
    return out


def moe(experts, top, ff, identity=None, groups=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def mafalorn(vocab, width, layers, logit_scale=None, eps=1e-5):
    out = {"architecture": "Mafalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if logit_scale is not None:
        out["logit_scale"] = logit_scale
    return out


# side by side first (grouped softmax heads with scaled frequencies on a part of the head; delta heads 2:1 with values
# wider than the keys); a latent narrower than a page's window; retention with a part of the head turned
MAF_A = mafalorn(
    vocab=300, width=96, logit_scale=0.7,
    layers=[
        layer("parallel", parallel(softmax(4, 2, 32, scale=0.25, rot=(16, 5000.0, (4.0, 64, 8.0, 1.0))), delta(4, 2, 16, 24, 3), 0.6, 1.3),
              moe(6, 2, 24, identity=2, groups=(4, 2))),
        layer("retention", retention(3, 16, 32, (0.9, 0.97, 0.995), rot=(8, 1e4)), moe(5, 2, 16, identity=1, groups=(2, 1))),
        layer("latent_attention", latent(4, 16, 8, 24, 40, scale=0.3, window=37)),
        layer("retention", retention(2, 24, 8, (1.0, 0.5)), moe(3, 1, 40)),
    ])
# a latent first, its window longer than a page; one softmax head group; delta heads 1:1 with five taps and values
# narrower than the keys; a retention whose whole head is turned; no logit scale
MAF_B = mafalorn(
    vocab=257, width=64, eps=3e-6,
    layers=[
        layer("latent_attention", latent(3, 32, 16, 16, 48, scale=0.15, base=100.0, window=70), moe(3, 3, 24, identity=3, groups=(3, 3))),
        layer("parallel", parallel(softmax(3, 1, 16, scale=0.3), delta(2, 2, 32, 8, 5), 1.0, 0.25), None),
        layer("retention", retention(4, 16, 16, (0.75, 0.9, 0.99, 0.999), rot=(16, 50.0)), moe(12, 3, 8, identity=4, groups=(4, 3))),
    ])
# retention first; a latent without a window; softmax heads 1:1 whose whole head is turned with scaled frequencies; delta
# heads 4:2 with two taps; one group is no grouping; a router that keeps one of two groups
MAF_C = mafalorn(
    vocab=512, width=128, logit_scale=2.0,
    layers=[
        layer("retention", retention(2, 32, 48, (0.96, 0.6), rot=(32, 1e6)), moe(4, 2, 32, identity=0, groups=(1, 1))),
        layer("latent_attention", latent(2, 24, 8, 40, 24, scale=0.2, base=1e6), moe(7, 2, 16, identity=1, groups=(2, 1))),
        layer("parallel", parallel(softmax(2, 2, 64, scale=0.12, rot=(64, 2e4, (8.0, 32, 4.0, 0.5))), delta(4, 2, 16, 16, 2), 1.5, 0.8),
              moe(2, 1, 48, identity=2)),
        layer("parallel", parallel(softmax(6, 2, 16, scale=0.3, rot=(4, 1e3)), delta(1, 1, 48, 32, 4), 0.3, 1.0)),
    ])

MAFALORN_CONFIGS = {"A": (MAF_A, 61), "B": (MAF_B, 62), "C": (MAF_C, 63)}
