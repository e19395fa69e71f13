"""Small Robopel configurations for the tests: every size differs between them
where it can (grouped heads 2:1, 3:1 and 1:1; values narrower and wider than
the keys; a rotation of all and of a part of a head's channels, bent and not;
windows shorter and longer than a page with pooled blocks of 1 to 24 tokens;
layers that read an earlier layer's keys and values with the same pooled
blocks, with others, and with none; routers that choose 1 to 3 of 3 to 9
experts with 0 to 2 identity outputs; layers without a feed-forward; either
mixer first)."""


def attention(heads, kv_heads, dim, vdim, scale=0.25, softcap=None, rot=None, window=None, pool=None, kv_from=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        out["softcap"] = softcap
    if rot:
        out["rot"] = {"dims": rot[0], "base": rot[1]}
        if len(rot) > 2:
            out["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), rot[2]))
    if window:
        out["mask"] = {"size": window}
        if pool:
            out["mask"]["pool"] = pool
    if kv_from is not None:
        out["kv_from"] = kv_from
    return out


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def robopel(vocab, width, layers, scale=None, eps=1e-5):
    out = {"architecture": "Robopel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if scale is not None:
        out["embedding"] = {"scale": scale}
    return out


# attention first; the third layer reads the first's keys and values and its pooled blocks; a bent rotation of the whole head
ROB_A = robopel(
    vocab=300, width=96, scale=9.0,
    layers=[
        layer("attention", attention(4, 2, 32, 16, scale=0.2, softcap=15.0, rot=(32, 5000.0, (4.0, 1.0, 2.0, 64)), window=37, pool=8), dense(136)),
        layer("mingru", {"width": 72}, moe(5, 2, 24, identity=1)),
        layer("attention", attention(4, 2, 32, 16, scale=0.3, softcap=25.0, rot=(32, 5000.0, (4.0, 1.0, 2.0, 64)), window=37, pool=8, kv_from=0)),
        layer("mingru", {"width": 96}, dense(64)),
    ])
# a minGRU first; one key/value head; a rotation of a part of the head, not bent; a window longer than a page with blocks of 24;
# the layer that reads layer 1's keys has a shorter window and smaller blocks of its own; a router without identity outputs
ROB_B = robopel(
    vocab=257, width=64, eps=3e-6,
    layers=[
        layer("mingru", {"width": 40}),
        layer("attention", attention(3, 1, 16, 48, scale=0.31, softcap=30.0, rot=(8, 100.0), window=70, pool=24), moe(3, 1, 40)),
        layer("attention", attention(3, 1, 16, 48, scale=0.2, rot=(8, 100.0), window=20, pool=5, kv_from=1), dense(80)),
    ])
# heads 1:1; no cap; no rotation in one layer; pooled blocks of one token (every key outside the window stays, as itself);
# a window without pooled blocks reading keys that come with them; full attention; two identity outputs and three chosen
ROB_C = robopel(
    vocab=512, width=128, scale=1.0,
    layers=[
        layer("attention", attention(2, 2, 32, 16, scale=0.18, window=9, pool=1), moe(9, 3, 16, identity=2)),
        layer("attention", attention(2, 2, 32, 16, scale=0.25, softcap=10.0, window=64, kv_from=0), dense(72)),
        layer("mingru", {"width": 136}, moe(4, 2, 32, identity=0)),
        layer("attention", attention(6, 2, 24, 40, scale=0.2, softcap=40.0, rot=(24, 1e4, (8.0, 1.0, 4.0, 32))), dense(48)),
        layer("attention", attention(6, 2, 24, 40, scale=0.2, softcap=40.0, rot=(16, 1e4), window=33, pool=16, kv_from=3)),
    ])

ROBOPEL_CONFIGS = {"A": (ROB_A, 51), "B": (ROB_B, 52), "C": (ROB_C, 53)}
