"""Small Zifunex configurations for the tests: every size differs between them
and from one another where it can (streams 1 to 4, one or several key/value
heads, values narrower than, as wide as and wider than the keys, a rotation of
part of a head and of all of it, scans of 8 to 40 states, convolutions of 2 to
5 taps, a loop that runs a stretch 1, 2 or 3 times, or no loop at all)."""


def attention(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, scale=0.25, softcap=20.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"dims": rot_dims, "base": base},
            "scale": scale, "softcap": softcap}


def scan(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def parallel(left, right, ff=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def gla(heads, dim, vdim, tau, rank, ff=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def zifunex(vocab, width, streams, layers, loop=None, eps=1e-5, buckets=211, mul_prev=31, mul_cur=5):
    config = {"architecture": "Zifunex", "vocab": vocab, "width": width, "streams": streams, "norm": {"eps": eps},
              "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "layers": layers}
    if loop is not None:
        config["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return config


# two streams; grouped heads 4:2 with values narrower than the keys and half a head rotated; a loop over the first two layers
ZIF_A = zifunex(
    vocab=300, width=96, streams=2,
    layers=[
        gla(heads=3, dim=16, vdim=24, tau=8.0, rank=8, ff=128),
        parallel(attention(4, 2, 32, 16, 16, base=10000.0, scale=0.2, softcap=10.0), scan(80, 12, 5, 3)),
        parallel(attention(2, 1, 16, 48, 16, base=500.0, scale=0.31, softcap=25.0), scan(64, 8, 8, 2), ff=160),
    ],
    loop=(0, 2, 2))
# one stream and no loop; values as wide as the keys; a scan whose states fill five lanes' worth; a layer that ends the model without a feed-forward
ZIF_B = zifunex(
    vocab=257, width=64, streams=1, eps=3e-6, buckets=97, mul_prev=1, mul_cur=1,
    layers=[
        parallel(attention(2, 2, 32, 32, 32, base=2000.0, scale=0.18, softcap=50.0), scan(48, 40, 3, 5), ff=96),
        gla(heads=2, dim=40, vdim=20, tau=1.0, rank=16),
    ])
# four streams; the looped stretch in the middle, three times; one key/value head for six query heads; key channels that fill no tile
ZIF_C = zifunex(
    vocab=512, width=128, streams=4, buckets=1009, mul_prev=7919, mul_cur=104729,
    layers=[
        parallel(attention(6, 1, 48, 64, 24, base=100000.0, scale=0.1443, softcap=15.0), scan(96, 16, 6, 4), ff=200),
        gla(heads=1, dim=64, vdim=128, tau=32.0, rank=24, ff=144),
        parallel(attention(2, 2, 64, 32, 64, base=10000.0, scale=0.13, softcap=28.0), scan(160, 20, 10, 4)),
        gla(heads=5, dim=24, vdim=40, tau=12.0, rank=8),
    ],
    loop=(1, 3, 3))

ZIFUNEX_CONFIGS = {"A": (ZIF_A, 21), "B": (ZIF_B, 22), "C": (ZIF_C, 23)}
