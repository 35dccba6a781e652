"""Small Mutedra configurations for the tests: every size differs between them
and from one another where it can (grouped heads 2:1, 3:1 and 1:1; values
narrower and wider than the keys; windows shorter and longer than a page, with
and without kept first tokens; latents of 24 to 64 channels, some no multiple
of 16; a rotated part as wide as, narrower and wider than the plain part; an
embedding scale of 1; layers without a feed-forward; a loop from the first
layer, from a later one, and one that runs once)."""


def windowed(heads, kv_heads, dim, vdim, window, keep_first, bias_max, buckets, scale=0.25):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max,
            "bias_buckets": buckets, "mask": {"size": window, "keep_first": keep_first}}


def latent(heads, dim, vdim, q_rank, kv_rank, scale=0.25, rot_dim=None, base=10000.0):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if rot_dim:
        out.update(rot_dim=rot_dim, rot={"dims": rot_dim, "base": base})
    return out


def layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def mutedra(vocab, width, layers, loop, scale=1.0, softcap=30.0, eps=1e-5):
    return {"architecture": "Mutedra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "logit_softcap": softcap, "layers": layers, "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


# a loop over the last two layers, three times (the first layer runs once, before any pass begins)
MUT_A = mutedra(
    vocab=300, width=96, scale=3.0, softcap=12.0,
    layers=[
        layer("latent_attention_2", latent(3, 16, 24, 40, 32, scale=0.2, rot_dim=16, base=1000.0), ff=128),
        layer("attention", windowed(4, 2, 32, 16, window=37, keep_first=5, bias_max=50, buckets=12, scale=0.2)),
        layer("latent_attention", latent(2, 24, 8, 16, 48, scale=0.3), ff=160),
    ],
    loop=(1, 3, 3))
# an embedding scale of 1, no kept first tokens, a window longer than a page, a loop that runs once
MUT_B = mutedra(
    vocab=257, width=64, scale=1.0, softcap=50.0, eps=3e-6,
    layers=[
        layer("attention", windowed(3, 1, 16, 48, window=70, keep_first=0, bias_max=90, buckets=8, scale=0.31), ff=96),
        layer("latent_attention_2", latent(2, 32, 32, 24, 64, scale=0.15, rot_dim=32, base=50000.0)),
    ],
    loop=(0, 2, 1))
# the loop from the first layer on, twice; latents that fill no tile of the matrix cores; a window of a few tokens and one of a page
MUT_C = mutedra(
    vocab=512, width=128, scale=7.5, softcap=20.0,
    layers=[
        layer("attention", windowed(6, 6, 32, 16, window=8, keep_first=3, bias_max=20, buckets=6, scale=0.18), ff=200),
        layer("latent_attention", latent(5, 8, 40, 48, 40, scale=0.35), ff=144),
        layer("latent_attention_2", latent(4, 24, 16, 32, 24, scale=0.25, rot_dim=8, base=100.0)),
        layer("attention", windowed(2, 1, 16, 48, window=64, keep_first=64, bias_max=33, buckets=10, scale=0.3), ff=64),
    ],
    loop=(0, 2, 2))

MUTEDRA_CONFIGS = {"A": (MUT_A, 31), "B": (MUT_B, 32), "C": (MUT_C, 33)}
