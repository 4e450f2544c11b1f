"""Tiny Kikunex configurations for the tests.  They differ in every size and option: the order of the
two kinds of mixer, heads, the head sizes and the latents' sizes (equal to each other or not, multiples
of four or not), the rotary base, windows that differ between layers (or none), decays near 1 and near
0, dense, routed and absent feed-forwards, experts in groups or not, one expert chosen or several, the
logits' scale, and where the repeated stretch of layers lies (from the first layer, in the middle,
nowhere)."""


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window, base=10000.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": {"base": base, "dims": rot_dim}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=None, keep=None, scale=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups, "keep": keep}
    if scale is not None:
        router["scale"] = scale
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


# the whole stack runs three times; attention first; windows of 24 and 40; three groups of which two are kept
K_A = {
    "architecture": "Kikunex", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
    "layers": [
        layer(latent(2, 16, 8, 24, 32, 20, 0.2, 24), dense(96)),
        layer(lightning(2, 16, 24, (0.9, 0.99)), moe(48, 6, 2, groups=3, keep=2, scale=1.5)),
        layer(latent(2, 16, 8, 24, 32, 20, 0.2, 40), moe(32, 4, 4, scale=0.7)),
    ],
    "loop": {"start": 0, "stop": 3, "times": 3},
}

# nothing divides by four; the loop lies in the middle; one layer has no feed-forward, one attention layer no
# window; one expert of five; a head that never forgets and one that forgets at once; no scale on the logits
K_B = {
    "architecture": "Kikunex", "vocab": 131, "width": 50, "norm": {"eps": 3e-6},
    "layers": [
        layer(lightning(3, 7, 9, (1.0, 0.5, 0.02)), dense(70)),
        layer(latent(3, 7, 10, 9, 21, 13, 0.31, 17, base=500.0), None),
        layer(lightning(1, 14, 11, (0.97,)), moe(30, 5, 1)),
        layer(latent(1, 14, 6, 11, 13, 30, 0.25, None, base=77.0), moe(22, 6, 3, groups=2, keep=1, scale=2.5)),
        layer(lightning(5, 6, 5, (0.8, 0.85, 0.9, 0.95, 0.999)), dense(33)),
    ],
    "loop": {"start": 1, "stop": 4, "times": 2},
}

# no loop; sizes that the matrix-core kernels take; a long window and a short one
K_C = {
    "architecture": "Kikunex", "vocab": 384, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
    "layers": [
        layer(latent(4, 32, 16, 32, 48, 64, 0.15, 100, base=100000.0), moe(128, 8, 2, groups=4, keep=2, scale=1.0)),
        layer(lightning(4, 32, 32, (0.7, 0.9, 0.97, 0.995)), dense(256)),
        layer(latent(8, 16, 16, 16, 64, 32, 0.18, 20, base=100000.0), dense(256)),
        layer(lightning(2, 64, 64, (0.95, 0.999)), moe(64, 16, 4, groups=8, keep=3, scale=0.5)),
    ],
}

ALL = {"A": (K_A, 4, 11), "B": (K_B, 8, 12), "C": (K_C, 16, 13)}
STD = 0.05      # spread of the random weights: every branch moves the logits, and no router call is so close that bfloat16 flips it


def random_configuration(seed):
    """A configuration drawn at random: every size, the layers' order and kinds, the windows, the decays,
    the routers' groups and the place of the repeated stretch."""
    import random
    rng = random.Random(seed)
    width = rng.choice([24, 40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        if rng.random() < 0.5:
            heads = rng.choice([1, 2, 3, 4, 6, 8])
            dim = rng.choice([0, 4, 8, 12, 16, 32])
            rot_dim = rng.choice([2, 4, 8, 16, 32] if dim else [4, 8, 16])
            mixer = latent(heads, dim, rot_dim, rng.choice([4, 8, 12, 16, 32]), rng.choice([8, 16, 24, 32, 48, 56, 64, 80]),
                           rng.choice([5, 16, 24, 40]), rng.choice([0.1, 0.2, 0.35]), rng.choice([None, 5, 16, 31, 64, 100]),
                           base=rng.choice([100.0, 10000.0, 500000.0]))
        else:
            heads = rng.choice([1, 2, 3, 4, 8])
            mixer = lightning(heads, rng.choice([4, 8, 12, 16, 32, 48]), rng.choice([4, 8, 12, 16, 32, 40]),
                              [rng.choice([0.3, 0.8, 0.95, 0.99, 0.999, 1.0]) for _ in range(heads)])
        kind = rng.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.55:
            mlp = dense(rng.choice([32, 48, 100, 128]))
        else:
            groups = rng.choice([None, 1, 2, 4])
            per = rng.choice([1, 2, 3, 4])
            if groups:
                keep = rng.randint(1, groups)
                experts = groups * per
                top = rng.randint(1, min(4, keep * per))
            else:
                keep, experts = None, rng.choice([2, 4, 7, 16])
                top = rng.randint(1, min(4, experts))
            mlp = moe(rng.choice([16, 24, 40, 64]), experts, top, groups, keep, rng.choice([None, 0.5, 1.0, 2.5]))
        layers.append(layer(mixer, mlp))
    cfg = {"architecture": "Kikunex", "vocab": rng.choice([50, 257, 400]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.7:
        cfg["logit_scale"] = rng.choice([0.125, 0.3, 1.0, 3.0])
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return cfg, rng.choice([4, 8, 16, 32])
