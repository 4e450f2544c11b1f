"""Tiny Rununex configurations for the tests.  They differ in every size and option: the order of the two kinds of
layer, heads and kv heads (equal, or one kv head for all), key and value sizes (equal or not, multiples of four or
not), chunks that differ between layers (or none), taps of the convolutions, rotated entries (all of a head's or
some), the frequency scaling (or none), state sizes, groups of the state-space mixer and of its norm, scales of the
two side-by-side mixers, experts (one chosen or several, a shared one or not, no feed-forward at all), the
embedding's, the residual's and the logits' factors."""


def attention(heads, kv_heads, dim, vdim, scale, diff, conv, chunk, rot_dims=None, base=10000.0, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "conv": conv}
    if chunk:
        m["mask"] = {"size": chunk}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": m}


def parallel(left, right, left_scale, right_scale):
    heads, kv_heads, dim, vdim, scale, chunk = left
    lm = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        lm["mask"] = {"size": chunk}
    rheads, rvdim, state, groups, conv, norm_groups = right
    rm = {"heads": rheads, "vdim": rvdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}
    return {"type": "parallel", "mixer": {"left": lm, "right": rm, "left_scale": left_scale, "right_scale": right_scale}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def moe(ff, experts, top, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


# parallel first; chunks of 9 and 14; three taps; some entries rotated, frequencies scaled; two experts of five
R_A = {
    "architecture": "Rununex", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "residual_mult": 0.5, "logit_scale": 0.5,
    "layers": [
        layer(parallel((4, 2, 16, 8, 0.3, 9), (4, 8, 16, 2, 3, 2), 0.6, 1.3), moe(24, 5, 2, shared=40)),
        layer(attention(2, 1, 16, 24, 0.2, 0.25, 3, 14, rot_dims=8, base=100.0, scaling=(4.0, 1.0, 3.0, 16)), moe(32, 4, 1)),
        layer(parallel((2, 2, 8, 12, 0.4, 14), (2, 12, 8, 1, 2, 1), 1.0, 1.0), None),
    ],
}

# nothing divides by four; no chunk in one attention layer; two taps and five; one layer without a feed-forward;
# every expert chosen; no factors at the ends
R_B = {
    "architecture": "Rununex", "vocab": 131, "width": 50, "norm": {"eps": 3e-6},
    "layers": [
        layer(attention(3, 3, 10, 7, 0.31, 0.4, 2, None, rot_dims=10, base=500.0), None),
        layer(parallel((3, 1, 7, 9, 0.25, 6), (3, 5, 7, 3, 5, 3), 0.7, 0.9), moe(30, 3, 3, shared=22)),
        layer(attention(1, 1, 14, 11, 0.25, 0.1, 5, 11, rot_dims=6, base=77.0, scaling=(8.0, 1.0, 4.0, 64)), moe(22, 6, 3)),
        layer(parallel((5, 5, 6, 5, 0.5, None), (1, 9, 11, 1, 1, 1), 1.5, 0.4), moe(16, 2, 1, shared=16)),
    ],
}

# sizes in powers of two; a long chunk and a short one; no rotation in one layer; no convolution in one
R_C = {
    "architecture": "Rununex", "vocab": 384, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 11.3},
    "residual_mult": 0.8, "logit_scale": 2.0,
    "layers": [
        layer(attention(4, 2, 32, 32, 0.18, 0.3, 4, 100, rot_dims=32, base=100000.0, scaling=(8.0, 1.0, 4.0, 256)), moe(64, 8, 2, shared=128)),
        layer(parallel((8, 2, 16, 16, 0.25, 20), (4, 32, 32, 2, 4, 2), 0.8, 1.1), moe(64, 16, 4)),
        layer(attention(2, 2, 64, 16, 0.12, 0.2, 0, 20), moe(128, 4, 1, shared=64)),
        layer(parallel((2, 1, 64, 64, 0.125, 100), (8, 16, 64, 4, 4, 4), 1.0, 0.5), moe(32, 8, 1, shared=32)),
    ],
}

ALL = {"A": (R_A, 4, 11), "B": (R_B, 8, 12), "C": (R_C, 16, 13)}
STD = 0.05      # spread of the random weights: every branch moves the logits


def random_configuration(seed):
    """A configuration drawn at random: every size, the layers' order and kinds, the chunks, taps, groups."""
    import random
    rng = random.Random(seed)
    width = rng.choice([24, 40, 64, 72, 96])
    layers = []
    for _ in range(rng.randint(1, 4)):
        if rng.random() < 0.5:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([4, 6, 8, 12, 16, 32])
            rot = rng.choice([None, 2, 4, dim])
            mixer = attention(kv * rng.choice([1, 2, 3]), kv, dim, rng.choice([4, 7, 8, 16, 24]), rng.choice([0.1, 0.2, 0.35]),
                              rng.choice([0.1, 0.3, 0.5]), rng.choice([0, 1, 2, 3, 4]), rng.choice([None, 3, 5, 16, 31, 64]),
                              rot_dims=min(rot, dim) if rot else None, base=rng.choice([100.0, 10000.0, 500000.0]),
                              scaling=rng.choice([None, (8.0, 1.0, 4.0, 32), (2.0, 0.5, 2.0, 8)]))
        else:
            kv = rng.choice([1, 2])
            groups = rng.choice([1, 2])
            heads = groups * rng.choice([1, 2, 3])
            vdim = rng.choice([4, 6, 8, 16])
            parts = rng.choice([p for p in (1, 2, 3, 4) if (heads * vdim) % p == 0])
            mixer = parallel((kv * rng.choice([1, 2, 4]), kv, rng.choice([4, 7, 8, 16]), rng.choice([4, 5, 8, 16]),
                              rng.choice([0.1, 0.25, 0.5]), rng.choice([None, 2, 7, 16, 33])),
                             (heads, vdim, rng.choice([4, 8, 12, 16]), groups, rng.choice([1, 2, 3, 4]), parts),
                             rng.choice([0.5, 1.0, 1.4]), rng.choice([0.3, 1.0, 1.2]))
        if rng.random() < 0.2:
            mlp = None
        else:
            experts = rng.choice([1, 2, 4, 7])
            mlp = moe(rng.choice([16, 24, 40]), experts, rng.randint(1, min(3, experts)), rng.choice([None, 16, 28]))
        layers.append(layer(mixer, mlp))
    cfg = {"architecture": "Rununex", "vocab": rng.choice([50, 257, 400]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.7:
        cfg["logit_scale"] = rng.choice([0.125, 0.3, 1.0, 3.0])
    if rng.random() < 0.7:
        cfg["residual_mult"] = rng.choice([0.4, 0.9, 1.3])
    if rng.random() < 0.7:
        cfg["embedding"] = {"scale": rng.choice([0.5, 4.0, 9.5])}
    return cfg, rng.choice([4, 8, 16, 32])
