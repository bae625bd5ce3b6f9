"""Tiny Pubodra configurations for the tests.  They differ in every size and option: heads, the
three head sizes and the latent's size (equal to each other or not, multiples of four or not),
how many of the rotated entries turn, the rotary base and its stretching (or none), windows that
differ between layers (or none), dense, routed and absent feed-forwards, one expert chosen or
several, and where the repeated stretch of layers lies (from the first layer, in the middle,
nowhere)."""


def _mixer(heads, dim, rot_dim, vdim, kv_rank, scale, window, base=10000.0, dims=None, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    return m


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}

# the whole stack runs three times; windows of 24 and 40; sizes in multiples of four
P_A = {
    "architecture": "Pubodra", "vocab": 200, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_mixer(2, 16, 8, 24, 32, 0.2, 24, scaling=YARN), _dense(96)),
        _layer(_mixer(2, 16, 8, 24, 32, 0.2, 40, scaling=YARN), _moe(48, 6, 2)),
    ],
    "loop": {"start": 0, "stop": 2, "times": 3},
}

# nothing divides by four; the loop lies in the middle; one layer has no feed-forward, one no
# window; one expert of five; only six of the ten rotated entries turn
P_B = {
    "architecture": "Pubodra", "vocab": 131, "width": 50, "norm": {"eps": 3e-6},
    "layers": [
        _layer(_mixer(3, 7, 10, 9, 21, 0.31, 17, base=500.0, dims=6), _dense(70)),
        _layer(_mixer(1, 14, 6, 11, 13, 0.25, None, base=77.0), None),
        _layer(_mixer(5, 6, 2, 5, 18, 0.4, 33, base=1000.0), _moe(30, 5, 1)),
        _layer(_mixer(2, 10, 4, 10, 10, 0.3, 9, base=1000.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
               _moe(22, 3, 3)),
    ],
    "loop": {"start": 1, "stop": 3, "times": 2},
}

# no loop; sizes that the matrix-core products take; a long window and a short one
P_C = {
    "architecture": "Pubodra", "vocab": 384, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        _layer(_mixer(4, 32, 16, 32, 48, 0.15, 100, base=100000.0, scaling=YARN), _moe(128, 8, 2)),
        _layer(_mixer(8, 16, 16, 16, 64, 0.18, 20, base=100000.0), _dense(256)),
    ],
}

ALL = {"A": (P_A, 4, 11), "B": (P_B, 8, 12), "C": (P_C, 16, 13)}
STD = 0.05      # spread of the random weights: every branch moves the logits, and no router call is so close that bfloat16 flips it


def random_configuration(seed):
    """A configuration drawn at random: every size, the layers' order and kinds, the windows, the
    rotary constants and the place of the repeated stretch."""
    import random
    rng = random.Random(seed)
    width = rng.choice([24, 40, 64, 72, 96, 128])
    layers = []
    for _ in range(rng.randint(1, 4)):
        heads = rng.choice([1, 2, 3, 4, 6, 8])
        dim = rng.choice([0, 4, 8, 12, 16, 32])
        rot_dim = rng.choice([2, 4, 8, 16, 32] if dim else [4, 8, 16])
        dims = rng.choice([rot_dim, rot_dim, max(2, rot_dim // 2)])
        scaling = None
        if rng.random() < 0.5:
            scaling = {"factor": rng.choice([2.0, 4.0, 16.0]), "original": rng.choice([16, 64, 512]),
                       "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
        mixer = _mixer(heads, dim, rot_dim, rng.choice([4, 8, 12, 16, 32]), rng.choice([8, 16, 24, 32, 48, 56, 64, 80]),
                       rng.choice([0.1, 0.2, 0.35]), rng.choice([None, 5, 16, 31, 64, 100]),
                       base=rng.choice([100.0, 10000.0, 500000.0]), dims=dims, scaling=scaling)
        kind = rng.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.6:
            mlp = _dense(rng.choice([32, 48, 100, 128]))
        else:
            experts = rng.choice([2, 4, 7, 16])
            mlp = _moe(rng.choice([16, 24, 40, 64]), experts, rng.randint(1, min(4, experts)))
        layers.append(_layer(mixer, mlp))
    cfg = {"architecture": "Pubodra", "vocab": rng.choice([50, 257, 400]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return cfg, rng.choice([4, 8, 16, 32])
