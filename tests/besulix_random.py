"""Random valid Besulix configurations drawn by a seeded generator: layer order, head counts, sizes, rotations, chunks,
caps, limits and weights."""


def _left(rng, head_sizes):
    kv = rng.choice([1, 2, 3])
    dim = rng.choice(head_sizes)
    vdim = rng.choice([dim, rng.choice(head_sizes)])
    return {"heads": kv * rng.choice([1, 2, 4]), "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": rng.choice([dim ** -0.5, 0.1, 0.3]),
            "rot": {"base": rng.choice([10000.0, 100.0, 2.5e5]), "dims": rng.choice([0, 2 * rng.randint(1, dim // 2), dim])},
            "mask": {"size": rng.choice([1, 2, 5, 16, 24, 64, 100, 4096])}}


def _mlp(rng):
    if rng.random() < 0.3:
        return None
    return {"kind": "dense", "ff": rng.choice([16 * rng.randint(2, 20), rng.randint(20, 300)]), "limit": rng.choice([0.5, 1.0, 3.0, 7.0])}


def draw(rng, head_sizes=(8, 12, 16, 24, 32, 40, 48, 64)):
    layers = []
    for _ in range(rng.randint(1, 6)):
        if rng.random() < 0.5:
            mixer = {"left": _left(rng, head_sizes), "left_scale": rng.choice([1.0, 0.5, 1.3]),
                     "right": {"heads": rng.choice([1, 2, 3, 6]), "dim": rng.choice([4, 12, 16, 32, 48, 64, 72, 130])},
                     "right_scale": rng.choice([1.0, 0.8, 1.1])}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": _mlp(rng)})
        else:
            mixer = {"heads": rng.choice([1, 2, 3, 6]), "dim": rng.choice([4, 12, 16, 32, 48, 64, 72, 130]),
                     "vdim": rng.choice([6, 16, 40, 64, 70, 128, 200]), "gate_cap": rng.choice([5.0, 12.0, 15.0])}
            layers.append({"type": "mlstm", "mixer": mixer, "mlp": _mlp(rng)})
    return {"architecture": "Besulix", "vocab": rng.randint(50, 2000), "width": 8 * rng.randint(4, 40) + rng.choice([0, 0, 0, 4, 2]),
            "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "logit_softcap": rng.choice([None, 30.0, 8.0]), "layers": layers}
