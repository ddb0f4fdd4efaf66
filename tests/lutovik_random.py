"""Random valid Lutovik configurations drawn by a seeded generator: layer order, head counts, sizes, rotations, taps,
groups, experts, every optional key present or absent."""


def _rot(rng, dim):
    dims = rng.choice([0, 2 * rng.randint(1, dim // 2), dim - dim % 2])
    r = {"base": rng.choice([10000.0, 100.0, 5e5]), "dims": dims}
    if dims and rng.random() < 0.5:
        low = rng.choice([1.0, 2.0])
        r["scaling"] = {"factor": rng.choice([2.0, 4.0, 8.0, 32.0]), "low": low, "high": low + rng.choice([1.0, 3.0, 6.0]),
                        "original": rng.choice([16, 64, 512, 4096])}
    return r


def _attention(rng, head_sizes):
    kv = rng.choice([1, 2, 3])
    dim = rng.choice(head_sizes)
    vdim = rng.choice([dim, rng.choice(head_sizes)])
    return {"heads": kv * rng.choice([1, 2, 4]), "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": rng.choice([dim ** -0.5, 0.1, 0.3]),
            "rot": _rot(rng, dim)}


def _state_space(rng):
    groups = rng.choice([1, 2, 3])
    heads = groups * rng.choice([1, 2, 4])
    vdim = rng.choice([4, 12, 16, 48, 64, 72])
    ng = rng.choice([g for g in (1, 2, 3, 4, heads) if (heads * vdim) % g == 0])
    return {"heads": heads, "vdim": vdim, "state": rng.choice([4, 8, 16, 24, 32, 64, 100]), "groups": groups,
            "conv": rng.choice([1, 2, 3, 4, 5]), "norm_groups": ng}


def _mlp(rng):
    kind = rng.choice(["dense", "moe", "moe", None])
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": rng.choice([16 * rng.randint(2, 20), rng.randint(20, 300)])}
    experts = rng.choice([2, 3, 5, 8, 17])
    d = {"kind": "moe", "expert": {"ff": rng.choice([16 * rng.randint(1, 8), rng.randint(10, 90)])},
         "router": {"experts": experts, "top": rng.randint(1, min(experts, 4))}}
    if rng.random() < 0.6:
        d["shared"] = {"ff": rng.choice([16 * rng.randint(1, 8), rng.randint(10, 90)])}
    return d


def draw(rng, head_sizes=(8, 12, 16, 24, 32, 40, 48, 64)):
    layers, owners = [], []
    for i in range(rng.randint(1, 6)):
        kind = rng.choice(["attention", "attention", "parallel"])
        if kind == "parallel":
            mixer = {"left": _attention(rng, head_sizes), "right": _state_space(rng)}
        elif owners and rng.random() < 0.4:
            j = rng.choice(owners)
            mixer = dict(layers[j]["mixer"], heads=layers[j]["mixer"]["kv_heads"] * rng.choice([1, 2, 4]), kv_from=j,
                         scale=rng.choice([0.1, 0.2]))
        else:
            mixer = _attention(rng, head_sizes)
            owners.append(i)
        layers.append({"type": kind, "mixer": mixer, "mlp": _mlp(rng)})
    return {"architecture": "Lutovik", "vocab": rng.randint(50, 2000), "width": 8 * rng.randint(4, 40) + rng.choice([0, 0, 0, 4, 2]),
            "embedding": {"scale": rng.choice([1.0, 4.0, 11.5])}, "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}
