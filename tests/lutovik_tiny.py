"""The tests' own small Lutovik configurations.

P mixes everything: attention layers with values larger and smaller than keys, a rotation of part of a head with
scaled frequencies, layers on another layer's cache (with another number of query heads), parallel layers whose
attention rotates all or part of a head, state-space mixers with several groups, taps and norm groups, a layer
without a feed-forward, dense layers, mixtures with and without a shared expert, two and all experts chosen.
Q takes the values that hide faults when they are 1 or equal: one head, one kv head, equal key and value sizes, no
rotation at all, one tap (no convolution state), one group, one norm group, one expert chosen of many, a width that
no matrix-core kernel takes.
S is P's shape with the attentions' scores scaled up until a softmax picks single keys: a key that is lost, or seen
one place off, then changes the logits by far more than any tolerance.
"""
import json
import os

from trapetum_amd.config import LutovikConfig
from trapetum_amd.weights import write_model_folder


def _rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def _att(heads, kv_heads, dim, vdim, scale, rot, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _moe(ff, experts, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def config_p(scale=1.0):
    scaled = _rot(500.0, 8, (8.0, 1.0, 3.0, 64))           # wavelengths 6 .. 200: kept, mixed and divided frequencies
    a = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.2 * scale, rot=scaled)
    b = dict(heads=3, kv_heads=3, dim=24, vdim=8, scale=0.25 * scale, rot=_rot(77.0, 24))
    A = lambda m, mlp: {"type": "attention", "mixer": m, "mlp": mlp}
    Pl = lambda left, right, mlp: {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}
    return {"architecture": "Lutovik", "vocab": 211, "width": 96, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
            "layers": [A(_att(**a), {"kind": "dense", "ff": 72}),
                       Pl(_att(2, 1, 32, 16, 0.15 * scale, _rot(1000.0, 32)), _ssm(4, 12, 16, 2, 4, 3), _moe(40, 5, 2, shared=24)),
                       A(_att(**dict(a, heads=6), kv_from=0), None),
                       Pl(_att(3, 3, 16, 16, 0.3 * scale, _rot(50.0, 8)), _ssm(3, 20, 8, 1, 2, 1), _moe(24, 4, 1)),
                       A(_att(**b), _moe(32, 3, 3, shared=16)),
                       A(_att(**b, kv_from=4), {"kind": "dense", "ff": 56})]}


def config_q():
    one = _att(1, 1, 12, 12, 0.3, _rot(10000.0, 0))
    return {"architecture": "Lutovik", "vocab": 97, "width": 50, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
            "layers": [{"type": "parallel", "mixer": {"left": one, "right": _ssm(1, 10, 4, 1, 1, 1)}, "mlp": _moe(30, 9, 1)},
                       {"type": "attention", "mixer": dict(one, heads=5, rot=_rot(10000.0, 6)), "mlp": _moe(18, 2, 2, shared=20)}]}


CONFIGS = {"P": (config_p(), dict(seed=21, sigma=0.12, sigma_norm=0.3)),
           "Q": (config_q(), dict(seed=22, sigma=0.15, sigma_norm=0.2)),
           "S": (config_p(scale=12.0), dict(seed=23, sigma=0.12, sigma_norm=0.3))}


def make_folder(tmp_path, which):
    cfg, init = CONFIGS[which]
    folder = os.path.join(str(tmp_path), f"lutovik_{which}")
    write_model_folder(LutovikConfig.from_dict(cfg), folder, **init)
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == cfg                     # the configuration writes back what it read
    return folder
