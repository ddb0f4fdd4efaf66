"""Golepel's configuration: a nested config.json.

    {"architecture": "Golepel", "vocab": V, "width": D, "logit_scale": s,
     "norm": {"eps": e, "groups": g}, "canon": {"taps": t},
     "layers": [{"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot": {"base", "dims"}, "kv_from"?},
                 "mlp": null | {"kind": "dense", "ff"} |
                        {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"}}}, ...]}

Every size and constant is read from there; the layers may come in any order and number.  `kv_from: j` marks a layer
without a down-projection of its own: it attends over what layer j cached.
"""
import dataclasses
from typing import Optional, Tuple

from .base import ConfigError, ModelConfig, _coerce


def _need(d, name, kind, where):
    if not isinstance(d, dict):
        raise ConfigError(f"config.json: '{where}' must be an object")
    if name not in d:
        raise ConfigError(f"config.json has no '{where}.{name}'" if where else f"config.json has no '{name}'")
    return _coerce(f"{where}.{name}" if where else name, kind, d[name])


@dataclasses.dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int                 # unrotated query/key elements per head
    rot_dim: int             # rotated query/key elements per head; the key's are shared by the heads
    vdim: int                # value elements per head
    kv_rank: int             # size of the cached latent
    scale: float
    rot_base: float
    rot_dims: int            # how many of the rot_dim elements turn
    kv_from: Optional[int] = None

    @staticmethod
    def from_dict(d, where):
        rot = d.get("rot") if isinstance(d, dict) else None
        m = LatentMixerConfig(
            heads=_need(d, "heads", "int", where), dim=_need(d, "dim", "int", where),
            rot_dim=_need(d, "rot_dim", "int", where), vdim=_need(d, "vdim", "int", where),
            kv_rank=_need(d, "kv_rank", "int", where), scale=_need(d, "scale", "float", where),
            rot_base=_need(rot, "base", "float", where + ".rot"), rot_dims=_need(rot, "dims", "int", where + ".rot"),
            kv_from=_coerce(where + ".kv_from", "opt_int", d.get("kv_from")))
        for name in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
            if getattr(m, name) <= 0:
                raise ConfigError(f"config key '{where}.{name}' must be positive, found {getattr(m, name)}")
        if m.scale <= 0 or m.rot_base <= 0:
            raise ConfigError(f"'{where}': scale and rot.base must be positive")
        if m.rot_dims % 2 or not 0 <= m.rot_dims <= m.rot_dim:
            raise ConfigError(f"'{where}.rot.dims' ({m.rot_dims}) must be even and at most rot_dim ({m.rot_dim})")
        return m

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclasses.dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                # "dense" or "moe"
    ff: int                  # width of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    limit: float = 0.0

    @staticmethod
    def from_dict(d, where):
        kind = _need(d, "kind", "str", where)
        if kind == "dense":
            f = FeedForwardConfig("dense", _need(d, "ff", "int", where))
        elif kind == "moe":
            ex, ro = d.get("expert"), d.get("router")
            f = FeedForwardConfig("moe", _need(ex, "ff", "int", where + ".expert"),
                                  experts=_need(ro, "experts", "int", where + ".router"),
                                  top=_need(ro, "top", "int", where + ".router"),
                                  limit=_need(ex, "limit", "float", where + ".expert"))
            if not 0 < f.top <= f.experts:
                raise ConfigError(f"'{where}.router': top ({f.top}) must lie between 1 and experts ({f.experts})")
            if f.limit <= 0:
                raise ConfigError(f"'{where}.expert.limit' must be positive, found {f.limit}")
        else:
            raise ConfigError(f"'{where}.kind' is '{kind}': neither dense nor moe")
        if f.ff <= 0:
            raise ConfigError(f"'{where}': ff must be positive, found {f.ff}")
        return f

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top}}


@dataclasses.dataclass(frozen=True)
class GolepelLayerConfig:
    type: str
    mixer: LatentMixerConfig
    mlp: Optional[FeedForwardConfig]


@dataclasses.dataclass
class GolepelConfig(ModelConfig):
    architecture = "Golepel"

    vocab_size: int = 0
    hidden_size: int = 0
    logit_scale: float = 1.0
    norm_eps: float = 1e-6
    norm_groups: int = 1
    canon_taps: int = 1
    layers: Tuple[GolepelLayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, d):
        if not isinstance(d, dict):
            raise ConfigError("config.json must hold a JSON object")
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("config.json has no 'layers' list")
        out = []
        for i, l in enumerate(layers):
            where = f"layers[{i}]"
            kind = _need(l, "type", "str", where)
            if kind != "latent_attention":
                raise ConfigError(f"'{where}.type' is '{kind}': this design's mixer is latent_attention")
            mlp = l.get("mlp")
            out.append(GolepelLayerConfig(kind, LatentMixerConfig.from_dict(l.get("mixer"), where + ".mixer"),
                                          None if mlp is None else FeedForwardConfig.from_dict(mlp, where + ".mlp")))
        cfg = cls(vocab_size=_need(d, "vocab", "int", ""), hidden_size=_need(d, "width", "int", ""),
                  logit_scale=_need(d, "logit_scale", "float", ""),
                  norm_eps=_need(d.get("norm"), "eps", "float", "norm"), norm_groups=_need(d.get("norm"), "groups", "int", "norm"),
                  canon_taps=_need(d.get("canon"), "taps", "int", "canon"), layers=tuple(out))
        cfg.validate()
        return cfg

    def to_dict(self):
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "canon": {"taps": self.canon_taps},
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                           for l in self.layers]}

    def validate(self):
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"vocab ({self.vocab_size}) and width ({self.hidden_size}) must be positive")
        if self.norm_groups <= 0 or self.hidden_size % self.norm_groups:
            raise ConfigError(f"norm.groups ({self.norm_groups}) must divide the width ({self.hidden_size})")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.canon_taps < 1:
            raise ConfigError(f"canon.taps must be at least 1, found {self.canon_taps}")
        for i, l in enumerate(self.layers):
            j = l.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < i:
                raise ConfigError(f"layers[{i}].mixer.kv_from names layer {j}, which does not run before it")
            o = self.layers[j].mixer
            if o.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from names layer {j}, which has no down-projection of its own")
            if (o.kv_rank, o.rot_dim, o.rot_base, o.rot_dims) != (l.mixer.kv_rank, l.mixer.rot_dim, l.mixer.rot_base, l.mixer.rot_dims):
                raise ConfigError(f"layers[{i}] reads the cache of layer {j}: kv_rank, rot_dim and rotation must be equal")
