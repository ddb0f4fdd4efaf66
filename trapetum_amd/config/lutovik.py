"""Lutovik's configuration: a nested config.json.

    {"architecture": "Lutovik", "vocab": V, "width": D, "embedding": {"scale": s}, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "rot": ROT, "kv_from"?},
                 "mlp": MLP},
                {"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "rot": ROT},
                           "right": {"heads", "vdim", "state", "groups", "conv", "norm_groups"}},
                 "mlp": MLP}, ...]}
    ROT = {"base", "dims", "scaling"?: {"factor", "low", "high", "original"}}
    MLP = null | {"kind": "dense", "ff"} |
          {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}, "shared"?: {"ff"}}

Every size and constant is read from there; the layers may come in any order and number.  `kv_from: j` marks an
attention layer without key and value projections: it attends over what layer j cached.
"""
import dataclasses
from typing import Optional, Tuple, Union

from .base import ConfigError, ModelConfig, _coerce


def _need(d, name, kind, where):
    if not isinstance(d, dict):
        raise ConfigError(f"config.json: '{where}' must be an object")
    if name not in d:
        raise ConfigError(f"config.json has no '{where}.{name}'" if where else f"config.json has no '{name}'")
    return _coerce(f"{where}.{name}" if where else name, kind, d[name])


@dataclasses.dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]] = None      # (factor, low, high, original)

    @staticmethod
    def from_dict(d, where):
        sc = d.get("scaling") if isinstance(d, dict) else None
        r = RotationConfig(_need(d, "base", "float", where), _need(d, "dims", "int", where),
                           None if sc is None else tuple(_need(sc, k, "float", where + ".scaling")
                                                         for k in ("factor", "low", "high", "original")))
        if r.base <= 0 or r.dims < 0 or r.dims % 2:
            raise ConfigError(f"'{where}': base must be positive and dims ({r.dims}) even")
        if r.scaling is not None:
            factor, low, high, original = r.scaling
            if factor <= 0 or original <= 0 or low <= 0 or high <= low:
                raise ConfigError(f"'{where}.scaling': factor, low and original must be positive and high above low")
        return r

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            f, lo, hi, orig = self.scaling
            d["scaling"] = {"factor": f, "low": lo, "high": hi, "original": int(orig) if orig == int(orig) else orig}
        return d

    def scaling_dict(self):
        if self.scaling is None:
            return None
        return dict(zip(("factor", "low", "high", "original"), self.scaling))


@dataclasses.dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # query/key elements per head
    vdim: int                # value elements per head
    scale: float
    rot: RotationConfig
    kv_from: Optional[int] = None

    @staticmethod
    def from_dict(d, where):
        m = AttentionConfig(
            heads=_need(d, "heads", "int", where), kv_heads=_need(d, "kv_heads", "int", where),
            dim=_need(d, "dim", "int", where), vdim=_need(d, "vdim", "int", where), scale=_need(d, "scale", "float", where),
            rot=RotationConfig.from_dict(d.get("rot"), where + ".rot"),
            kv_from=_coerce(where + ".kv_from", "opt_int", d.get("kv_from")))
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(m, name) <= 0:
                raise ConfigError(f"config key '{where}.{name}' must be positive, found {getattr(m, name)}")
        if m.heads % m.kv_heads:
            raise ConfigError(f"'{where}': {m.heads} heads are no multiple of {m.kv_heads} kv_heads")
        if m.scale <= 0:
            raise ConfigError(f"'{where}.scale' must be positive")
        if m.rot.dims > m.dim:
            raise ConfigError(f"'{where}.rot.dims' ({m.rot.dims}) exceeds dim ({m.dim})")
        return m

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict()}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclasses.dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int                # channels per head
    state: int               # rows of a head's state
    groups: int              # heads of one group share B and C
    conv: int                # taps of the short convolution
    norm_groups: int

    @staticmethod
    def from_dict(d, where):
        m = StateSpaceConfig(**{k: _need(d, k, "int", where) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")})
        for name in ("heads", "vdim", "state", "groups", "conv", "norm_groups"):
            if getattr(m, name) <= 0:
                raise ConfigError(f"config key '{where}.{name}' must be positive, found {getattr(m, name)}")
        if m.heads % m.groups:
            raise ConfigError(f"'{where}': {m.heads} heads are no multiple of {m.groups} groups")
        if (m.heads * m.vdim) % m.norm_groups:
            raise ConfigError(f"'{where}': norm_groups ({m.norm_groups}) must divide heads * vdim ({m.heads * m.vdim})")
        return m

    def to_dict(self):
        return dataclasses.asdict(self)


@dataclasses.dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: StateSpaceConfig

    @staticmethod
    def from_dict(d, where):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        left = AttentionConfig.from_dict(d.get("left"), where + ".left")
        if left.kv_from is not None:
            raise ConfigError(f"'{where}.left' has kv_from: the attention of a parallel mixer keeps keys and values of its own")
        return ParallelConfig(left, StateSpaceConfig.from_dict(d.get("right"), where + ".right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclasses.dataclass(frozen=True)
class LutovikFeedForwardConfig:
    kind: str                # "dense" or "moe"
    ff: int                  # width of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None

    @staticmethod
    def from_dict(d, where):
        kind = _need(d, "kind", "str", where)
        if kind == "dense":
            f = LutovikFeedForwardConfig("dense", _need(d, "ff", "int", where))
        elif kind == "moe":
            ex, ro, sh = d.get("expert"), d.get("router"), d.get("shared")
            f = LutovikFeedForwardConfig("moe", _need(ex, "ff", "int", where + ".expert"),
                                         experts=_need(ro, "experts", "int", where + ".router"),
                                         top=_need(ro, "top", "int", where + ".router"),
                                         shared_ff=None if sh is None else _need(sh, "ff", "int", where + ".shared"))
            if not 0 < f.top <= f.experts:
                raise ConfigError(f"'{where}.router': top ({f.top}) must lie between 1 and experts ({f.experts})")
            if f.shared_ff is not None and f.shared_ff <= 0:
                raise ConfigError(f"'{where}.shared.ff' must be positive, found {f.shared_ff}")
        else:
            raise ConfigError(f"'{where}.kind' is '{kind}': neither dense nor moe")
        if f.ff <= 0:
            raise ConfigError(f"'{where}': ff must be positive, found {f.ff}")
        return f

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        d = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclasses.dataclass(frozen=True)
class LutovikLayerConfig:
    type: str                # "attention" or "parallel"
    mixer: Union[AttentionConfig, ParallelConfig]
    mlp: Optional[LutovikFeedForwardConfig]


@dataclasses.dataclass
class LutovikConfig(ModelConfig):
    architecture = "Lutovik"

    vocab_size: int = 0
    hidden_size: int = 0
    embedding_scale: float = 1.0
    norm_eps: float = 1e-6
    layers: Tuple[LutovikLayerConfig, ...] = ()

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
            if kind == "attention":
                mixer = AttentionConfig.from_dict(l.get("mixer"), where + ".mixer")
            elif kind == "parallel":
                mixer = ParallelConfig.from_dict(l.get("mixer"), where + ".mixer")
            else:
                raise ConfigError(f"'{where}.type' is '{kind}': this design's mixers are attention and parallel")
            mlp = l.get("mlp")
            out.append(LutovikLayerConfig(kind, mixer, None if mlp is None else LutovikFeedForwardConfig.from_dict(mlp, where + ".mlp")))
        cfg = cls(vocab_size=_need(d, "vocab", "int", ""), hidden_size=_need(d, "width", "int", ""),
                  embedding_scale=_need(d.get("embedding"), "scale", "float", "embedding"),
                  norm_eps=_need(d.get("norm"), "eps", "float", "norm"), layers=tuple(out))
        cfg.validate()
        return cfg

    def to_dict(self):
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                           for l in self.layers]}

    def validate(self):
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"vocab ({self.vocab_size}) and width ({self.hidden_size}) must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        for i, l in enumerate(self.layers):
            j = l.mixer.kv_from if l.type == "attention" else None
            if j is None:
                continue
            if not 0 <= j < i:
                raise ConfigError(f"layers[{i}].mixer.kv_from names layer {j}, which does not run before it")
            if self.layers[j].type != "attention" or self.layers[j].mixer.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from names layer {j}, which has no attention with keys and values of its own")
            o, m = self.layers[j].mixer, l.mixer
            if (o.kv_heads, o.dim, o.vdim, o.rot) != (m.kv_heads, m.dim, m.vdim, m.rot):
                raise ConfigError(f"layers[{i}] reads the cache of layer {j}: kv_heads, dim, vdim and rotation must be equal")
