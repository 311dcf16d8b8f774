"""Besulix's configuration: a nested config.json.

    {"architecture": "Besulix", "vocab": V, "width": D, "norm": {"eps": e}, "logit_softcap": c,
     "layers": [{"type": "mlstm", "mixer": {"heads", "dim", "vdim", "gate_cap"}, "mlp": MLP},
                {"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "rot": {"base", "dims"}, "mask": {"size"}},
                           "right": {"heads", "dim"}, "left_scale", "right_scale"},
                 "mlp": MLP}, ...]}
    MLP = null | {"kind": "dense", "ff", "limit"}

Every size and constant is read from there; the layers may come in any order and number.
"""
import dataclasses
from typing import Optional, Tuple, Union

from .base import ConfigError, ModelConfig, _coerce
from .lutovik import RotationConfig, _need


def _positive(obj, names, where):
    for name in names:
        if getattr(obj, name) <= 0:
            raise ConfigError(f"config key '{where}.{name}' must be positive, found {getattr(obj, name)}")


@dataclasses.dataclass(frozen=True)
class ChunkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # query/key elements per head
    vdim: int                # value elements per head
    scale: float
    rot: RotationConfig
    chunk: int               # mask.size: a query sees the keys of its own chunk of this many positions

    @staticmethod
    def from_dict(d, where):
        m = ChunkAttentionConfig(
            heads=_need(d, "heads", "int", where), kv_heads=_need(d, "kv_heads", "int", where),
            dim=_need(d, "dim", "int", where), vdim=_need(d, "vdim", "int", where), scale=_need(d, "scale", "float", where),
            rot=RotationConfig.from_dict(d.get("rot"), where + ".rot"),
            chunk=_need(d.get("mask"), "size", "int", where + ".mask"))
        _positive(m, ("heads", "kv_heads", "dim", "vdim", "scale", "chunk"), where)
        if m.heads % m.kv_heads:
            raise ConfigError(f"'{where}': {m.heads} heads are no multiple of {m.kv_heads} kv_heads")
        if m.rot.dims > m.dim:
            raise ConfigError(f"'{where}.rot.dims' ({m.rot.dims}) exceeds dim ({m.dim})")
        if m.rot.scaling is not None:
            raise ConfigError(f"'{where}.rot': this design's rotation has no frequency scaling")
        if m.vdim % 2:
            raise ConfigError(f"'{where}.vdim' ({m.vdim}) must be even: values are rotated in pairs")
        return m

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "rot": self.rot.to_dict(), "mask": {"size": self.chunk}}


@dataclasses.dataclass(frozen=True)
class TimeMixConfig:
    heads: int
    dim: int                 # key channels of a head, and its value channels

    @staticmethod
    def from_dict(d, where):
        m = TimeMixConfig(_need(d, "heads", "int", where), _need(d, "dim", "int", where))
        _positive(m, ("heads", "dim"), where)
        return m

    def to_dict(self):
        return dataclasses.asdict(self)


@dataclasses.dataclass(frozen=True)
class BesulixParallelConfig:
    left: ChunkAttentionConfig
    right: TimeMixConfig
    left_scale: float
    right_scale: float

    @staticmethod
    def from_dict(d, where):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        return BesulixParallelConfig(ChunkAttentionConfig.from_dict(d.get("left"), where + ".left"),
                                     TimeMixConfig.from_dict(d.get("right"), where + ".right"),
                                     _need(d, "left_scale", "float", where), _need(d, "right_scale", "float", where))

    def to_dict(self):
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclasses.dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @staticmethod
    def from_dict(d, where):
        m = MatrixMemoryConfig(_need(d, "heads", "int", where), _need(d, "dim", "int", where), _need(d, "vdim", "int", where),
                               _need(d, "gate_cap", "float", where))
        _positive(m, ("heads", "dim", "vdim", "gate_cap"), where)
        return m

    def to_dict(self):
        return dataclasses.asdict(self)


@dataclasses.dataclass(frozen=True)
class BesulixFeedForwardConfig:
    ff: int
    limit: float

    @staticmethod
    def from_dict(d, where):
        kind = _need(d, "kind", "str", where)
        if kind != "dense":
            raise ConfigError(f"'{where}.kind' is '{kind}': this design's feed-forward is dense")
        f = BesulixFeedForwardConfig(_need(d, "ff", "int", where), _need(d, "limit", "float", where))
        _positive(f, ("ff", "limit"), where)
        return f

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclasses.dataclass(frozen=True)
class BesulixLayerConfig:
    type: str                # "mlstm" or "parallel"
    mixer: Union[MatrixMemoryConfig, BesulixParallelConfig]
    mlp: Optional[BesulixFeedForwardConfig]


@dataclasses.dataclass
class BesulixConfig(ModelConfig):
    architecture = "Besulix"

    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    logit_softcap: Optional[float] = None
    layers: Tuple[BesulixLayerConfig, ...] = ()

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
            if kind == "mlstm":
                mixer = MatrixMemoryConfig.from_dict(l.get("mixer"), where + ".mixer")
            elif kind == "parallel":
                mixer = BesulixParallelConfig.from_dict(l.get("mixer"), where + ".mixer")
            else:
                raise ConfigError(f"'{where}.type' is '{kind}': this design's mixers are mlstm and parallel")
            mlp = l.get("mlp")
            out.append(BesulixLayerConfig(kind, mixer, None if mlp is None else BesulixFeedForwardConfig.from_dict(mlp, where + ".mlp")))
        cfg = cls(vocab_size=_need(d, "vocab", "int", ""), hidden_size=_need(d, "width", "int", ""),
                  norm_eps=_need(d.get("norm"), "eps", "float", "norm"),
                  logit_softcap=_coerce("logit_softcap", "opt_float", d.get("logit_softcap")), layers=tuple(out))
        cfg.validate()
        return cfg

    def to_dict(self):
        return {"architecture": self.architecture,
                "layers": [{"mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict(), "type": l.type}
                           for l in self.layers],
                "logit_softcap": self.logit_softcap, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size}

    def validate(self):
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"vocab ({self.vocab_size}) and width ({self.hidden_size}) must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.logit_softcap is not None and self.logit_softcap <= 0:
            raise ConfigError("logit_softcap must be positive (or null for none)")
