"""Vogunex's configuration: a nested config.json.

    {"architecture": "Vogunex", "vocab": V, "width": D, "embedding": {"scale": s}, "norm": {"eps": e},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "rot": {"base", "dims"},
                           "mask": {"size", "pool"}},
                 "mlp": MLP, "weights_of"?: j},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot": {"base", "dims"},
                           "mask": {"size"}},
                 "mlp": MLP, "weights_of"?: j},
                {"type": "mamba2",
                 "mixer": {"heads", "vdim", "state", "groups", "conv", "norm_groups"},
                 "mlp": MLP, "weights_of"?: j}, ...]}
    MLP = null | {"kind": "dense", "ff"} |
          {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"}, "shared"?: {"ff", "limit"}}

Every size and constant is read from there; the layers may come in any order and number.  A layer with
`weights_of: j` has no tensors of its own: it runs on layer j's (mixer, feed-forward, norms, shift) with a cache and
states of its own, and the rest of its entry repeats layer j's.
"""
import dataclasses
from typing import Optional, Tuple, Union

from .base import ConfigError, ModelConfig, _coerce
from .lutovik import StateSpaceConfig


def _need(d, name, kind, where):
    if not isinstance(d, dict):
        raise ConfigError(f"config.json: '{where}' must be an object")
    if name not in d:
        raise ConfigError(f"config.json has no '{where}.{name}'" if where else f"config.json has no '{name}'")
    return _coerce(f"{where}.{name}" if where else name, kind, d[name])


def _positive(m, names, where):
    for name in names:
        if getattr(m, name) <= 0:
            raise ConfigError(f"config key '{where}.{name}' must be positive, found {getattr(m, name)}")


def _rotation(d, where, limit):
    rot = d.get("rot") if isinstance(d, dict) else None
    base, dims = _need(rot, "base", "float", where + ".rot"), _need(rot, "dims", "int", where + ".rot")
    if base <= 0 or dims % 2 or not 0 <= dims <= limit:
        raise ConfigError(f"'{where}.rot': base must be positive and dims ({dims}) even and at most {limit}")
    return base, dims


@dataclasses.dataclass(frozen=True)
class PooledAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # query/key elements per head
    vdim: int                # value elements per head
    scale: float
    softcap: Optional[float]
    rot_base: float
    rot_dims: int
    window: int              # positions a query sees token by token, its own included
    pool: Optional[int]      # tokens per pooled block before the window (None: nothing is seen there)

    @staticmethod
    def from_dict(d, where):
        mask = d.get("mask") if isinstance(d, dict) else None
        m = PooledAttentionConfig(
            heads=_need(d, "heads", "int", where), kv_heads=_need(d, "kv_heads", "int", where),
            dim=_need(d, "dim", "int", where), vdim=_need(d, "vdim", "int", where), scale=_need(d, "scale", "float", where),
            softcap=_coerce(where + ".softcap", "opt_float", d.get("softcap")),
            rot_base=0.0, rot_dims=0, window=_need(mask, "size", "int", where + ".mask"),
            pool=_coerce(where + ".mask.pool", "opt_int", mask.get("pool")))
        base, dims = _rotation(d, where, m.dim)
        m = dataclasses.replace(m, rot_base=base, rot_dims=dims)
        _positive(m, ("heads", "kv_heads", "dim", "vdim", "window"), where)
        if m.heads % m.kv_heads:
            raise ConfigError(f"'{where}': {m.heads} heads are no multiple of {m.kv_heads} kv_heads")
        if m.scale <= 0 or (m.softcap is not None and m.softcap <= 0) or (m.pool is not None and m.pool <= 0):
            raise ConfigError(f"'{where}': scale, softcap and mask.pool must be positive")
        return m

    def to_dict(self):
        mask = {"size": self.window}
        if self.pool is not None:
            mask["pool"] = self.pool
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "softcap": self.softcap, "rot": {"base": self.rot_base, "dims": self.rot_dims}, "mask": mask}


@dataclasses.dataclass(frozen=True)
class WindowedLatentConfig:
    heads: int
    dim: int                 # unrotated query/key elements per head
    rot_dim: int             # rotated query/key elements per head; the key's are shared by the heads
    vdim: int
    kv_rank: int             # size of the cached latent
    q_rank: int              # size of the queries' latent
    scale: float
    rot_base: float
    rot_dims: int
    window: int

    @staticmethod
    def from_dict(d, where):
        mask = d.get("mask") if isinstance(d, dict) else None
        m = WindowedLatentConfig(
            **{k: _need(d, k, "int", where) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank")},
            scale=_need(d, "scale", "float", where), rot_base=0.0, rot_dims=0, window=_need(mask, "size", "int", where + ".mask"))
        _positive(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "window"), where)
        base, dims = _rotation(d, where, m.rot_dim)
        if m.scale <= 0:
            raise ConfigError(f"'{where}.scale' must be positive")
        return dataclasses.replace(m, rot_base=base, rot_dims=dims)

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "q_rank": self.q_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims},
                "mask": {"size": self.window}}


@dataclasses.dataclass(frozen=True)
class VogunexFeedForwardConfig:
    kind: str                # "dense" or "moe"
    ff: int                  # width of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    limit: float = 0.0
    shared_ff: Optional[int] = None
    shared_limit: float = 0.0

    @staticmethod
    def from_dict(d, where):
        kind = _need(d, "kind", "str", where)
        if kind == "dense":
            f = VogunexFeedForwardConfig("dense", _need(d, "ff", "int", where))
        elif kind == "moe":
            ex, ro, sh = d.get("expert"), d.get("router"), d.get("shared")
            f = VogunexFeedForwardConfig(
                "moe", _need(ex, "ff", "int", where + ".expert"), experts=_need(ro, "experts", "int", where + ".router"),
                top=_need(ro, "top", "int", where + ".router"), limit=_need(ex, "limit", "float", where + ".expert"),
                shared_ff=None if sh is None else _need(sh, "ff", "int", where + ".shared"),
                shared_limit=0.0 if sh is None else _need(sh, "limit", "float", where + ".shared"))
            if not 0 < f.top <= f.experts:
                raise ConfigError(f"'{where}.router': top ({f.top}) must lie between 1 and experts ({f.experts})")
            if f.limit <= 0 or (f.shared_ff is not None and (f.shared_ff <= 0 or f.shared_limit <= 0)):
                raise ConfigError(f"'{where}': the experts' limits and the shared expert's ff must be positive")
        else:
            raise ConfigError(f"'{where}.kind' is '{kind}': neither dense nor moe")
        if f.ff <= 0:
            raise ConfigError(f"'{where}': ff must be positive, found {f.ff}")
        return f

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        d = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


MIXERS = {"attention": PooledAttentionConfig, "latent_attention": WindowedLatentConfig, "mamba2": StateSpaceConfig}


@dataclasses.dataclass(frozen=True)
class VogunexLayerConfig:
    type: str
    mixer: Union[PooledAttentionConfig, WindowedLatentConfig, StateSpaceConfig]
    mlp: Optional[VogunexFeedForwardConfig]
    weights_of: Optional[int] = None


@dataclasses.dataclass
class VogunexConfig(ModelConfig):
    architecture = "Vogunex"

    vocab_size: int = 0
    hidden_size: int = 0
    embedding_scale: float = 1.0
    norm_eps: float = 1e-6
    layers: Tuple[VogunexLayerConfig, ...] = ()

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
            if kind not in MIXERS:
                raise ConfigError(f"'{where}.type' is '{kind}': this design's mixers are {', '.join(MIXERS)}")
            mlp = l.get("mlp")
            out.append(VogunexLayerConfig(kind, MIXERS[kind].from_dict(l.get("mixer"), where + ".mixer"),
                                          None if mlp is None else VogunexFeedForwardConfig.from_dict(mlp, where + ".mlp"),
                                          _coerce(where + ".weights_of", "opt_int", l.get("weights_of"))))
        cfg = cls(vocab_size=_need(d, "vocab", "int", ""), hidden_size=_need(d, "width", "int", ""),
                  embedding_scale=_need(d.get("embedding"), "scale", "float", "embedding"),
                  norm_eps=_need(d.get("norm"), "eps", "float", "norm"), layers=tuple(out))
        cfg.validate()
        return cfg

    def to_dict(self):
        layers = []
        for l in self.layers:
            e = {"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps}, "layers": layers}

    def validate(self):
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"vocab ({self.vocab_size}) and width ({self.hidden_size}) must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        for i, l in enumerate(self.layers):
            j = l.weights_of
            if j is None:
                continue
            if not 0 <= j < len(self.layers) or j == i or self.layers[j].weights_of is not None:
                raise ConfigError(f"layers[{i}].weights_of names layer {j}, which is no other layer with tensors of its own")
            o = self.layers[j]
            if (o.type, o.mixer, o.mlp) != (l.type, l.mixer, l.mlp):
                raise ConfigError(f"layers[{i}] runs on the weights of layer {j}: type, mixer and mlp must be equal")
