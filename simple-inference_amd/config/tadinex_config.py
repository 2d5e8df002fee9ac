"""Typed configuration of the Tadinex design, read from its own config.json keys.

A Tadinex config.json names the design in ``architecture`` and describes every layer in ``layers``: the kind of its
mixer (``type``: ``delta`` or ``parallel``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``:
``dense``, ``moe`` or null).  ``embedding.scale`` multiplies the embedded rows, ``norm.eps`` is the constant of every
root mean square and ``residual_mult`` the factor on every sublayer's result.  Every size and constant comes from
here; what the file does not mention is not there (no rotation scaling, no shared expert, no identity experts, no
feed-forward).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .famepel_config import Rotation
from .model_config import ConfigError
from .mogisun_config import _need, _positive, _positive_int


def _number(v, what: str) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != v:
        raise ConfigError(f"{what} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d, where):
        m = cls(*(_positive_int(_need(d, k, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim", "conv")))
        if m.heads % m.kv_heads:
            raise ConfigError(f"{where}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        return m

    def to_dict(self) -> dict:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class WindowAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    scale: float
    rot: Rotation

    @classmethod
    def from_dict(cls, d, where):
        ints = [_positive_int(_need(d, k, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim")]
        if ints[0] % ints[1]:
            raise ConfigError(f"{where}: heads {ints[0]} is not a multiple of kv_heads {ints[1]}")
        if ints[3] != ints[2]:
            raise ConfigError(f"{where}: the values are the keys, so vdim {ints[3]} must equal dim {ints[2]}")
        window = _positive_int(_need(_need(d, "mask", where), "size", f"{where}.mask"), f"{where}.mask.size")
        rot = Rotation.from_dict(_need(d, "rot", where), f"{where}.rot")
        if rot.dims > ints[2]:
            raise ConfigError(f"{where}: rot.dims {rot.dims} exceeds dim {ints[2]}")
        return cls(*ints, window, _positive(_need(d, "scale", where), f"{where}.scale"), rot)

    def to_dict(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "mask": {"size": self.window},
                "rot": self.rot.to_dict(), "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class DecayAttention:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def from_dict(cls, d, where):
        ints = [_positive_int(_need(d, k, where), f"{where}.{k}") for k in ("heads", "dim", "vdim")]
        decay = _need(d, "decay", where)
        if not isinstance(decay, (list, tuple)) or len(decay) != ints[0]:
            raise ConfigError(f"{where}.decay must list one number for each of the {ints[0]} heads")
        return cls(*ints, tuple(_number(x, f"{where}.decay[{i}]") for i, x in enumerate(decay)))

    def to_dict(self) -> dict:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelMixer:
    left: WindowAttention
    right: DecayAttention
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d, where):
        return cls(WindowAttention.from_dict(_need(d, "left", where), f"{where}.left"),
                   DecayAttention.from_dict(_need(d, "right", where), f"{where}.right"),
                   _number(_need(d, "left_scale", where), f"{where}.left_scale"),
                   _number(_need(d, "right_scale", where), f"{where}.right_scale"))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseMlp:
    ff: int

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class ClampedExperts:
    experts: int          # experts with tensors of their own
    identity: int         # further outputs of the router: experts that return their input
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int]
    shared_limit: Optional[float]

    @classmethod
    def from_dict(cls, d, where):
        router = _need(d, "router", where)
        rw = f"{where}.router"
        experts = _positive_int(_need(router, "experts", rw), f"{rw}.experts")
        identity = router.get("identity", 0)
        if isinstance(identity, bool) or not isinstance(identity, int) or identity < 0:
            raise ConfigError(f"{rw}.identity must be a count, got {identity!r}")
        top = _positive_int(_need(router, "top", rw), f"{rw}.top")
        if top > experts + identity:
            raise ConfigError(f"{rw}.top {top} exceeds the {experts + identity} outputs of the router")
        expert = _need(d, "expert", where)
        ff = _positive_int(_need(expert, "ff", f"{where}.expert"), f"{where}.expert.ff")
        limit = _positive(_need(expert, "limit", f"{where}.expert"), f"{where}.expert.limit")
        shared = d.get("shared")
        sff = slim = None
        if shared is not None:
            sff = _positive_int(_need(shared, "ff", f"{where}.shared"), f"{where}.shared.ff")
            slim = _positive(_need(shared, "limit", f"{where}.shared"), f"{where}.shared.limit")
        return cls(experts, identity, top, ff, limit, sff, slim)

    def to_dict(self) -> dict:
        d = {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
             "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


@dataclass(frozen=True)
class TadinexLayer:
    type: str
    mixer: Union[DeltaMixer, ParallelMixer]
    mlp: Union[DenseMlp, ClampedExperts, None]

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


_MIXERS = {"delta": DeltaMixer, "parallel": ParallelMixer}


@dataclass(frozen=True)
class TadinexConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    layers: Tuple[TadinexLayer, ...]
    architecture: str = "Tadinex"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TadinexConfig":
        vocab = _positive_int(_need(d, "vocab", "config"), "vocab")
        width = _positive_int(_need(d, "width", "config"), "width")
        eps = _positive(_need(_need(d, "norm", "config"), "eps", "norm"), "norm.eps")
        entries = _need(d, "layers", "config")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError("config.json's layers must be a list with at least one layer")
        layers = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"{where}.type {kind!r} is not implemented (known: {', '.join(sorted(_MIXERS))})")
            mixer = _MIXERS[kind].from_dict(_need(e, "mixer", where), f"{where}.mixer")
            mlp = e.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", f"{where}.mlp")
                if mk == "dense":
                    mlp = DenseMlp(_positive_int(_need(mlp, "ff", f"{where}.mlp"), f"{where}.mlp.ff"))
                elif mk == "moe":
                    mlp = ClampedExperts.from_dict(mlp, f"{where}.mlp")
                else:
                    raise ConfigError(f"{where}.mlp.kind {mk!r} is not implemented (known: 'dense', 'moe')")
            layers.append(TadinexLayer(str(kind), mixer, mlp))
        emb = d.get("embedding", {})
        scale = emb.get("scale", 1.0) if isinstance(emb, Mapping) else 1.0
        return cls(vocab, width, eps, _positive(scale, "embedding.scale"),
                   _number(d.get("residual_mult", 1.0), "residual_mult"), tuple(layers),
                   str(d.get("architecture", "Tadinex")))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
