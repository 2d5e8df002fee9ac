"""Typed configuration of the Famepel design, read from its own config.json keys.

A Famepel config.json names the design in ``architecture`` and describes every layer in ``layers``: the kind of its
mixer (``type``: ``mamba2``, ``hgrn2`` or ``latent_attention``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: a mixture of experts, or null).  ``embedding.scale`` multiplies the embedded rows and
``norm.eps`` is the constant of every root mean square.  Every size and constant comes from here; what the file does
not mention is not there (no rotation scaling, no expert groups, no feed-forward).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .model_config import ConfigError
from .mogisun_config import _need, _positive, _positive_int


@dataclass(frozen=True)
class Mamba2:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, d, where):
        m = cls(*(_positive_int(_need(d, k, where), f"{where}.{k}")
                  for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")))
        if m.heads % m.groups:
            raise ConfigError(f"{where}: heads {m.heads} is not a multiple of groups {m.groups}")
        if (m.heads * m.vdim) % m.norm_groups:
            raise ConfigError(f"{where}: heads * vdim {m.heads * m.vdim} is not a multiple of norm_groups {m.norm_groups}")
        return m

    def to_dict(self) -> dict:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class Hgrn2:
    heads: int
    dim: int
    vdim: int

    @classmethod
    def from_dict(cls, d, where):
        return cls(*(_positive_int(_need(d, k, where), f"{where}.{k}") for k in ("heads", "dim", "vdim")))

    def to_dict(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class RotationScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self) -> dict:
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: Optional[RotationScaling]

    @classmethod
    def from_dict(cls, d, where):
        dims = _positive_int(_need(d, "dims", where), f"{where}.dims")
        if dims % 2:
            raise ConfigError(f"{where}.dims must be even, got {dims}")
        sc = d.get("scaling")
        if sc is not None:
            sc = RotationScaling(*(_positive(_need(sc, k, f"{where}.scaling"), f"{where}.scaling.{k}")
                                   for k in ("factor", "original", "fast", "slow")))
        return cls(_positive(_need(d, "base", where), f"{where}.base"), dims, sc)

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class LatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Rotation
    kv_from: Optional[int]

    @classmethod
    def from_dict(cls, d, where):
        ints = [_positive_int(_need(d, k, where), f"{where}.{k}") for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank")]
        rot = Rotation.from_dict(_need(d, "rot", where), f"{where}.rot")
        if rot.dims > ints[2]:
            raise ConfigError(f"{where}: rot.dims {rot.dims} exceeds rot_dim {ints[2]}")
        src = d.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or src < 0):
            raise ConfigError(f"{where}.kv_from must name a layer, got {src!r}")
        return cls(*ints, _positive(_need(d, "scale", where), f"{where}.scale"), rot, src)

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
             "rot": self.rot.to_dict(), "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class RoutedMlp:
    experts: int
    top: int
    ff: int
    scale: float
    groups: Optional[Tuple[int, int]]     # (count, keep)

    @classmethod
    def from_dict(cls, d, where):
        router = _need(d, "router", where)
        rw = f"{where}.router"
        experts = _positive_int(_need(router, "experts", rw), f"{rw}.experts")
        top = _positive_int(_need(router, "top", rw), f"{rw}.top")
        groups = router.get("groups")
        if groups is not None:
            count = _positive_int(_need(groups, "count", f"{rw}.groups"), f"{rw}.groups.count")
            keep = _positive_int(_need(groups, "keep", f"{rw}.groups"), f"{rw}.groups.keep")
            if experts % count or keep > count:
                raise ConfigError(f"{rw}: {experts} experts do not form {count} equal groups of which {keep} are kept")
            groups = (count, keep)
        allowed = experts if groups is None else experts // groups[0] * groups[1]
        if top > allowed:
            raise ConfigError(f"{rw}.top {top} exceeds the {allowed} experts a token can choose from")
        ff = _positive_int(_need(_need(d, "expert", where), "ff", f"{where}.expert"), f"{where}.expert.ff")
        return cls(experts, top, ff, _positive(router.get("scale", 1.0), f"{rw}.scale"), groups)

    def to_dict(self) -> dict:
        router = {"experts": self.experts, "scale": self.scale, "top": self.top}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": router}


@dataclass(frozen=True)
class FamepelLayer:
    type: str
    mixer: Union[Mamba2, Hgrn2, LatentAttention]
    mlp: Optional[RoutedMlp]

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


_MIXERS = {"mamba2": Mamba2, "hgrn2": Hgrn2, "latent_attention": LatentAttention}


@dataclass(frozen=True)
class FamepelConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: Tuple[FamepelLayer, ...]
    architecture: str = "Famepel"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "FamepelConfig":
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
                if mk != "moe":
                    raise ConfigError(f"{where}.mlp.kind {mk!r} is not implemented (known: 'moe')")
                mlp = RoutedMlp.from_dict(mlp, f"{where}.mlp")
            layers.append(FamepelLayer(str(kind), mixer, mlp))
        for i, layer in enumerate(layers):
            m = layer.mixer
            if isinstance(m, LatentAttention) and m.kv_from is not None:
                src = layers[m.kv_from].mixer if m.kv_from < i else None
                if not isinstance(src, LatentAttention) or src.kv_from is not None:
                    raise ConfigError(f"layers[{i}].mixer.kv_from names layer {m.kv_from}, which is no earlier layer "
                                      f"with a latent of its own")
                if (src.kv_rank, src.rot_dim, src.rot) != (m.kv_rank, m.rot_dim, m.rot):
                    raise ConfigError(f"layers[{i}] cannot read the latent of layer {m.kv_from}: their kv_rank, rot_dim "
                                      f"or rotation differ")
        scale = d.get("embedding", {}).get("scale", 1.0) if isinstance(d.get("embedding", {}), Mapping) else 1.0
        return cls(vocab, width, eps, _positive(scale, "embedding.scale"), tuple(layers),
                   str(d.get("architecture", "Famepel")))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
                "vocab": self.vocab, "width": self.width}
