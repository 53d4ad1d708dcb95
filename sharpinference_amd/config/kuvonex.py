"""Configuration of the Kuvonex design: a list of layers, each a latent attention mixer and,
optionally, a routed feed-forward, with norms on the branches' outputs.

``config.json`` of this design is nested: ``embedding.scale``, ``norm.eps``, ``vocab``, ``width`` and
``layers``, one object per layer with ``type``, the mixer's sizes (``mixer``) and its feed-forward
(``mlp``, or null).  Every size and constant is read here and nowhere else; a key this reader does
not know is refused with its name when its value could change the computation.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, special_tokens_from

LAYER_TYPES = ("latent_attention",)
MLP_KINDS = ("moe",)


def _only(d: Dict[str, Any], known, where: str) -> None:
    extra = sorted(k for k in d if k not in known)
    if extra:
        raise ConfigError(f"{where}: unknown key(s) {', '.join(extra)}")


def _num(d: Dict[str, Any], key: str, where: str, kind=int, default=None):
    if key not in d or d[key] is None:
        if default is not None:
            return default
        raise ConfigError(f"{where}: '{key}' is missing")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (kind is int and int(v) != v):
        raise ConfigError(f"{where}: '{key}' must be {'an integer' if kind is int else 'a number'} (got {v!r})")
    return kind(v)


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int                    # unrotated width of a query / key head
    rot_dim: int                # rotated width
    vdim: int                   # width of a value head
    kv_rank: int                # width of the latent
    scale: float                # of the scores
    rot_base: float
    rot_dims: int               # leading elements of the rotated part that turn (pairs 2i, 2i + 1)
    kv_from: Optional[int] = None   # the layer whose latent and rotated key part this one attends over

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LatentMixerConfig":
        _only(d, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot", "kv_from"), where)
        rot = d.get("rot")
        if not isinstance(rot, dict):
            raise ConfigError(f"{where}: 'rot' (base, dims) is missing")
        _only(rot, ("base", "dims"), where + ".rot")
        dim, rot_dim = _num(d, "dim", where), _num(d, "rot_dim", where)
        return cls(heads=_num(d, "heads", where), dim=dim, rot_dim=rot_dim, vdim=_num(d, "vdim", where),
                   kv_rank=_num(d, "kv_rank", where),
                   scale=_num(d, "scale", where, float, 1.0 / math.sqrt(dim + rot_dim)),
                   rot_base=_num(rot, "base", where + ".rot", float), rot_dims=_num(rot, "dims", where + ".rot", int, rot_dim),
                   kv_from=None if d.get("kv_from") is None else _num(d, "kv_from", where))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "scale": self.scale,
                               "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class RoutedMlpConfig:
    experts: int
    top: int
    ff: int                     # an expert's inner width
    groups: int = 1             # equal groups of neighbouring experts
    keep: int = 1               # groups whose experts can be chosen

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RoutedMlpConfig":
        _only(d, ("kind", "expert", "router"), where)
        if d.get("kind") not in MLP_KINDS:
            raise ConfigError(f"{where}: feed-forward kind {d.get('kind')!r} is not known ({', '.join(MLP_KINDS)})")
        expert, router = d.get("expert"), d.get("router")
        if not isinstance(expert, dict) or not isinstance(router, dict):
            raise ConfigError(f"{where}: 'expert' and 'router' objects are wanted")
        _only(expert, ("ff",), where + ".expert")
        _only(router, ("experts", "top", "groups"), where + ".router")
        groups = router.get("groups")
        if groups is not None:
            if not isinstance(groups, dict):
                raise ConfigError(f"{where}.router: 'groups' must be an object (count, keep)")
            _only(groups, ("count", "keep"), where + ".router.groups")
        return cls(experts=_num(router, "experts", where + ".router"), top=_num(router, "top", where + ".router"),
                   ff=_num(expert, "ff", where + ".expert"),
                   groups=1 if groups is None else _num(groups, "count", where + ".router.groups"),
                   keep=1 if groups is None else _num(groups, "keep", where + ".router.groups"))

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if (self.groups, self.keep) != (1, 1):
            router["groups"] = {"count": self.groups, "keep": self.keep}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": router}


@dataclass(frozen=True)
class KuvonexLayerConfig:
    type: str
    mixer: LatentMixerConfig
    mlp: Optional[RoutedMlpConfig]

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "KuvonexLayerConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: a layer must be an object")
        _only(d, ("type", "mixer", "mlp"), where)
        if d.get("type") not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {d.get('type')!r} is not known ({', '.join(LAYER_TYPES)})")
        if not isinstance(d.get("mixer"), dict):
            raise ConfigError(f"{where}: 'mixer' is missing")
        mlp = d.get("mlp")
        return cls(type=d["type"], mixer=LatentMixerConfig.from_dict(d["mixer"], where + ".mixer"),
                   mlp=None if mlp is None else RoutedMlpConfig.from_dict(mlp, where + ".mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass
class KuvonexConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    layers: Tuple[KuvonexLayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KuvonexConfig":
        _only(d, ("architecture", "architectures", "embedding", "layers", "norm", "vocab", "width", "eos_token_id",
                  "bos_token_id"), "config.json")
        emb, norm = d.get("embedding") or {}, d.get("norm") or {}
        if not isinstance(emb, dict) or not isinstance(norm, dict):
            raise ConfigError("config.json: 'embedding' and 'norm' must be objects")
        _only(emb, ("scale",), "embedding")
        _only(norm, ("eps",), "norm")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        name = d.get("architecture") or (d.get("architectures") or ["Kuvonex"])[0]
        return cls(architecture=str(name), vocab_size=_num(d, "vocab", "config.json"), width=_num(d, "width", "config.json"),
                   norm_eps=_num(norm, "eps", "norm", float), embedding_scale=_num(emb, "scale", "embedding", float, 1.0),
                   layers=tuple(KuvonexLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   **special_tokens_from(d))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                               "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                               "vocab": self.vocab_size, "width": self.width}
        out.update(self.special_tokens_dict())
        return out

    def validate(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{i}].mixer"
            if min(m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank) < 1:
                raise ConfigError(f"{where}: heads, dim, rot_dim, vdim and kv_rank must be positive")
            if m.rot_dims % 2 or not 2 <= m.rot_dims <= m.rot_dim:
                raise ConfigError(f"{where}: rot.dims {m.rot_dims} must be even and lie in 2..rot_dim {m.rot_dim}")
            if not m.rot_base > 0:
                raise ConfigError(f"{where}: rot.base must be positive")
            if m.kv_from is not None:
                if not 0 <= m.kv_from < i:
                    raise ConfigError(f"{where}: kv_from {m.kv_from} must name an earlier layer")
                src = self.layers[m.kv_from].mixer
                if src.kv_from is not None:
                    raise ConfigError(f"{where}: kv_from names layer {m.kv_from}, which keeps no latent of its own")
                if (src.kv_rank, src.rot_dim, src.rot_base, src.rot_dims) != (m.kv_rank, m.rot_dim, m.rot_base, m.rot_dims):
                    raise ConfigError(f"{where}: kv_rank, rot_dim and rot must equal those of layer {m.kv_from}")
            f = layer.mlp
            if f is not None:
                where = f"layers[{i}].mlp"
                if f.ff < 1 or not 1 <= f.top <= f.experts:
                    raise ConfigError(f"{where}: expert.ff must be positive and 1 <= top <= experts")
                if not 1 <= f.keep <= f.groups or f.experts % f.groups:
                    raise ConfigError(f"{where}: {f.groups} groups (keep {f.keep}) do not divide {f.experts} experts")
                if f.top > f.keep * (f.experts // f.groups):
                    raise ConfigError(f"{where}: top {f.top} exceeds the experts of the {f.keep} kept group(s)")
