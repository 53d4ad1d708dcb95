"""Configuration of the Pazatar design: a list of layers, each a mixer between two norms and,
optionally, a dense feed-forward between two more; a stretch of the layers may run several times.

``config.json`` of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``layers`` (one object
per layer: ``type`` "attention" or "parallel", the mixer's sizes in ``mixer``, the feed-forward in
``mlp`` or null) and ``loop`` (``start``, ``stop``, ``times``: layers start .. stop - 1 run `times`
times in a row with the same weights).  Every size and constant is read here and nowhere else; a
key this reader does not know is refused with its name.

One size is in no key of the file: the narrow middle of the decay projection of a gated linear
mixer.  It is the first dimension of the tensor ``l<i>.mix.right.a1`` and is taken from there when
a model folder is opened (``with_tensor_shapes``); a configuration made by hand may give it as
``decay_rank`` (random-weights mode falls back to DEFAULT_DECAY_RANK).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, special_tokens_from
from .kuvonex import _num, _only

LAYER_TYPES = ("attention", "parallel")
MLP_KINDS = ("dense",)
DEFAULT_DECAY_RANK = 16


@dataclass(frozen=True)
class RotConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[Tuple[str, float], ...]] = None    # the scaling rule's numbers, sorted by name

    def scaling_dict(self) -> Optional[Dict[str, float]]:
        return None if self.scaling is None else dict(self.scaling)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, scaling_keys: Tuple[str, ...]) -> "RotConfig":
        _only(d, ("base", "dims", "scaling"), where)
        sc = d.get("scaling")
        scaling = None
        if sc is not None:
            if not isinstance(sc, dict):
                raise ConfigError(f"{where}.scaling must be an object ({', '.join(scaling_keys)})")
            _only(sc, scaling_keys, where + ".scaling")
            scaling = tuple(sorted((k, _num(sc, k, where + ".scaling", float)) for k in scaling_keys))
        return cls(base=_num(d, "base", where, float), dims=_num(d, "dims", where), scaling=scaling)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(self.scaling)
        return out


YARN_KEYS = ("factor", "original", "fast", "slow")
WAVELENGTH_KEYS = ("factor", "low", "high", "original")


@dataclass(frozen=True)
class SoftmaxMixerConfig:
    """A softmax attention mixer: the 'attention' layer's, or the left half of a 'parallel' one."""

    heads: int
    kv_heads: int
    dim: int                    # width of a query / key head
    vdim: int                   # width of a value head
    scale: float                # of the scores
    mask_size: int = 0          # chunk length (0: every earlier key is seen)
    rot: Optional[RotConfig] = None
    softcap: float = 0.0        # 0: scores are not capped
    conv: int = 0               # taps of the short convolutions behind the projections (0: none)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, left: bool) -> "SoftmaxMixerConfig":
        known = ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot") + (("softcap", "conv") if left else ())
        _only(d, known, where)
        mask = d.get("mask")
        if mask is not None:
            if not isinstance(mask, dict):
                raise ConfigError(f"{where}.mask must be an object (size)")
            _only(mask, ("size",), where + ".mask")
        rot = d.get("rot")
        if rot is not None and not isinstance(rot, dict):
            raise ConfigError(f"{where}.rot must be an object (base, dims, scaling)")
        heads, dim = _num(d, "heads", where), _num(d, "dim", where)
        return cls(heads=heads, kv_heads=_num(d, "kv_heads", where, int, heads), dim=dim, vdim=_num(d, "vdim", where, int, dim),
                   scale=_num(d, "scale", where, float, 1.0 / math.sqrt(dim)),
                   mask_size=0 if mask is None else _num(mask, "size", where + ".mask"),
                   rot=None if rot is None else RotConfig.from_dict(rot, where + ".rot", WAVELENGTH_KEYS if left else YARN_KEYS),
                   softcap=float(d["softcap"]) if left and d.get("softcap") is not None else 0.0,
                   conv=int(d["conv"]) if left and d.get("conv") is not None else 0)

    def to_dict(self, left: bool) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.mask_size:
            out["mask"] = {"size": self.mask_size}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if left and self.softcap:
            out["softcap"] = self.softcap
        if left and self.conv:
            out["conv"] = self.conv
        return out


@dataclass(frozen=True)
class GatedLinearMixerConfig:
    heads: int
    dim: int                    # key channels of a head
    vdim: int                   # value channels of a head
    tau: float
    decay_rank: Optional[int] = None     # None: not known yet (it is a tensor's shape)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "GatedLinearMixerConfig":
        _only(d, ("heads", "dim", "vdim", "tau", "decay_rank"), where)
        dim = _num(d, "dim", where)
        return cls(heads=_num(d, "heads", where), dim=dim, vdim=_num(d, "vdim", where, int, dim), tau=_num(d, "tau", where, float),
                   decay_rank=None if d.get("decay_rank") is None else _num(d, "decay_rank", where))

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


@dataclass(frozen=True)
class PazatarLayerConfig:
    type: str
    attention: Optional[SoftmaxMixerConfig] = None      # type "attention": the mixer; "parallel": its left half
    linear: Optional[GatedLinearMixerConfig] = None     # type "parallel": its right half
    ff: int = 0                                         # inner width of the dense feed-forward (0: none)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "PazatarLayerConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: a layer must be an object")
        _only(d, ("type", "mixer", "mlp"), where)
        kind = d.get("type")
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: layer type {kind!r} is not known ({', '.join(LAYER_TYPES)})")
        mixer = d.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"{where}: 'mixer' is missing")
        mlp = d.get("mlp")
        ff = 0
        if mlp is not None:
            if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp: feed-forward kind is not known ({', '.join(MLP_KINDS)})")
            _only(mlp, ("kind", "ff"), where + ".mlp")
            ff = _num(mlp, "ff", where + ".mlp")
        if kind == "attention":
            return cls(kind, SoftmaxMixerConfig.from_dict(mixer, where + ".mixer", left=False), None, ff)
        _only(mixer, ("left", "right"), where + ".mixer")
        if not isinstance(mixer.get("left"), dict) or not isinstance(mixer.get("right"), dict):
            raise ConfigError(f"{where}.mixer: 'left' and 'right' objects are wanted")
        return cls(kind, SoftmaxMixerConfig.from_dict(mixer["left"], where + ".mixer.left", left=True),
                   GatedLinearMixerConfig.from_dict(mixer["right"], where + ".mixer.right"), ff)

    def to_dict(self) -> Dict[str, Any]:
        if self.type == "attention":
            mixer = self.attention.to_dict(left=False)
        else:
            mixer = {"left": self.attention.to_dict(left=True), "right": self.linear.to_dict()}
        return {"type": self.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": self.ff} if self.ff else None}


@dataclass
class PazatarConfig(ModelConfig):
    vocab_size: int = 0
    width: int = 0
    norm_eps: float = 1e-5
    layers: Tuple[PazatarLayerConfig, ...] = ()
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1          # 1 with start == stop: no loop

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PazatarConfig":
        _only(d, ("architecture", "architectures", "layers", "loop", "norm", "vocab", "width", "eos_token_id", "bos_token_id"),
              "config.json")
        norm = d.get("norm") or {}
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        _only(norm, ("eps",), "norm")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json: 'loop' must be an object (start, stop, times)")
            _only(loop, ("start", "stop", "times"), "loop")
            start, stop, times = _num(loop, "start", "loop"), _num(loop, "stop", "loop"), _num(loop, "times", "loop")
        name = d.get("architecture") or (d.get("architectures") or ["Pazatar"])[0]
        return cls(architecture=str(name), vocab_size=_num(d, "vocab", "config.json"), width=_num(d, "width", "config.json"),
                   norm_eps=_num(norm, "eps", "norm", float),
                   layers=tuple(PazatarLayerConfig.from_dict(l, f"layers[{i}]") for i, l in enumerate(layers)),
                   loop_start=start, loop_stop=stop, loop_times=times, **special_tokens_from(d))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                               "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.width}
        if self.has_loop:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        out.update(self.special_tokens_dict())
        return out

    def with_tensor_shapes(self, available: Dict[str, tuple]) -> "PazatarConfig":
        """The sizes that only a tensor's shape gives, filled in from a weight file's index
        (name -> (shape, dtype)): the decay projections' narrow middle."""
        layers = list(self.layers)
        for i, layer in enumerate(layers):
            if layer.linear is not None and layer.linear.decay_rank is None:
                entry = available.get(f"l{i}.mix.right.a1")
                if entry is not None and len(entry[0]) == 2:
                    layers[i] = replace(layer, linear=replace(layer.linear, decay_rank=int(entry[0][0])))
        return replace(self, layers=tuple(layers))

    def validate(self) -> None:
        if self.vocab_size < 1 or self.width < 1 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if (self.loop_start, self.loop_stop, self.loop_times) != (0, 0, 1):
            if not 0 <= self.loop_start < self.loop_stop <= len(self.layers) or self.loop_times < 1:
                raise ConfigError(f"loop: 0 <= start < stop <= {len(self.layers)} layers and times >= 1 are wanted")
        for i, layer in enumerate(self.layers):
            m, where = layer.attention, f"layers[{i}].mixer" + (".left" if layer.type == "parallel" else "")
            if min(m.heads, m.kv_heads, m.dim, m.vdim) < 1 or m.heads % m.kv_heads:
                raise ConfigError(f"{where}: heads, kv_heads, dim and vdim must be positive and kv_heads divide heads")
            if m.dim % 2:
                raise ConfigError(f"{where}: dim must be even")
            if layer.type == "attention" and m.vdim != m.dim:
                raise ConfigError(f"{where}: the values are the keys, so vdim must equal dim")
            if m.mask_size < 0 or m.softcap < 0 or m.conv < 0 or m.conv == 1:
                raise ConfigError(f"{where}: mask.size and softcap cannot be negative; conv is 0 or at least 2 taps")
            if not m.scale > 0:
                raise ConfigError(f"{where}: scale must be positive")
            if m.rot is not None:
                if m.rot.dims % 2 or not 2 <= m.rot.dims <= m.dim or not m.rot.base > 1:
                    raise ConfigError(f"{where}.rot: dims must be even and lie in 2..dim {m.dim}, base above 1")
                sc = m.rot.scaling_dict()
                if sc is not None and min(sc.values()) <= 0:
                    raise ConfigError(f"{where}.rot.scaling: every number must be positive")
                if sc is not None and "high" in sc and sc["high"] == sc["low"]:
                    raise ConfigError(f"{where}.rot.scaling: low and high must differ")
            if layer.linear is not None:
                r, where = layer.linear, f"layers[{i}].mixer.right"
                if min(r.heads, r.dim, r.vdim) < 1 or not r.tau > 0 or (r.decay_rank is not None and r.decay_rank < 1):
                    raise ConfigError(f"{where}: heads, dim, vdim, tau (and decay_rank) must be positive")
            if layer.ff < 0:
                raise ConfigError(f"layers[{i}].mlp: ff must be positive")
