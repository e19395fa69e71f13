"""Typed configuration of Mafalorn, read from its own config.json keys.

A Mafalorn folder names its design in ``architecture`` and gives every size
and constant that may differ between models: ``vocab``, ``width``,
``norm.eps``, ``logit_scale`` and ``layers``, each with ``type``
(``retention``, ``parallel`` or ``latent_attention``), the mixer's sizes in
``mixer`` and its feed-forward in ``mlp``: ``{"kind": "moe", "expert": {"ff":
n}, "router": {"experts", "top", "identity", "groups": {"count", "keep"}}}`` or
null (or absent) for none.  No size has a default: a size that is missing is
an error, so that a model never runs on a guess.  A mechanism that the file
does not mention at all does not exist in that model: without ``logit_scale``
the logits leave as they are; a mixer without ``rot`` turns nothing, a
rotation without ``scaling`` keeps its frequencies, a latent attention without
``mask`` sees every earlier token; a router without ``identity`` has no
outputs that hand the input through, and one without ``groups`` chooses among
all its outputs.
"""

from __future__ import annotations

import copy
import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidInput, Unsupported
from .zifunex import _get, _int, _number

ARCHITECTURE = "Mafalorn"
MIXERS = ("retention", "parallel", "latent_attention")


def _real(raw, key, where) -> float:
    value = _get(raw, key, where)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(float(value)):
        raise InvalidInput(f"config.json {where}.{key} must be a finite number; got {value!r}")
    return float(value)


@dataclass
class Rotation:
    """``dims`` channels of a head turned by the position, frequency i = base^(-2i / dims); ``ramp``: (factor,
    original, fast, slow), frequencies divided by ``factor`` where they turn slowly, blended over the pairs between."""

    dims: int
    base: float
    ramp: Optional[Tuple[float, float, float, float]] = None

    @classmethod
    def from_dict(cls, raw, where, most):
        out = cls(_int(raw, "dims", where, least=2), _number(raw, "base", where))
        if out.dims % 2 or out.dims > most:
            raise InvalidInput(f"config.json {where}.dims must be even and at most {most}; got {out.dims}")
        scaling = raw.get("scaling")
        if scaling is not None:
            spot = where + ".scaling"
            out.ramp = (_number(scaling, "factor", spot), _number(scaling, "original", spot), _number(scaling, "fast", spot),
                        _number(scaling, "slow", spot))
        return out

    def key(self):
        return (self.dims, self.base, self.ramp)


@dataclass
class RetentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: List[float]
    rot: Optional[Rotation] = None

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_int(raw, "heads", where), _int(raw, "dim", where), _int(raw, "vdim", where), [])
        decay = _get(raw, "decay", where)
        if not isinstance(decay, list) or len(decay) != out.heads:
            raise InvalidInput(f"config.json {where}.decay must list one decay for each of the {out.heads} heads")
        for value in decay:
            if isinstance(value, bool) or not isinstance(value, (int, float)) or not 0.0 < float(value) <= 1.0:
                raise InvalidInput(f"config.json {where}.decay: a decay lies in (0, 1]; got {value!r}")
        out.decay = [float(value) for value in decay]
        if raw.get("rot") is not None:
            out.rot = Rotation.from_dict(raw["rot"], where + ".rot", out.dim)
        return out


@dataclass
class SoftmaxSizes:
    """The left side of a ``parallel`` mixer: grouped causal attention whose values are the keys as projected."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    rot: Optional[Rotation] = None

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_int(raw, "heads", where), _int(raw, "kv_heads", where), _int(raw, "dim", where), _number(raw, "scale", where))
        if out.heads % out.kv_heads:
            raise InvalidInput(f"config.json {where}: {out.heads} heads do not divide into {out.kv_heads} kv_heads")
        if raw.get("vdim") is not None and _int(raw, "vdim", where) != out.dim:
            raise InvalidInput(f"config.json {where}: the values are the keys, so vdim must be dim ({out.dim}); got {raw['vdim']}")
        if raw.get("rot") is not None:
            out.rot = Rotation.from_dict(raw["rot"], where + ".rot", out.dim)
        return out


@dataclass
class DeltaSizes:
    """The right side of a ``parallel`` mixer: the gated delta rule."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_int(raw, "heads", where), _int(raw, "kv_heads", where), _int(raw, "dim", where), _int(raw, "vdim", where),
                  _int(raw, "conv", where))
        if out.heads % out.kv_heads:
            raise InvalidInput(f"config.json {where}: {out.heads} heads do not divide into {out.kv_heads} kv_heads")
        return out


@dataclass
class LatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float = 0.0
    window: int = 0  # 0: every earlier token is seen

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_int(raw, "heads", where), _int(raw, "dim", where),
                  _int(raw, "rot_dim", where, least=0) if raw.get("rot_dim") is not None else 0,
                  _int(raw, "vdim", where), _int(raw, "kv_rank", where), _number(raw, "scale", where))
        if out.rot_dim:
            rot = Rotation.from_dict(_get(raw, "rot", where), where + ".rot", out.rot_dim)
            if rot.dims != out.rot_dim or rot.ramp is not None:
                raise InvalidInput(f"config.json {where}.rot turns the rot_dim ({out.rot_dim}) channels, all of them, unscaled")
            out.rot_base = rot.base
        if raw.get("mask") is not None:
            out.window = _int(raw["mask"], "size", where + ".mask")
        return out


@dataclass
class RouterSizes:
    experts: int
    top: int
    identity: int
    expert_ff: int
    groups: Optional[Tuple[int, int]] = None  # (count, keep)


@dataclass
class LayerSizes:
    type: str
    retention: Optional[RetentionSizes] = None
    left: Optional[SoftmaxSizes] = None
    right: Optional[DeltaSizes] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    latent: Optional[LatentSizes] = None
    router: Optional[RouterSizes] = None


def _router(mlp, where) -> RouterSizes:
    form = _get(mlp, "kind", where)
    if form != "moe":
        raise Unsupported(f"config.json {where}.kind {form!r}; this design's feed-forward is a mixture of experts (moe)")
    router = _get(mlp, "router", where)
    spot = where + ".router"
    out = RouterSizes(_int(router, "experts", spot), _int(router, "top", spot),
                      _int(router, "identity", spot, least=0) if router.get("identity") is not None else 0,
                      _int(_get(mlp, "expert", where), "ff", where + ".expert"))
    outputs = out.experts + out.identity
    if out.top > outputs:
        raise InvalidInput(f"config.json {spot}: the {out.top} largest of {outputs} outputs")
    groups = router.get("groups")
    if groups is not None:
        count, keep = _int(groups, "count", spot + ".groups"), _int(groups, "keep", spot + ".groups")
        if outputs % count or keep > count or out.top > keep * (outputs // count):
            raise InvalidInput(f"config.json {spot}.groups: {outputs} outputs in {count} equal groups of which {keep} are kept "
                               f"must leave {out.top} to choose")
        if count > 1:
            out.groups = (count, keep)
    return out


@dataclass
class MafalornConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: List[LayerSizes]
    raw: Dict[str, Any] = field(default_factory=dict)
    architecture: str = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "MafalornConfig":
        layers = _get(raw, "layers", "file")
        if not isinstance(layers, list) or not layers:
            raise InvalidInput("config.json layers must be a list with at least one layer")
        out_layers: List[LayerSizes] = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind, mixer = _get(layer, "type", where), _get(layer, "mixer", where)
            spot = where + ".mixer"
            if kind == "retention":
                sizes = LayerSizes(kind, retention=RetentionSizes.from_dict(mixer, spot))
            elif kind == "parallel":
                sizes = LayerSizes(kind, left=SoftmaxSizes.from_dict(_get(mixer, "left", spot), spot + ".left"),
                                   right=DeltaSizes.from_dict(_get(mixer, "right", spot), spot + ".right"),
                                   left_scale=_real(mixer, "left_scale", spot), right_scale=_real(mixer, "right_scale", spot))
            elif kind == "latent_attention":
                sizes = LayerSizes(kind, latent=LatentSizes.from_dict(mixer, spot))
            else:
                raise Unsupported(f"config.json {where}.type {kind!r}; this design has the mixers {', '.join(MIXERS)}")
            mlp = layer.get("mlp") if isinstance(layer, dict) else None  # (absent or null: the layer has no feed-forward)
            if mlp is not None:
                sizes.router = _router(mlp, where + ".mlp")
            out_layers.append(sizes)
        return cls(
            vocab=_int(raw, "vocab", "file"), width=_int(raw, "width", "file"), eps=_number(_get(raw, "norm", "file"), "eps", "norm"),
            logit_scale=_real(raw, "logit_scale", "file") if raw.get("logit_scale") is not None else 1.0,
            layers=out_layers, raw=copy.deepcopy(raw))

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
