"""Typed configuration of Robopel, read from its own config.json keys.

A Robopel folder names its design in ``architecture`` and gives every size and
constant that may differ between models: ``vocab``, ``width``, ``norm.eps``,
``embedding.scale`` and ``layers``, each with ``type`` (``attention`` or
``mingru``), the mixer's sizes in ``mixer`` and its feed-forward in ``mlp``:
``{"kind": "dense", "ff": n}``, ``{"kind": "moe", "expert": {"ff": n},
"router": {"experts", "top", "identity"}}`` or null (or absent) for none.  No size has a
default: a size that is missing is an error, so that a model never runs on a
guess.  A mechanism that the file does not mention at all does not exist in
that model: without ``embedding.scale`` rows stay as they are; an attention
mixer without ``rot`` turns nothing, without ``rot.scaling`` bends no
frequency, without ``softcap`` caps no score, without ``mask`` sees every
earlier key, without ``mask.pool`` sees no pooled blocks, and without
``kv_from`` has keys and values of its own; a router without ``identity`` has
no outputs that hand the input through.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import InvalidInput, Unsupported
from .zifunex import _get, _int, _number

ARCHITECTURE = "Robopel"
MIXERS = ("attention", "mingru")


@dataclass
class FrequencyScaling:
    """Frequencies bent by their wavelength: kept below ``original / high``,
    divided by ``factor`` above ``original / low``, blended in between."""

    factor: float
    low: float
    high: float
    original: float

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_number(raw, "factor", where), _number(raw, "low", where), _number(raw, "high", where), _number(raw, "original", where))
        if out.high == out.low:
            raise InvalidInput(f"config.json {where}: low and high must differ; both are {out.low}")
        return out

    def key(self):
        return (self.factor, self.low, self.high, self.original)


@dataclass
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0  # 0: scores are not capped
    rot_dims: int = 0  # 0: nothing is turned
    rot_base: float = 0.0
    rot_scaling: Optional[FrequencyScaling] = None
    window: int = 0  # 0: every earlier key is seen
    pool: int = 0  # 0: no pooled blocks beside the window
    kv_from: Optional[int] = None

    @classmethod
    def from_dict(cls, raw, where):
        out = cls(_int(raw, "heads", where), _int(raw, "kv_heads", where), _int(raw, "dim", where), _int(raw, "vdim", where),
                  _number(raw, "scale", where))
        if out.heads % out.kv_heads:
            raise InvalidInput(f"config.json {where}: {out.heads} heads do not divide into {out.kv_heads} kv_heads")
        if raw.get("softcap") not in (None, 0, 0.0):  # (a cap of zero caps nothing, as a missing one)
            out.softcap = _number(raw, "softcap", where)
        rot = raw.get("rot")
        if rot is not None:
            out.rot_dims, out.rot_base = _int(rot, "dims", where + ".rot", least=2), _number(rot, "base", where + ".rot")
            if out.rot_dims % 2 or out.rot_dims > out.dim:
                raise InvalidInput(f"config.json {where}.rot.dims must be even and at most dim ({out.dim}); got {out.rot_dims}")
            if rot.get("scaling") is not None:
                out.rot_scaling = FrequencyScaling.from_dict(rot["scaling"], where + ".rot.scaling")
        mask = raw.get("mask")
        if mask is not None:
            out.window = _int(mask, "size", where + ".mask")
            if mask.get("pool") not in (None, 0):  # (blocks of no tokens are no blocks, as a missing size)
                out.pool = _int(mask, "pool", where + ".mask")
        if raw.get("kv_from") is not None:
            out.kv_from = _int(raw, "kv_from", where, least=0)
        return out


@dataclass
class RouterSizes:
    experts: int
    top: int
    identity: int
    expert_ff: int


@dataclass
class LayerSizes:
    type: str
    attention: Optional[AttentionSizes] = None
    gru_width: Optional[int] = None
    ff: Optional[int] = None  # a dense feed-forward's inner size
    router: Optional[RouterSizes] = None  # a mixture of experts


@dataclass
class RobopelConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: List[LayerSizes]
    raw: Dict[str, Any] = field(default_factory=dict)
    architecture: str = ARCHITECTURE

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "RobopelConfig":
        layers = _get(raw, "layers", "file")
        if not isinstance(layers, list) or not layers:
            raise InvalidInput("config.json layers must be a list with at least one layer")
        out_layers: List[LayerSizes] = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            kind, mixer = _get(layer, "type", where), _get(layer, "mixer", where)
            mlp = layer.get("mlp") if isinstance(layer, dict) else None  # (absent or null: the layer has no feed-forward)
            if kind == "attention":
                sizes = LayerSizes(kind, attention=AttentionSizes.from_dict(mixer, where + ".mixer"))
                source = sizes.attention.kv_from
                if source is not None:
                    if source >= index or out_layers[source].type != "attention" or out_layers[source].attention.kv_from is not None:
                        raise InvalidInput(f"config.json {where}.mixer.kv_from {source} must name an earlier attention layer "
                                           "with keys and values of its own")
                    own, other = sizes.attention, out_layers[source].attention
                    if (own.kv_heads, own.dim, own.vdim) != (other.kv_heads, other.dim, other.vdim):
                        raise InvalidInput(f"config.json {where}.mixer: keys and values of layer {source} have other sizes")
            elif kind == "mingru":
                sizes = LayerSizes(kind, gru_width=_int(mixer, "width", where + ".mixer"))
            else:
                raise Unsupported(f"config.json {where}.type {kind!r}; this design has the mixers {', '.join(MIXERS)}")
            if mlp is not None:
                form = _get(mlp, "kind", where + ".mlp")
                if form == "dense":
                    sizes.ff = _int(mlp, "ff", where + ".mlp")
                elif form == "moe":
                    router = _get(mlp, "router", where + ".mlp")
                    sizes.router = RouterSizes(
                        _int(router, "experts", where + ".mlp.router"), _int(router, "top", where + ".mlp.router"),
                        _int(router, "identity", where + ".mlp.router", least=0) if router.get("identity") is not None else 0,
                        _int(_get(mlp, "expert", where + ".mlp"), "ff", where + ".mlp.expert"))
                    if sizes.router.top > sizes.router.experts + sizes.router.identity:
                        raise InvalidInput(f"config.json {where}.mlp.router: the {sizes.router.top} largest of "
                                           f"{sizes.router.experts + sizes.router.identity} outputs")
                else:
                    raise Unsupported(f"config.json {where}.mlp.kind {form!r}; this design has dense and moe feed-forwards")
            out_layers.append(sizes)
        embedding = raw.get("embedding") or {}
        return cls(
            vocab=_int(raw, "vocab", "file"), width=_int(raw, "width", "file"), eps=_number(_get(raw, "norm", "file"), "eps", "norm"),
            embedding_scale=_number(embedding, "scale", "embedding") if embedding.get("scale") is not None else 1.0,
            layers=out_layers, raw=copy.deepcopy(raw))

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)
