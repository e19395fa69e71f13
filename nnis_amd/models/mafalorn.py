"""Mafalorn as a model description.  A decoder whose layers norm every
sublayer on the way in and on the way out with RMS norms; whose mixers are
retention (linear attention with one fixed decay a head, rotated queries and
keys and no softmax), two mixers side by side whose outputs are added with a
factor each (grouped causal attention whose values are its keys as projected,
with frequencies scaled over a ramp and a sigmoid gate a head, beside the
gated delta rule behind short convolutions), or attention over a cached
latent in a sliding window with a rotated key part and a gate element by
element; whose feed-forward is a mixture of SiLU-gated experts with identity
outputs, chosen among the best groups; whose logits are scaled.  Tensor names
are the checkpoint's: layer i's start with ``l<i>.``.
"""

from __future__ import annotations

from ..config.mafalorn import MafalornConfig
from .spec import ModelSpec, ScheduleEntry


def _norm(cfg: MafalornConfig, name: str):
    return {"kind": "rms", "width": cfg.width, "eps": cfg.eps, "weight": name}


def _rotation(positions, rot, kind):
    """The name of the position encoding of a rotation; rotations that agree in everything share their tables."""
    if rot is None:
        return None
    name = f"{kind}_{rot.dims}_{rot.base!r}_{rot.ramp!r}"
    positions.setdefault(name, {"kind": "rotary_" + kind, "rot_dim": rot.dims, "theta": rot.base, "max_positions": None,
                                "angles": "float64", "ramp": rot.ramp})
    return name


def _retention(cfg, prefix, sizes, positions):
    return {"kind": "retention", "width": cfg.width, "heads": sizes.heads, "key_dim": sizes.dim, "value_dim": sizes.vdim,
            "decay": list(sizes.decay), "eps": cfg.eps, "position": _rotation(positions, sizes.rot, "half"),
            "q": prefix + "q", "k": prefix + "k", "v": prefix + "v", "g": prefix + "g", "o": prefix + "o"}


def _parallel(cfg, prefix, layer, positions):
    left, right = layer.left, layer.right
    softmax = {"kind": "causal_attention", "width": cfg.width, "heads": left.heads, "kv_heads": left.kv_heads, "head_dim": left.dim,
               "scale": left.scale, "position": _rotation(positions, left.rot, "half"), "values_from_keys": True,
               "head_gate": prefix + "left.g", "q": prefix + "left.q", "k": prefix + "left.k", "v": None, "o": prefix + "left.o"}
    r = prefix + "right."
    delta = {"kind": "gated_delta_rule", "width": cfg.width, "heads": right.heads, "qk_heads": right.kv_heads, "key_dim": right.dim,
             "value_dim": right.vdim, "taps": right.conv, "eps": cfg.eps, "q": r + "q", "k": r + "k", "v": r + "v",
             "q_conv": r + "q.conv", "k_conv": r + "k.conv", "v_conv": r + "v.conv", "b": r + "b", "a": r + "a", "a_log": r + "A_log",
             "dt_bias": r + "dt_bias", "norm": r + "norm", "g": r + "g", "o": r + "o"}
    return {"kind": "side_by_side", "width": cfg.width, "eps": cfg.eps, "branches": [softmax, delta],
            "scales": [layer.left_scale, layer.right_scale]}


def _latent(cfg, prefix, sizes, positions):
    position = None
    if sizes.rot_dim:
        position = f"pairs_{sizes.rot_dim}_{sizes.rot_base!r}_None"
        positions.setdefault(position, {"kind": "rotary_pairs", "rot_dim": sizes.rot_dim, "theta": sizes.rot_base,
                                        "max_positions": None, "angles": "float64"})
    return {"kind": "latent_attention", "width": cfg.width, "heads": sizes.heads, "key_dim": sizes.dim, "value_dim": sizes.vdim,
            "q_rank": None, "kv_rank": sizes.kv_rank, "scale": sizes.scale, "eps": cfg.eps, "q": prefix + "q", "dkv": prefix + "dkv",
            "dkv_norm": prefix + "dkv.norm", "uk": prefix + "uk", "uv": prefix + "uv", "o": prefix + "o",
            "rot_dim": sizes.rot_dim, "position": position, "window": sizes.window or None, "channel_gate": prefix + "g"}


def _feed_forward(cfg, prefix, router):
    return {"kind": "routed", "width": cfg.width, "inner": router.expert_ff, "experts": router.experts, "top": router.top,
            "identity": router.identity, "groups": router.groups, "activation": "silu_gated", "router": prefix + "router",
            "correction": prefix + "correction", "gate": prefix + "e{}.gate", "up": prefix + "e{}.up", "down": prefix + "e{}.down"}


def mafalorn_spec(cfg: MafalornConfig) -> ModelSpec:
    positions, layers = {}, []
    for index, layer in enumerate(cfg.layers):
        prefix = f"l{index}."
        if layer.type == "retention":
            mixer = _retention(cfg, prefix + "mix.", layer.retention, positions)
        elif layer.type == "parallel":
            mixer = _parallel(cfg, prefix + "mix.", layer, positions)
        else:
            mixer = _latent(cfg, prefix + "mix.", layer.latent, positions)
        block = {"kind": "pre_post_norm", "width": cfg.width, "norm1": _norm(cfg, prefix + "norm1"),
                 "post1": _norm(cfg, prefix + "norm1b"), "mixer": mixer}
        if layer.router is not None:
            block.update(norm2=_norm(cfg, prefix + "norm2"), post2=_norm(cfg, prefix + "norm2b"),
                         feed_forward=_feed_forward(cfg, prefix + "mlp.", layer.router))
        layers.append(block)
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=None,  # the design names no last position
        stored_dtype="bfloat16",
        embedding={"kind": "table", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "embed"},
        positions=positions,
        layers=layers,
        schedule=[ScheduleEntry(layer=index) for index in range(len(layers))],
        final_norm=_norm(cfg, "final.norm"),
        head={"kind": "linear", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "head", "tied_to": None,
              "scale": None if cfg.logit_scale == 1.0 else cfg.logit_scale},
        stop_token_ids=(),
        config_json=cfg.to_dict(),
    )
    spec.validate()
    return spec
