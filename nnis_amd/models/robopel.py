"""Robopel as a model description.  A decoder whose sublayers read the
residual stream as it is and are normed on their way out only (RMS norm with a
weight stored around zero); whose mixers are a minGRU (``mingru``) or grouped
attention with normed and rotated queries and keys, capped scores, a sliding
window with pooled blocks, a learned sink and a sigmoid gate on the heads
(``attention``), which may read an earlier layer's keys and values instead of
keeping its own; whose feed-forward is dense with a PolyNorm activation, a
mixture of experts with identity outputs, or absent; whose embedding is
scaled.  Tensor names are the checkpoint's: layer i's start with ``l<i>.``.
"""

from __future__ import annotations

from ..config.robopel import RobopelConfig
from .spec import ModelSpec, ScheduleEntry


def _norm(cfg: RobopelConfig, name: str):
    return {"kind": "rms", "width": cfg.width, "eps": cfg.eps, "weight": name, "offset": 1.0}


def _attention(cfg: RobopelConfig, prefix: str, sizes, position, source):
    out = {
        "kind": "gated_window_attention", "width": cfg.width, "heads": sizes.heads, "kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "value_dim": sizes.vdim, "scale": sizes.scale, "eps": cfg.eps, "softcap": sizes.softcap or None, "window": sizes.window or None,
        "pool": sizes.pool or None, "position": position, "q": prefix + "q", "o": prefix + "o", "gate": prefix + "g",
        "q_norm": prefix + "q.norm", "sink": prefix + "sink",
    }
    if source is None:
        out.update(k=prefix + "k", v=prefix + "v", k_norm=prefix + "k.norm")
    else:
        out.update(own_kv=False, source_pool=source.pool or None)
    return out


def _feed_forward(cfg: RobopelConfig, prefix: str, layer):
    if layer.ff is not None:
        return {"kind": "poly_norm", "width": cfg.width, "inner": layer.ff, "eps": cfg.eps, "up": prefix + "up",
                "down": prefix + "down", "act": prefix + "act"}
    router = layer.router
    return {"kind": "routed", "width": cfg.width, "inner": router.expert_ff, "experts": router.experts, "top": router.top,
            "identity": router.identity, "router": prefix + "router", "correction": prefix + "correction",
            "up": prefix + "e{}.up", "down": prefix + "e{}.down"}


def robopel_spec(cfg: RobopelConfig) -> ModelSpec:
    positions, layers, schedule = {}, [], []
    for index, layer in enumerate(cfg.layers):
        prefix = f"l{index}."
        source = None
        if layer.type == "attention":
            sizes, position = layer.attention, None
            if sizes.rot_dims:
                # rotations that agree in size, base and bending share their tables
                bend = None if sizes.rot_scaling is None else sizes.rot_scaling.key()
                position = f"pairs_{sizes.rot_dims}_{sizes.rot_base!r}_{bend!r}"
                positions.setdefault(position, {"kind": "rotary_pairs", "rot_dim": sizes.rot_dims, "theta": sizes.rot_base,
                                                "max_positions": None, "angles": "float64", "scaling": bend})
            source = sizes.kv_from
            mixer = _attention(cfg, prefix + "mix.", sizes, position, None if source is None else cfg.layers[source].attention)
        else:
            mixer = {"kind": "min_gru", "width": cfg.width, "channels": layer.gru_width, "z": prefix + "mix.z",
                     "z_bias": prefix + "mix.z.b", "x": prefix + "mix.x", "x_bias": prefix + "mix.x.b", "g": prefix + "mix.g",
                     "o": prefix + "mix.o"}
        block = {"kind": "post_norm", "width": cfg.width, "norm1": _norm(cfg, prefix + "norm1"), "mixer": mixer}
        if layer.ff is not None or layer.router is not None:
            block.update(norm2=_norm(cfg, prefix + "norm2"), feed_forward=_feed_forward(cfg, prefix + "mlp.", layer))
        layers.append(block)
        schedule.append(ScheduleEntry(layer=index, reads_cache_of=source))  # (every layer runs once: entry i is layer i)
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=None,  # the design names no last position
        stored_dtype="bfloat16",
        embedding={"kind": "table", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "embed", "scale": cfg.embedding_scale},
        positions=positions,
        layers=layers,
        schedule=schedule,
        final_norm=_norm(cfg, "final.norm"),
        head={"kind": "linear", "vocab_size": cfg.vocab, "width": cfg.width, "weight": "head", "tied_to": None},
        stop_token_ids=(),
        config_json=cfg.to_dict(),
    )
    spec.validate()
    return spec
