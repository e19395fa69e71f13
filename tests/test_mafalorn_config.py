"""Mafalorn on the CPU: its configuration reader, its model description, the
cache it asks for, the rotation tables with frequencies scaled over a ramp,
and the plain implementation's own mechanisms against special cases."""

import copy
import math

import pytest
import torch

import nnis_amd
import plain_mafalorn as P
from nnis_amd.config.registry import spec_from_config
from nnis_amd.errors import InvalidInput, Unsupported
from nnis_amd.models.decoder import DecoderModel
from nnis_amd.parts.base import KVRequest, StateRequest
from nnis_amd.parts.rope import rotary_tables
from mafalorn_configs import MAF_A, MAF_B, MAF_C, delta, latent, layer, mafalorn, moe, parallel, retention, softmax


def test_the_architecture_is_chosen_by_its_name():
    cfg, spec = spec_from_config(MAF_A)
    assert spec.architecture == "Mafalorn" and spec.width == 96 and spec.vocab_size == 300 and spec.max_positions is None
    assert "Mafalorn" in nnis_amd.config.registered_architectures()
    assert cfg.logit_scale == 0.7 and spec.head["scale"] == 0.7
    assert spec_from_config(MAF_B)[0].logit_scale == 1.0 and spec_from_config(MAF_B)[1].head["scale"] is None
    with pytest.raises(Unsupported):
        spec_from_config(dict(MAF_A, architecture="Mafalorn2"))


def test_layers_and_their_parts():
    kinds = {"retention": "retention", "parallel": "side_by_side", "latent_attention": "latent_attention"}
    for config in (MAF_A, MAF_B, MAF_C):
        _, spec = spec_from_config(config)
        assert [entry.layer for entry in spec.schedule] == list(range(len(config["layers"])))
        for raw, block in zip(config["layers"], spec.layers):
            assert block["kind"] == "pre_post_norm" and block["norm1"]["kind"] == block["post1"]["kind"] == "rms"
            assert ("feed_forward" in block) == (raw["mlp"] is not None) == ("post2" in block)
            assert block["mixer"]["kind"] == kinds[raw["type"]]
            if raw["mlp"] is not None:
                assert block["feed_forward"]["kind"] == "routed" and block["feed_forward"]["activation"] == "silu_gated"
    _, spec = spec_from_config(MAF_A)
    side = spec.layers[0]["mixer"]
    assert side["scales"] == [0.6, 1.3] and [b["kind"] for b in side["branches"]] == ["causal_attention", "gated_delta_rule"]
    assert side["branches"][0]["values_from_keys"] and side["branches"][0]["v"] is None
    assert spec.layers[0]["feed_forward"]["groups"] == (4, 2) and spec.layers[3]["feed_forward"]["groups"] is None
    assert spec.layers[3]["mixer"]["position"] is None and len(spec.positions) == 3  # scaled halves, plain halves, pairs
    assert spec.positions[side["branches"][0]["position"]]["ramp"] == (4.0, 64.0, 8.0, 1.0)
    names = {t.name: t.shape for t in DecoderModel(spec).tensors()}
    assert names["l0.mix.left.q"] == (128, 96) and names["l0.mix.left.k"] == (64, 96) and names["l0.mix.left.g"] == (4, 96)
    assert "l0.mix.left.v" not in names and names["l0.mix.right.q.conv"] == (32, 3) and names["l0.mix.right.v"] == (96, 96)
    assert names["l0.mix.right.A_log"] == (4,) and names["l0.mix.right.norm"] == (24,) and names["l0.mix.right.b"] == (4, 96)
    assert names["l0.mlp.router"] == (8, 96) and names["l0.mlp.correction"] == (8,) and names["l0.mlp.e5.gate"] == (24, 96)
    assert "l0.mlp.e6.up" not in names and names["l1.mix.g"] == (96, 96) and names["l1.norm2b"] == (96,)
    assert names["l2.mix.q"] == (4 * 24, 96) and names["l2.mix.dkv"] == (48, 96) and names["l2.mix.uk"] == (64, 40)
    assert names["l2.mix.uv"] == (96, 40) and names["l2.mix.g"] == (96, 96) and names["l2.mix.o"] == (96, 96)
    assert not any(name.startswith("l2.mlp") or name.startswith("l2.norm2") for name in names)


def test_missing_and_wrong_keys_are_refused():
    for path in (["vocab"], ["norm", "eps"], ["layers", 0, "mixer", "left"], ["layers", 0, "mixer", "left", "scale"],
                 ["layers", 0, "mixer", "left", "rot", "base"], ["layers", 0, "mixer", "left", "rot", "scaling", "fast"],
                 ["layers", 0, "mixer", "right", "conv"], ["layers", 0, "mixer", "right_scale"], ["layers", 0, "mlp", "router", "top"],
                 ["layers", 0, "mlp", "router", "groups", "keep"], ["layers", 0, "mlp", "expert"], ["layers", 1, "mixer", "decay"],
                 ["layers", 1, "mixer", "vdim"], ["layers", 2, "mixer", "kv_rank"], ["layers", 2, "mixer", "rot"], ["layers", 2, "mixer", "mask", "size"]):
        raw = copy.deepcopy(MAF_A)
        at = raw
        for key in path[:-1]:
            at = at[key]
        del at[path[-1]]
        with pytest.raises(InvalidInput):
            spec_from_config(raw)
    for change, error in ((lambda raw: raw["layers"][1].update(type="attention"), Unsupported),
                          (lambda raw: raw["layers"][0]["mlp"].update(kind="dense"), Unsupported),
                          (lambda raw: raw["layers"][1]["mixer"].update(decay=[0.5, 0.5]), InvalidInput),  # one decay a head
                          (lambda raw: raw["layers"][1]["mixer"].update(decay=[0.5, 0.5, 1.5]), InvalidInput),
                          (lambda raw: raw["layers"][0]["mixer"]["left"].update(vdim=16), InvalidInput),  # the values are the keys
                          (lambda raw: raw["layers"][0]["mixer"]["left"].update(heads=5), InvalidInput),
                          (lambda raw: raw["layers"][0]["mixer"]["right"].update(kv_heads=3), InvalidInput),
                          (lambda raw: raw["layers"][0]["mixer"]["left"]["rot"].update(dims=34), InvalidInput),
                          (lambda raw: raw["layers"][2]["mixer"]["rot"].update(dims=4), InvalidInput),  # all of rot_dim is turned
                          (lambda raw: raw["layers"][0]["mlp"]["router"]["groups"].update(count=3), InvalidInput),  # 8 outputs
                          (lambda raw: raw["layers"][0]["mlp"]["router"]["groups"].update(keep=5), InvalidInput),
                          (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=4), InvalidInput),  # one group of 3 is kept
                          (lambda raw: raw["layers"][3]["mlp"]["router"].update(top=4), InvalidInput)):
        raw = copy.deepcopy(MAF_A)
        change(raw)
        with pytest.raises(error):
            spec_from_config(raw)


def test_what_the_file_does_not_mention_does_not_exist():
    bare = mafalorn(vocab=50, width=32, layers=[{"type": "retention", "mixer": retention(2, 8, 8, (0.9, 0.8))}])  # no "mlp" at all
    cfg, spec = spec_from_config(bare)
    assert "feed_forward" not in spec.layers[0] and spec.layers[0]["mixer"]["position"] is None and not spec.positions
    assert cfg.logit_scale == 1.0
    config = mafalorn(vocab=50, width=32, layers=[
        layer("latent_attention", {k: v for k, v in latent(2, 8, 0, 8, 16).items() if k not in ("rot", "rot_dim")}, moe(3, 2, 8)),
        layer("parallel", parallel(softmax(2, 1, 16), delta(2, 1, 8, 8, 2)))])
    cfg, spec = spec_from_config(config)
    assert (cfg.layers[0].latent.rot_dim, cfg.layers[0].latent.window) == (0, 0) and cfg.layers[0].router.identity == 0
    assert cfg.layers[0].router.groups is None and cfg.layers[1].left.rot is None and not spec.positions
    assert spec.layers[0]["mixer"]["window"] is None and spec.layers[0]["mixer"]["position"] is None
    assert dict(DecoderModel(spec).cache_requests()[0])[0] == KVRequest(1, 16, None, None)


def test_the_cache_it_asks_for():
    """Retention and the delta rule keep a 32-bit matrix a head, the delta rule also its convolution's last inputs; the
    softmax side keeps keys and values of one size; a latent is one key/value head whose values are narrower than its
    keys by the rotated part, in a window's group where it has one."""
    requests, shared = DecoderModel(spec_from_config(MAF_A)[1]).cache_requests()
    assert shared == {}
    assert requests == [(0, (KVRequest(2, 32, None, None), (StateRequest((4, 24, 16)), StateRequest((2, 2 * 2 * 16 + 4 * 24))))),
                        (1, StateRequest((3, 16, 32))), (2, KVRequest(1, 48, 37, 40)), (3, StateRequest((2, 24, 8)))]
    requests, _ = DecoderModel(spec_from_config(MAF_C)[1]).cache_requests()
    assert dict(requests)[1] == KVRequest(1, 32, None, 24)


def test_frequencies_scaled_over_a_ramp():
    """Pairs below the ramp keep their frequency, pairs above it are divided by the factor, those on it are blended;
    cosine and sine carry the factor 0.1 ln(factor) + 1."""
    rot = {"dims": 32, "base": 1e4, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    f, magnitude = P.frequencies(rot)
    plain = [1e4 ** (-2.0 * i / 32) for i in range(16)]
    lo = math.floor(32 * math.log(64 / (2 * math.pi * 8.0)) / (2 * math.log(1e4)))
    hi = math.ceil(32 * math.log(64 / (2 * math.pi * 1.0)) / (2 * math.log(1e4)))
    assert 0 <= lo < hi < 15 and abs(magnitude - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    for i in range(16):
        if i <= lo:
            assert f[i] == plain[i]
        elif i >= hi:
            assert abs(f[i] - plain[i] / 4.0) < 1e-15
        else:
            assert plain[i] / 4.0 < f[i] < plain[i]
    cos, sin = rotary_tables(70, 32, 1e4, "float64", ramp=(4.0, 64, 8.0, 1.0))
    angle = torch.arange(70, dtype=torch.float64)[:, None] * f[None, :]
    assert torch.allclose(cos.double(), torch.cos(angle) * magnitude, atol=1e-6) and torch.allclose(sin.double(), torch.sin(angle) * magnitude, atol=1e-6)
    with pytest.raises(InvalidInput):
        rotary_tables(8, 32, 1e4, "float32", ramp=(4.0, 64, 8.0, 1.0))
    # a ramp that no pair reaches (its feet beyond the last pair) leaves the frequencies as they are but for the factor on the tables
    f2, _ = P.frequencies({"dims": 8, "base": 1e4, "scaling": {"factor": 2.0, "original": 1e9, "fast": 1.0, "slow": 0.5}})
    assert [float(v) for v in f2] == [1e4 ** (-2.0 * i / 8) for i in range(4)]


def test_the_plain_mechanisms_against_special_cases():
    g = torch.Generator().manual_seed(0)
    # retention with a decay of one and no rotation is a running sum of outer products
    h = torch.randn(6, 8, generator=g, dtype=torch.float64)
    w = {k: torch.randn(s, generator=g, dtype=torch.float64) for k, s in (("q", (4, 8)), ("k", (4, 8)), ("v", (6, 8)), ("g", (6, 8)), ("o", (8, 6)))}
    _, state = P.retention(h, w, {"heads": 1, "dim": 4, "vdim": 6, "decay": [1.0]}, 1e-6)
    k, v = (h @ w["k"].T) * 0.5, h @ w["v"].T
    assert torch.allclose(state[0], k.T @ v)
    # the delta rule with beta = 1 and g = 1 stores v under a unit key: reading with the same key returns it
    S = torch.zeros(4, 3, dtype=torch.float64)
    key, value = torch.tensor([0.6, 0.8, 0.0, 0.0], dtype=torch.float64), torch.tensor([1.0, -2.0, 3.0], dtype=torch.float64)
    S = S + key[:, None] * (value - S.T @ key)[None, :]
    assert torch.allclose(S.T @ key, value)
    # groups: with one of two groups kept, the chosen outputs lie in the group of the largest corrected score
    s = torch.tensor([0.05, 0.30, 0.05, 0.10, 0.25, 0.25], dtype=torch.float64)
    assert P.chosen_outputs(s, torch.zeros(6, dtype=torch.float64), 2, {"count": 2, "keep": 1}) == [1, 0]
    assert P.chosen_outputs(s, torch.zeros(6, dtype=torch.float64), 2, None) == [1, 4]
    correction = torch.tensor([0.0, -0.5, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)  # negative corrected scores still beat a closed group
    assert P.chosen_outputs(s, correction, 3, {"count": 3, "keep": 1}) == [4, 5]
    assert P.chosen_outputs(s, correction - 1.0, 2, {"count": 2, "keep": 1}) == [4, 5]
    # a short convolution of one tap is a scaling; of two taps it reads the token before
    x = torch.arange(8, dtype=torch.float64).view(4, 2)
    assert torch.equal(P.short_convolution(x, torch.tensor([[2.0], [3.0]], dtype=torch.float64)), x * torch.tensor([2.0, 3.0], dtype=torch.float64))
    two = P.short_convolution(x, torch.tensor([[1.0, 0.0], [1.0, 0.0]], dtype=torch.float64))
    assert torch.equal(two[1:], x[:-1]) and torch.equal(two[0], torch.zeros(2, dtype=torch.float64))


def test_a_random_model_is_written_and_read(tmp_path):
    folder = str(tmp_path / "m")
    nnis_amd.write_random_model(folder, MAF_B, 5)
    plain = P.PlainMafalorn(folder)
    logits = plain.logits([3, 1, 4, 1, 5, 9, 2, 6])
    assert logits.shape == (8, 257) and bool(torch.isfinite(logits).all())
    streams = []
    plain.logits([3, 1, 4], stream_after=streams)
    assert len(streams) == 3 and torch.allclose(plain.logits([3, 1, 4, 1, 5, 9, 2, 6])[:3], plain.logits([3, 1, 4]))
