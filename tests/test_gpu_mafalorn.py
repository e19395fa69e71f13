"""Mafalorn on the GPU against the plain implementation (``plain_mafalorn``):
each mechanism alone, then whole models through the engine -- prompts whole, in
portions and token by token, unequal batches, slots, pages and states used
again, keys far away, at page borders and at the edges of a window, the first
tokens, long decoding, greedy generation through the library's entry point,
the trace runner.  32-bit is held to rounding; bfloat16 to the error of the
plain model run with its activations rounded where the engine rounds them.
"""

import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import nnis_amd
import plain_mafalorn as P
import replay
from gpu_helpers import cache_for, context, runtime
from mafalorn_configs import MAFALORN_CONFIGS, delta, latent, layer, mafalorn, moe, parallel, retention, softmax

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
CUTS = ([[200], [3], [67]], [[61, 63, 64, 66, 128, 130, 131, 200], [1, 2, 3], [2, 4, 64, 65, 66, 67]],
        [[150] + list(range(151, 201)), [3], [60] + list(range(61, 68))])


def _relative(got, want):
    got, want = torch.as_tensor(np.asarray(got)).double(), torch.as_tensor(np.asarray(want)).double()
    return float((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-30))


def _close(got, want, dtype, what="", bf16=3e-2, f32=3e-5):
    error = _relative(got.detach().float().cpu() if isinstance(got, torch.Tensor) else got, want)
    bound = f32 if dtype == "float32" else bf16
    assert error <= bound, f"{what}: relative error {error:.3g} (bound {bound:.3g})"


def _weights(part, dtype, seed, scale=None):
    """Random tensors for a part, by its own declarations: (for the plain functions in 64-bit, for the part)."""
    from nnis_amd.weights.random_init import _INIT_RULES

    generator = torch.Generator().manual_seed(seed)
    stored = {}
    for t in part.tensors():
        value = _INIT_RULES[t.init](t, generator, torch.bfloat16)
        for ending, factor in (scale or {}).items():
            if t.name == ending or t.name.endswith("." + ending):
                value = (value.float() * factor).to(torch.bfloat16)
        stored[t.name] = value
    wide = torch.float32 if dtype == "float32" else torch.bfloat16
    return {n: v.double() for n, v in stored.items()}, {n: v.to(wide).cuda() for n, v in stored.items()}


def _run_in_steps(forward, cache, rt, xs, cuts):
    """Runs sequences through ``forward(x, ctx)``, all of them in every step; ``cuts[i]`` lists where sequence i's portions end."""
    slots = [cache.acquire() for _ in xs]
    done = [0] * len(xs)
    outs = [[] for _ in xs]
    cuts = [list(c) for c in cuts]
    while any(cuts):
        batch = [i for i in range(len(xs)) if cuts[i]]
        ends = [cuts[i].pop(0) for i in batch]
        ctx = context(cache, [(slots[i], end - done[i]) for i, end in zip(batch, ends)])
        x = torch.cat([xs[i][done[i]:end] for i, end in zip(batch, ends)]).to(rt.dtype).cuda()
        y = forward(x, ctx)
        row = 0
        for i, end in zip(batch, ends):
            outs[i].append(y[row:row + end - done[i]].float().cpu())
            row += end - done[i]
            done[i] = end
    for slot in slots:
        cache.release(slot)
    return [torch.cat(o) for o in outs]


def _positions(descriptions, rt, reach=1024):
    from nnis_amd.parts import build_part

    out = {}
    for name, description in descriptions.items():
        out[name] = build_part("position", description)
        out[name].bind({}, rt)
        out[name].reach(reach)
    return out


def _rounding(dtype):
    return P.identity if dtype == "float32" else P.bf16_round


def _inputs(lengths, width, seed=5):
    generator = torch.Generator().manual_seed(seed)
    return [torch.randn(n, width, generator=generator).to(torch.bfloat16).double() for n in lengths]


# ---------------------------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, width", [(1, 8), (37, 50), (5, 1030), (9, 2048), (3, 4096), (2, 4104), (300, 96)])
def test_the_step_between_two_sublayers(y_dtype, tokens, width):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(tokens + width)
    x = torch.randn(tokens, width, generator=generator)
    y = (3.0 * torch.randn(tokens, width, generator=generator)).to(y_dtype)
    w_out, w_in = 1.0 + 0.3 * torch.randn(width, generator=generator), 1.0 + 0.3 * torch.randn(width, generator=generator)
    stream_want = x.double() + P.rms_norm(y.double(), w_out.double(), 1e-5)
    rows_want = P.rms_norm(stream_want, w_in.double(), 1e-5)
    stream, rows = x.clone().cuda(), torch.empty(tokens, width, device="cuda", dtype=y_dtype)
    ops.rms_between(stream, y.cuda(), w_out.cuda(), w_in.cuda(), 1e-5, h=rows)
    assert _relative(stream.cpu(), stream_want) < 1e-6 and _relative(rows.float().cpu(), rows_want) < (1e-6 if y_dtype == torch.float32 else 4e-3)
    stream = x.clone().cuda()
    ops.rms_between(stream, y.cuda(), w_out.cuda(), None, 1e-5)  # no rows asked for
    assert _relative(stream.cpu(), stream_want) < 1e-6
    # a share of other rows joins y before the norm
    keep = torch.rand(tokens, generator=generator)
    rows_in = torch.randn(tokens, width, generator=generator).to(y_dtype)
    stream_want = x.double() + P.rms_norm(y.double() + keep.double()[:, None] * rows_in.double(), w_out.double(), 1e-5)
    stream = x.clone().cuda()
    ops.rms_between(stream, y.cuda(), w_out.cuda(), w_in.cuda(), 1e-5, h=rows, share=(keep.cuda(), rows_in.cuda()))
    assert _relative(stream.cpu(), stream_want) < 1e-6
    assert _relative(rows.float().cpu(), P.rms_norm(stream_want, w_in.double(), 1e-5)) < (1e-6 if y_dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, heads, n, k", [(1, 1, 8, 8), (3, 4, 24, 40), (70, 3, 16, 48), (300, 2, 40, 24), (5, 6, 33, 130)])
def test_a_map_of_its_own_for_every_head(dtype, tokens, heads, n, k):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(tokens + n)
    x = torch.randn(tokens, heads * k, generator=generator).to(dtype)
    w = torch.randn(heads, n, k, generator=generator).to(dtype)
    gate = torch.rand(tokens, heads * n, generator=generator)
    want = torch.einsum("hnk,thk->thn", w.double(), x.double().view(tokens, heads, k)).reshape(tokens, heads * n)
    got = ops.heads_linear(x.cuda(), w.cuda(), None, heads, torch.empty(tokens, heads * n, device="cuda", dtype=dtype))
    assert _relative(got.float().cpu(), want) < (2e-6 if dtype == torch.float32 else 4e-3)
    got = ops.heads_linear(x.cuda(), w.cuda(), gate.cuda(), heads, torch.empty(tokens, heads * n, device="cuda", dtype=dtype))
    assert _relative(got.float().cpu(), want * gate.double()) < (2e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_branches_added_with_a_factor_each_and_scaled_logits(dtype):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(1)
    ys = [torch.randn(37, 50, generator=generator).to(dtype) for _ in range(3)]
    got = ops.branch_sum([y.cuda() for y in ys], [0.8, -0.5, 2.0], torch.empty(37, 50, device="cuda", dtype=dtype))
    want = 0.8 * ys[0].double() - 0.5 * ys[1].double() + 2.0 * ys[2].double()
    assert _relative(got.float().cpu(), want) < (1e-6 if dtype == torch.float32 else 4e-3)
    logits = torch.randn(5, 300, generator=generator)
    assert torch.equal(ops.scale_rows(logits.clone().cuda(), 0.5).cpu(), logits * 0.5)


@pytest.mark.parametrize("experts, identity, top, count, keep", [(6, 2, 3, 4, 2), (5, 1, 2, 2, 1), (12, 4, 4, 4, 2), (3, 3, 3, 3, 3), (8, 0, 3, 4, 2),
                                                                 (60, 4, 6, 32, 4), (9, 3, 4, 3, 1), (4, 0, 2, 1, 1)])
def test_the_router_chooses_among_the_best_groups(experts, identity, top, count, keep):
    """The correction decides who is chosen and is negative for many outputs (a closed group counts as minus infinity,
    not as zero); the weights are the scores without it, not renormalised; the identity outputs' weights are summed
    apart.  Logits and choice in one kernel give the same."""
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(experts)
    n, rows, width = experts + identity, 40, 24
    x = torch.randn(rows, width, generator=generator)
    w = torch.randn(n, width, generator=generator)
    logits = x @ w.T
    correction = 0.5 * torch.randn(n, generator=generator) - 0.4
    groups = {"count": count, "keep": keep}
    scores = torch.softmax(logits.double(), dim=-1)
    want = torch.zeros(rows, n, dtype=torch.float64)
    closed_matter = False
    for r in range(rows):
        chosen = P.chosen_outputs(scores[r], correction.double(), top, groups)
        closed_matter |= chosen != P.chosen_outputs(scores[r], correction.double(), top, None)
        want[r, chosen] = scores[r, chosen]
    assert closed_matter or keep == count  # (fewer groups are kept than outputs chosen: a closed group costs somebody a place)
    for fused in (False, True):
        gates, kept = torch.empty(rows, experts, device="cuda"), torch.empty(rows, device="cuda")
        if fused:
            ops.route(x.cuda(), w.cuda(), correction.cuda(), experts, top, gates, kept, groups=(count, keep))
        else:
            ops.route_top(logits.cuda(), correction.cuda(), experts, top, gates, kept, groups=(count, keep))
        close = ((gates.cpu().double() - want[:, :experts]).abs().max(dim=1).values < 1e-5) & ((kept.cpu().double() - want[:, experts:].sum(dim=1)).abs() < 1e-5)
        assert float(close.double().mean()) > (0.97 if fused else 0.999)  # (a choice may differ where two sums round apart)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, inner, experts, top, identity, groups", [(64, 24, 6, 2, 2, (4, 2)), (48, 40, 3, 1, 0, None), (96, 16, 12, 3, 4, (4, 3)),
                                                                         (40, 9, 2, 3, 1, None), (56, 8, 5, 2, 1, (2, 1))])
def test_routed_feed_forward_alone(dtype, width, inner, experts, top, identity, groups):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    part = build_part("feed_forward", dict(kind="routed", width=width, inner=inner, experts=experts, top=top, identity=identity, groups=groups,
                                           activation="silu_gated", router="router", correction="correction", gate="e{}.gate", up="e{}.up",
                                           down="e{}.down"))
    plain_w, part_w = _weights(part, dtype, 3, scale={"router": 4.0, "correction": 0.5, "gate": 8.0, "up": 8.0, "down": 8.0})
    part.bind(part_w, rt)
    x = _inputs([70], width)[0]
    router = {"experts": experts, "top": top, "identity": identity}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    want = P.experts(x, plain_w, {"router": router}, _rounding(dtype))
    got = part.forward(x.to(rt.dtype).cuda(), None, rt)
    _close(got, want, dtype, "routed feed-forward")
    y, (keep, rows) = part.forward(x.to(rt.dtype).cuda(), None, rt, share_later=True) if identity else (got, (None, None))
    if identity:
        assert float(keep.max()) > 0.05  # identity outputs are chosen
        _close(y.float() + keep[:, None] * rows.float(), want, dtype, "routed feed-forward, the share apart")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim, decay, rot, width", [(3, 16, 32, (0.9, 0.97, 0.995), (8, 1e4), 64), (2, 24, 8, (1.0, 0.5), None, 48),
                                                                 (4, 16, 16, (0.75, 0.9, 0.99, 0.999), (16, 50.0), 40), (1, 40, 72, (0.98,), (40, 1e6), 56)])
def test_retention_alone(dtype, heads, dim, vdim, decay, rot, width):
    """Whole prompts (one long enough to be cut into pieces that run side by side), portions down to two tokens, single
    tokens; three unequal sequences in every step, their states apart."""
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    sizes = retention(heads, dim, vdim, decay, rot)
    positions = _positions({"r": {"kind": "rotary_half", "rot_dim": rot[0], "theta": rot[1], "max_positions": None, "angles": "float64"}}, rt) if rot else {}
    mixer = build_part("mixer", dict(kind="retention", width=width, heads=heads, key_dim=dim, value_dim=vdim, decay=decay, eps=1e-5,
                                     position="r" if rot else None, q="q", k="k", v="v", g="g", o="o"), positions=positions)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 6.0, "k": 6.0, "v": 6.0, "g": 12.0, "o": 5.0})
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    lengths = [200, 3, 67]
    xs = _inputs(lengths, width)
    want = [P.retention(x, plain_w, sizes, 1e-5, _rounding(dtype))[0] for x in xs]
    for cuts in CUTS:
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"retention {cuts[0][:2]} length {n}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_retention_reads_a_key_from_far_back(dtype):
    """One head with a decay close to one whose queries and keys read marked channels: the token marked hundreds of
    positions back decides the last token's output, at the first positions, at a page's border and beyond, and the
    rotation has turned it by its distance."""
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    width, dim, vdim, n = 32, 16, 16, 700
    sizes = retention(1, dim, vdim, (0.9995,), (16, 300.0))
    positions = _positions({"r": {"kind": "rotary_half", "rot_dim": 16, "theta": 300.0, "max_positions": None, "angles": "float64"}}, rt)
    mixer = build_part("mixer", dict(kind="retention", width=width, heads=1, key_dim=dim, value_dim=vdim, decay=(0.9995,), eps=1e-5, position="r",
                                     q="q", k="k", v="v", g="g", o="o"), positions=positions)
    plain_w, part_w = _weights(mixer, dtype, 11, scale={"v": 20.0, "o": 20.0, "g": 20.0})
    reads = {"q": torch.zeros(dim, width, dtype=torch.float64), "k": torch.zeros(dim, width, dtype=torch.float64)}
    reads["q"][:8, :8] = torch.eye(8, dtype=torch.float64)
    reads["k"][:8, 8:16] = torch.eye(8, dtype=torch.float64)
    for name in ("q", "k"):
        plain_w[name] = reads[name]
        part_w[name] = reads[name].to(part_w[name].dtype).cuda()
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=2048, max_positions=1024)
    generator = torch.Generator().manual_seed(2)
    for far in (0, 1, 63, 64, 500):
        x = (0.002 * torch.randn(n, width, generator=generator)).to(torch.bfloat16).double()
        x[far, 8:16], x[n - 1, :8] = 8.0, 8.0
        want = P.retention(x, plain_w, sizes, 1e-5)[0]
        without = x.clone()
        without[far, 8:16] = x[300, 8:16]
        assert _relative(P.retention(without, plain_w, sizes, 1e-5)[0][n - 1], want[n - 1]) > 0.3  # the mark decides
        for cuts in ([n], [n - 1, n], [650] + list(range(651, n + 1))):
            got = _run_in_steps(lambda h, ctx: mixer.forward(h, ctx, cache.view(0), rt), cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"far key at {far}, cuts {cuts[:2]}", bf16=3e-2, f32=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, taps, width", [(4, 2, 16, 24, 3, 64), (2, 2, 32, 8, 5, 48), (4, 2, 16, 16, 2, 40), (1, 1, 48, 32, 4, 56),
                                                                     (3, 1, 72, 20, 4, 40)])
def test_the_gated_delta_rule_alone(dtype, heads, kv_heads, dim, vdim, taps, width):
    """Decays that forget and betas between nought and one; the convolution's last inputs and the matrix state are carried
    across portions down to two tokens, across single tokens, and kept apart between three unequal sequences."""
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    sizes = delta(heads, kv_heads, dim, vdim, taps)
    mixer = build_part("mixer", dict(kind="gated_delta_rule", width=width, heads=heads, qk_heads=kv_heads, key_dim=dim, value_dim=vdim, taps=taps,
                                     eps=1e-5, q="q", k="k", v="v", q_conv="q.conv", k_conv="k.conv", v_conv="v.conv", b="b", a="a", a_log="A_log",
                                     dt_bias="dt_bias", norm="norm", g="g", o="o"))
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 8.0, "k": 8.0, "v": 8.0, "g": 12.0, "o": 5.0, "b": 10.0, "a": 10.0, "A_log": 8.0,
                                                       "dt_bias": 8.0, "q.conv": 2.0, "k.conv": 2.0, "v.conv": 2.0})
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    lengths = [200, 3, 67]
    xs = _inputs(lengths, width)
    want = [P.gated_delta_rule(x, plain_w, sizes, 1e-5, _rounding(dtype)) for x in xs]
    decays = torch.exp(-torch.exp(plain_w["A_log"]) * P.softplus(xs[0] @ plain_w["a"].T + plain_w["dt_bias"]))
    assert float(decays.min()) < 0.5 and float(decays.max()) > 0.9  # some tokens forget, some keep
    for cuts in CUTS:
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"gated delta rule {cuts[0][:2]} length {n}", bf16=4e-2, f32=1e-4)


def _softmax_part(sizes, width, rt):
    from nnis_amd.parts import build_part

    rot = sizes.get("rot")
    positions = {}
    if rot:
        scaling = rot.get("scaling")
        positions = _positions({"r": {"kind": "rotary_half", "rot_dim": rot["dims"], "theta": rot["base"], "max_positions": None, "angles": "float64",
                                      "ramp": None if scaling is None else (scaling["factor"], scaling["original"], scaling["fast"], scaling["slow"])}}, rt)
    return build_part("mixer", dict(kind="causal_attention", width=width, heads=sizes["heads"], kv_heads=sizes["kv_heads"], head_dim=sizes["dim"],
                                    scale=sizes["scale"], position="r" if rot else None, values_from_keys=True, head_gate="g", q="q", k="k", v=None,
                                    o="o"), positions=positions)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, rot, width", [(4, 2, 32, (16, 5000.0, (4.0, 64, 8.0, 1.0)), 64), (3, 1, 16, None, 48),
                                                              (2, 2, 64, (64, 2e4, (8.0, 32, 4.0, 0.5)), 40), (6, 2, 16, (4, 1e3), 56)])
def test_attention_whose_values_are_its_keys(dtype, heads, kv_heads, dim, rot, width):
    """The values are the keys before their rotation (a model whose values were the rotated keys, or that rotated the
    values, differs at every position but the first); one gate a head; frequencies scaled over a ramp."""
    rt = runtime(dtype)
    sizes = softmax(heads, kv_heads, dim, scale=0.4, rot=rot)
    mixer = _softmax_part(sizes, width, rt)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 6.0, "k": 6.0, "g": 20.0, "o": 5.0})
    mixer.check(rt)
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    lengths = [200, 3, 67]
    xs = _inputs(lengths, width)
    want = [P.softmax_attention(x, plain_w, sizes, _rounding(dtype)) for x in xs]
    for cuts in CUTS:
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"attention {cuts[0][:2]} length {n}", bf16=4e-2)


def _latent_part(sizes, width, rt):
    from nnis_amd.parts import build_part

    positions = _positions({"p": {"kind": "rotary_pairs", "rot_dim": sizes["rot_dim"], "theta": sizes["rot"]["base"], "max_positions": None,
                                  "angles": "float64"}}, rt) if sizes["rot_dim"] else {}
    return build_part("mixer", dict(kind="latent_attention", width=width, heads=sizes["heads"], key_dim=sizes["dim"], value_dim=sizes["vdim"],
                                    q_rank=None, kv_rank=sizes["kv_rank"], scale=sizes["scale"], eps=1e-5, q="q", dkv="dkv", dkv_norm="dkv.norm",
                                    uk="uk", uv="uv", o="o", rot_dim=sizes["rot_dim"], position="p" if sizes["rot_dim"] else None,
                                    window=(sizes.get("mask") or {}).get("size"), channel_gate="g"), positions=positions)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot_dim, vdim, kv_rank, window, width", [(4, 16, 8, 24, 40, 37, 64), (3, 32, 16, 16, 48, 70, 48), (2, 24, 8, 40, 24, None, 40),
                                                                               (2, 8, 4, 8, 16, 1, 40), (1, 16, 4, 12, 16, 64, 56)])
def test_latent_attention_in_a_window(dtype, heads, dim, rot_dim, vdim, kv_rank, window, width):
    rt = runtime(dtype)
    sizes = latent(heads, dim, rot_dim, vdim, kv_rank, scale=0.5, window=window)
    mixer = _latent_part(sizes, width, rt)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 6.0, "dkv": 6.0, "uk": 4.0, "uv": 4.0, "g": 20.0, "o": 5.0})
    mixer.check(rt)
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    lengths = [200, 3, 67]
    xs = _inputs(lengths, width)
    want = [P.latent_attention(x, plain_w, sizes, 1e-5, _rounding(dtype)) for x in xs]
    for cuts in CUTS:
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"latent attention {cuts[0][:2]} length {n}", bf16=5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [37, 64, 70, 9])
def test_the_edge_of_the_window_decides(dtype, window):
    """One head whose queries and latents read marked channels (no rotated part's weight, identity-like maps): a marked
    token just inside the window takes the last query's weight, one just outside is not seen at all; the last token
    comes in a prompt, in a portion of three, in a portion of one behind a prompt, and behind decoded tokens."""
    rt = runtime(dtype)
    width, n, rank = 32, 180, 16
    sizes = latent(1, 16, 4, 16, rank, scale=4.0, window=window)
    mixer = _latent_part(sizes, width, rt)
    plain_w, part_w = _weights(mixer, dtype, 11, scale={"uv": 10.0, "o": 20.0, "g": 5.0})
    reads = {"q": torch.zeros(20, width, dtype=torch.float64), "dkv": torch.zeros(rank + 4, width, dtype=torch.float64),
             "uk": torch.eye(16, rank, dtype=torch.float64), "dkv.norm": torch.ones(rank, dtype=torch.float64)}
    reads["q"][:8, :8] = torch.eye(8, dtype=torch.float64)
    reads["dkv"][:8, 8:16] = torch.eye(8, dtype=torch.float64)
    reads["dkv"][8, 16] = 1.0  # a channel that is one in every token keeps the norm from blowing noise up to a mark's size
    for name, value in reads.items():
        plain_w[name] = value
        part_w[name] = value.to(part_w[name].dtype).cuda()
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=2048, max_positions=1024)
    generator = torch.Generator().manual_seed(1)
    share = {}
    for what, place in (("inside", n - window), ("outside", n - window - 1)):
        x = (0.002 * torch.randn(n, width, generator=generator)).to(torch.bfloat16).double()
        x[:, 16] = 1.0
        x[place, 8:16], x[n - 1, :8] = 8.0, 8.0
        want = P.latent_attention(x, plain_w, sizes, 1e-5)
        without = x.clone()
        without[place, 8:16] = x[0, 8:16]
        share[what] = _relative(P.latent_attention(without, plain_w, sizes, 1e-5)[n - 1], want[n - 1])
        for cuts in ([n], [n - 3, n], [n - 1, n], [100] + list(range(101, n + 1))):
            got = _run_in_steps(lambda h, ctx: mixer.forward(h, ctx, cache.view(0), rt), cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"mark {what} at {place} (window {window}), cuts {cuts[:2]}", bf16=4e-2, f32=1e-4)
            _close(got, want, dtype, f"mark {what} at {place}, all tokens, cuts {cuts[:2]}", bf16=4e-2, f32=1e-4)
    assert share["inside"] > 0.3 and share["outside"] < 1e-6, share


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_mixers_side_by_side_are_added_with_their_factors(dtype):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    width = 64
    left, right = softmax(4, 2, 32, scale=0.4, rot=(16, 5000.0, (4.0, 64, 8.0, 1.0))), delta(4, 2, 16, 24, 3)
    sizes = parallel(left, right, 0.6, -1.3)
    positions = _positions({"r": {"kind": "rotary_half", "rot_dim": 16, "theta": 5000.0, "max_positions": None, "angles": "float64",
                                  "ramp": (4.0, 64, 8.0, 1.0)}}, rt)
    branches = [dict(kind="causal_attention", width=width, heads=4, kv_heads=2, head_dim=32, scale=0.4, position="r", values_from_keys=True,
                     head_gate="left.g", q="left.q", k="left.k", v=None, o="left.o"),
                dict(kind="gated_delta_rule", width=width, heads=4, qk_heads=2, key_dim=16, value_dim=24, taps=3, eps=1e-5, q="right.q", k="right.k",
                     v="right.v", q_conv="right.q.conv", k_conv="right.k.conv", v_conv="right.v.conv", b="right.b", a="right.a",
                     a_log="right.A_log", dt_bias="right.dt_bias", norm="right.norm", g="right.g", o="right.o")]
    mixer = build_part("mixer", dict(kind="side_by_side", width=width, eps=1e-5, branches=branches, scales=[0.6, -1.3]), positions=positions)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"q": 6.0, "k": 6.0, "v": 6.0, "g": 12.0, "o": 5.0, "b": 8.0, "a": 8.0})
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    lengths = [200, 3, 67]
    xs = _inputs(lengths, width)
    want = [P.parallel(x, plain_w, sizes, 1e-5, _rounding(dtype)) for x in xs]
    for cuts in CUTS:
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"side by side {cuts[0][:2]} length {n}", bf16=4e-2, f32=1e-4)


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def _sharpen(folder):
    """A random model's weights are too small for its mixers to matter: queries, keys and latents are scaled so that
    attention is sharper, gates and the decays' projections so that each of them matters, the head so that logits are of
    order one.  The routers' corrections are scaled most: they then decide most choices, and few choices hinge on what
    rounding does to a score (a choice that flips swaps a whole unit-norm output, in the plain twin as in the engine, at
    places of their own)."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key in tensors:
        if key.endswith((".mix.g", ".left.g", ".right.g", ".right.a", ".right.b")):
            factor = 6.0
        elif key.endswith(".mlp.router"):
            factor = 2.0
        elif key.endswith(".correction"):
            factor = 30.0
        elif key.endswith((".q", ".k", ".dkv", ".gate", ".up", ".down", ".v", ".o", ".uk", ".uv", ".conv")):
            factor = 3.0
        elif key.endswith((".A_log", ".dt_bias")) or key == "head":
            factor = 8.0
        else:
            continue
        tensors[key] = (tensors[key].float() * factor).to(torch.bfloat16)
    save_file(tensors, path)


def _folder(path, config, seed):
    nnis_amd.write_random_model(str(path), config, seed)
    _sharpen(str(path))
    return str(path)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: _folder(tmp_path_factory.mktemp(f"mafalorn_{name}"), config, seed) for name, (config, seed) in MAFALORN_CONFIGS.items()}


def _ids(count, vocab, seed):
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()


class Yardstick:
    """What the engine may differ from the plain 64-bit logits by, as root mean square relative to the logits' own: in
    32-bit, rounding (5e-5 over a prompt, 2e-4 at a single position); in bfloat16, three times what rounding the plain
    model's activations to bfloat16 does on the same tokens (a single position: four times the worst position's)."""

    def __init__(self, plain):
        self.plain, self.known = plain, {}
        self.least = (0.0, 0.0)
        self.least = self.twin(_ids(64, plain.config["vocab"], 999))[1:]

    def twin(self, ids):
        key = tuple(ids)
        if key not in self.known:
            want, twin = self.plain.logits(ids), self.plain.logits(ids, P.bf16_round)
            rows = [_relative(twin[i], want[i]) for i in range(len(ids))]
            self.known[key] = (want, _relative(twin, want), max(rows))
            assert 1e-4 < self.known[key][1] < 0.3, self.known[key][1]
        return self.known[key]

    def check(self, got, ids, dtype, what, rows=None):
        want, overall, worst = self.twin(ids)
        single = isinstance(rows, int)
        want = want if rows is None else want[rows]
        error = _relative(got, want)
        bound = (2e-4 if single else 5e-5) if dtype == "float32" else (4.0 * max(worst, self.least[1]) if single else 3.0 * max(overall, self.least[0]))
        assert error <= bound, f"{what}: relative error {error:.3g} (bound {bound:.3g})"


def _collect(engine, slot, ids, cuts):
    from nnis_amd.engine.batch import StepEntry

    rows, done = [], 0
    for end in cuts:
        rows.append(engine.step([StepEntry(slot, ids[done:end], list(range(end - done)))]).cpu())
        done = end
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MAFALORN_CONFIGS))
def test_the_stream_after_every_layer(folders, name, dtype):
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.parts.lazy import PostNormed, PreparedRows

    plain = P.PlainMafalorn(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=256)
    ids = _ids(90, MAFALORN_CONFIGS[name][0]["vocab"], 8)
    want, twin = [], []
    plain.logits(ids, stream_after=want)
    plain.logits(ids, P.bf16_round, stream_after=twin)  # what rounding to bfloat16 alone does to the stream behind each layer
    seen = []
    for block in engine.model.layers:
        def watched(stream, ctx, view, rt, following=None, inner=block.forward):
            out = inner(stream, ctx, view, rt, following=following) if following is not None else inner(stream, ctx, view, rt)
            if isinstance(out, PreparedRows):
                seen.append(out.x.clone())
            else:
                seen.append(out[0] + out[1].materialize(rt).float() if isinstance(out[1], PostNormed) else out[0].clone())
            return out
        block.forward = watched
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, ids, [0])])
    assert len(seen) == len(want) == len(MAFALORN_CONFIGS[name][0]["layers"])
    for run, (got, expected, rounded) in enumerate(zip(seen, want, twin)):
        assert _relative(got.cpu(), expected) < (1e-5 if dtype == "float32" else max(1e-2, 3.0 * _relative(rounded, expected))), f"layer {run}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(MAFALORN_CONFIGS))
def test_prompts_whole_in_portions_and_token_by_token(folders, name, dtype):
    config = MAFALORN_CONFIGS[name][0]
    plain = P.PlainMafalorn(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=1024)
    ids = _ids(150, config["vocab"], 1)
    yard = Yardstick(plain)
    for cuts in ([150], [2, 4, 5, 63, 64, 66, 128, 129, 150], [100] + list(range(101, 151)), list(range(1, 41))):
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, cuts)
        engine.end_sequence(slot)
        yard.check(got, ids, dtype, f"{name} cuts {cuts[:3]}..", rows=slice(0, cuts[-1]))
        for place in (0, 1, 2, cuts[-1] - 1):  # every position by itself, the first tokens among them
            yard.check(got[place], ids, dtype, f"{name} cuts {cuts[:3]}.. position {place}", rows=place)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_unequal_batches_equal_each_request_alone(folders, name, dtype):
    """Requests of different lengths start together, are decoded together and end one after the other; their slots,
    pages and states go to requests that start later.  Every logit equals the plain model's on that request alone."""
    from nnis_amd.engine.batch import StepEntry

    config = MAFALORN_CONFIGS[name][0]
    plain = P.PlainMafalorn(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=64 * 9, max_slots=4)
    yard = Yardstick(plain)
    pages = engine.free_pages()
    for batch_seed, lengths in ((0, [1, 70, 130, 9]), (1, [65, 3, 128]), (2, [2, 2, 200, 64])):
        requests = [_ids(n + decode, config["vocab"], 100 * batch_seed + i) for i, (n, decode) in enumerate(zip(lengths, (12, 5, 9, 1)))]
        slots = [engine.start_sequence() for _ in requests]
        at = list(lengths)
        logits = engine.step([StepEntry(s, r[:n], list(range(n))) for s, r, n in zip(slots, requests, lengths)]).cpu()
        row = 0
        for i, n in enumerate(lengths):
            yard.check(logits[row:row + n], requests[i], dtype, f"{name} batch {batch_seed} prompt {i}", rows=slice(0, n))
            row += n
        live = list(range(len(requests)))
        while live:
            live = [i for i in live if at[i] < len(requests[i]) or engine.end_sequence(slots[i])]
            if not live:
                break
            logits = engine.step([StepEntry(slots[i], [requests[i][at[i]]], [0]) for i in live]).cpu()
            for row, i in enumerate(live):
                yard.check(logits[row], requests[i], dtype, f"{name} batch {batch_seed} request {i} position {at[i]}", rows=at[i])
                at[i] += 1
        assert engine.free_slots() == 4 and engine.free_pages() == pages


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_across_windows_and_pages(tmp_path, dtype):
    """330 tokens one by one behind a prompt of 3: windows of 5 and 70 tokens pass over decoded tokens, five page borders
    are crossed, and the states of retention and of the delta rule are carried through every step."""
    config = mafalorn(vocab=200, width=64, logit_scale=1.5, layers=[
        layer("latent_attention", latent(2, 16, 4, 12, 16, scale=0.3, window=5), moe(4, 2, 16, identity=2, groups=(3, 2))),
        layer("parallel", parallel(softmax(2, 1, 16, scale=0.3, rot=(8, 1e4, (2.0, 16, 4.0, 1.0))), delta(2, 1, 16, 16, 4), 0.7, 0.9)),
        layer("retention", retention(2, 16, 16, (0.99, 0.8), rot=(16, 1e4)), moe(3, 1, 24)),
        layer("latent_attention", latent(2, 16, 4, 12, 16, scale=0.3, window=70))])
    folder = _folder(tmp_path / "m", config, 7)
    plain = P.PlainMafalorn(folder)
    engine = nnis_amd.load_engine(folder, dtype=dtype, max_tokens=512)
    ids = _ids(330, config["vocab"], 4)
    slot = engine.start_sequence()
    got = _collect(engine, slot, ids, [3] + list(range(4, 331)))
    yard = Yardstick(plain)
    yard.check(got, ids, dtype, "long decoding")
    yard.check(got[-1], ids, dtype, "long decoding, the last token", rows=len(ids) - 1)


@pytest.mark.parametrize("name", sorted(MAFALORN_CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name):
    """``nnis_amd.generate``: the library's scheduler, batches and selection on the device.  In 32-bit the tokens are
    the plain model's, unless two logits are closer than rounding."""
    config = MAFALORN_CONFIGS[name][0]
    plain = P.PlainMafalorn(folders[name])
    prompts = [_ids(n, config["vocab"], 50 + n) for n in (1, 19, 70)]
    got = nnis_amd.generate(folders[name], prompts, max_new_tokens=10, dtype="float32", stop_token_ids=[])
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == 10
        logits = plain.logits(prompt + tokens)[len(prompt) - 1:-1]
        for row, token in zip(logits, tokens):
            assert float(row[token]) >= float(row.max()) - 1e-4 * float(row.abs().max()), "a generated token is not the plain model's best"
    got16 = nnis_amd.generate(folders[name], prompts, max_new_tokens=6, dtype="bfloat16", stop_token_ids=[])
    assert [len(t) for t in got16] == [6, 6, 6]


def test_the_command_line_runs_the_model(folders):
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "nnis"), "generate", "--model", folders["B"], "--prompt-ids", "5,17,3",
                           "--max-new-tokens", "4", "--dtype", "float32"], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    plain = P.PlainMafalorn(folders["B"])
    assert [int(t) for t in done.stdout.strip().splitlines()[-1].split(",")] == plain.greedy([5, 17, 3], 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_runner_replays_schedules(folders, tmp_path, dtype):
    """The same requests whole, with their last tokens one by one, and in unequal batches whose slots are used again,
    through ``bin/trace_run`` in a cache too small to hold the schedules side by side."""
    config = MAFALORN_CONFIGS["A"][0]
    plain = P.PlainMafalorn(folders["A"])
    rng = np.random.default_rng(3)
    requests = {f"r{i}": rng.integers(0, config["vocab"], size=n).tolist() for i, n in enumerate([1, 7, 40, 65, 97, 130])}
    schedules = (("w", replay.whole(requests)), ("t", replay.tail_one_by_one(requests)), ("b", replay.unequal_batches(requests, batch=3, decode=32)))
    steps = [{"entries": [dict(e, id=tag + e["id"]) for e in step["entries"]], "end": [tag + n for n in step.get("end", [])]}
             for tag, schedule in schedules for step in schedule]
    rows = replay.run_trace(folders["A"], dtype, steps, str(tmp_path), max_tokens=6 * 64, vocab=config["vocab"])
    yard = Yardstick(plain)
    for tag, _ in schedules:
        for name, ids in requests.items():
            got = np.stack([rows[(tag + name, p)] for p in range(len(ids))])
            yard.check(got, ids, dtype, f"schedule {tag} request {name}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_model_without_the_optional_mechanisms(tmp_path, dtype):
    """No logit scale, no rotation anywhere but the latent's own part, no window, no identity outputs, no groups, a layer
    without a feed-forward."""
    config = mafalorn(vocab=120, width=48, layers=[
        layer("retention", retention(2, 16, 16, (0.9, 0.99)), moe(3, 2, 24)),
        layer("parallel", parallel(softmax(2, 1, 16, scale=0.3), delta(2, 1, 16, 16, 2))),
        layer("latent_attention", latent(2, 16, 4, 12, 16, scale=0.3), moe(2, 1, 16))])
    folder = _folder(tmp_path / "bare", config, 41)
    plain = P.PlainMafalorn(folder)
    engine = nnis_amd.load_engine(folder, dtype=dtype, max_tokens=512)
    ids = _ids(100, config["vocab"], 6)
    slot = engine.start_sequence()
    got = _collect(engine, slot, ids, [70] + list(range(71, 101)))
    Yardstick(plain).check(got, ids, dtype, "a model without the optional mechanisms")


LATENT_SIZES = [(40, 8), (48, 16), (24, 8), (16, 4)]  # (latent, rotated part) whose attention modules are built beforehand
HEAD_SIZES = [16, 32, 48, 64]


def test_other_sizes_drawn_from_a_seed(tmp_path):
    """Configurations whose every size is drawn at random, in 32-bit against the plain model: prompt, a portion, single tokens."""
    import random

    for seed in range(6):
        r = random.Random(seed)
        layers = []
        for index in range(r.randint(1, 5)):
            mlp = None
            if r.random() < 0.75:
                experts, identity = r.randint(1, 6), r.choice([None, 0, 1, 3])
                outputs = experts + (identity or 0)
                count = r.choice([c for c in (1, 2, 3, 4) if outputs % c == 0])
                keep = r.randint(1, count)
                mlp = moe(experts, r.randint(1, keep * (outputs // count)), r.randint(4, 40), identity=identity,
                          groups=r.choice([None, (count, keep)]) if keep == count else (count, keep))
            kind = r.choice(["retention", "parallel", "latent_attention"])
            if kind == "retention":
                heads, dim = r.randint(1, 4), 2 * r.randint(2, 40)
                rot = r.choice([None, (2 * r.randint(1, dim // 2), r.choice([50.0, 1e4, 1e6]))])
                mixer = retention(heads, dim, r.randint(1, 70), [r.choice([1.0, r.uniform(0.3, 0.9999)]) for _ in range(heads)], rot)
            elif kind == "parallel":
                dim, k = r.choice(HEAD_SIZES), r.randint(1, 2)
                rot = r.choice([None, (2 * r.randint(1, dim // 2), r.choice([50.0, 1e4])),
                                (dim, 1e4, (r.uniform(1.5, 16.0), r.choice([16, 64, 1024]), r.uniform(2.0, 32.0), r.uniform(0.25, 1.5)))])
                g = r.randint(1, 2)
                mixer = parallel(softmax(r.randint(1, 3) * k, k, dim, scale=r.uniform(0.05, 0.5), rot=rot),
                                 delta(r.randint(1, 2) * g, g, r.randint(1, 70), r.randint(1, 50), r.randint(2, 5)),
                                 r.uniform(0.2, 2.0), r.uniform(0.2, 2.0))
            else:
                rank, rot_dim = r.choice(LATENT_SIZES)
                mixer = latent(r.randint(1, 4), r.randint(1, 40), rot_dim, r.randint(1, 40), rank, scale=r.uniform(0.05, 0.5),
                               base=r.choice([50.0, 1e4, 1e6]), window=r.choice([None, r.randint(1, 90)]))
            layers.append(layer(kind, mixer, mlp))
        config = mafalorn(vocab=r.randint(20, 400), width=4 * r.randint(3, 30), layers=layers, logit_scale=r.choice([None, 1.0, r.uniform(0.2, 4.0)]),
                          eps=r.choice([1e-5, 1e-6, 1e-3]))
        folder = _folder(tmp_path / f"m{seed}", config, seed)
        plain = P.PlainMafalorn(folder)
        engine = nnis_amd.load_engine(folder, dtype="float32", max_tokens=256)
        ids = _ids(80, config["vocab"], seed)
        want = plain.logits(ids)
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, [66, 70] + list(range(71, 81)))
        assert _relative(got, want) < 5e-5, f"seed {seed}: {config}"
