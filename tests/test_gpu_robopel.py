"""Robopel on the GPU against the plain implementation (``plain_robopel``):
each mechanism alone, then whole models through the engine -- prompts whole, in
portions and token by token, unequal batches, slots and pages used again, keys
far away, at page borders and at the edges of a window and of a pooled block,
long decoding, greedy generation through the library's entry point, the trace
runner.  32-bit is held to rounding; bfloat16 to the error of the plain model
run with its activations rounded where the engine rounds them.
"""

import copy
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import nnis_amd
import plain_robopel as R
import replay
from gpu_helpers import cache_for, context, runtime
from robopel_configs import ROBOPEL_CONFIGS, attention, dense, layer, moe, robopel

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def _relative(got, want):
    got, want = torch.as_tensor(np.asarray(got)).double(), torch.as_tensor(np.asarray(want)).double()
    return float((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-30))


def _close(got, want, dtype, what="", bf16=3e-2):
    error = _relative(got.detach().float().cpu() if isinstance(got, torch.Tensor) else got, want)
    bound = 3e-5 if dtype == "float32" else bf16
    assert error <= bound, f"{what}: relative error {error:.3g} (bound {bound:.3g})"


def _weights(part, dtype, seed, scale=None):
    """Random tensors for a part, by its own declarations: (for the plain functions in 64-bit, for the part)."""
    from nnis_amd.weights.random_init import _INIT_RULES

    generator = torch.Generator().manual_seed(seed)
    stored = {}
    for t in part.tensors():
        value = _INIT_RULES[t.init](t, generator, torch.bfloat16)
        if scale and t.name in scale:
            value = (value.float() * scale[t.name]).to(torch.bfloat16)
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


# ---------------------------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, width", [(1, 8), (37, 50), (5, 1030), (9, 2048), (3, 4096), (2, 4104), (300, 96)])
def test_the_norm_on_the_way_out(y_dtype, tokens, width):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(tokens + width)
    x = torch.randn(tokens, width, generator=generator)
    y = (3.0 * torch.randn(tokens, width, generator=generator)).to(y_dtype)
    w = 0.3 * torch.randn(width, generator=generator)
    want = x.double() + R.rms_norm(y.double(), 1.0 + w.double(), 1e-5)
    stream, rows = x.clone().cuda(), torch.empty(tokens, width, device="cuda", dtype=torch.bfloat16)
    ops.rms_post_step(stream, y.cuda(), w.cuda(), 1.0, 1e-5, h=rows)
    assert _relative(stream.cpu(), want) < 1e-6 and _relative(rows.float().cpu(), want) < 4e-3
    stream = x.clone().cuda()
    ops.rms_post_step(stream, y.cuda(), (1.0 + w).cuda(), 0.0, 1e-5)  # (the offset added beforehand, no rows asked for)
    assert _relative(stream.cpu(), want) < 1e-6
    # a share of other rows joins y before the norm; the rows may be the very buffer that receives the new ones
    keep = torch.rand(tokens, generator=generator)
    rows_in = torch.randn(tokens, width, generator=generator).to(torch.bfloat16)
    want = x.double() + R.rms_norm(y.double() + keep.double()[:, None] * rows_in.double(), 1.0 + w.double(), 1e-5)
    stream, rows = x.clone().cuda(), rows_in.clone().cuda()
    ops.rms_post_step(stream, y.cuda(), w.cuda(), 1.0, 1e-5, h=rows, share=(keep.cuda(), rows))
    assert _relative(stream.cpu(), want) < 1e-6 and _relative(rows.float().cpu(), want) < 4e-3
    picked = torch.tensor([tokens - 1, 0], dtype=torch.int32).cuda()
    got = ops.cast_rows(stream, torch.empty(2, width, device="cuda", dtype=torch.bfloat16), picked)
    assert torch.equal(got.cpu(), stream.cpu()[[tokens - 1, 0]].to(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows, inner", [(1, 8), (33, 72), (4, 1500), (7, 5632), (2, 8192), (3, 8200), (40, 74)])
def test_poly_norm(dtype, rows, inner):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(rows)
    z = (2.0 * torch.randn(rows, inner, generator=generator)).to(dtype)
    coefficients = torch.tensor([0.7, -0.4, 0.25, 0.1])
    got = ops.poly_norm(z.cuda(), coefficients.cuda(), 1e-5, torch.empty(rows, inner, device="cuda", dtype=dtype))
    zz, one = z.double(), torch.ones(inner, dtype=torch.float64)
    want = 0.7 * R.rms_norm(zz, one, 1e-5) - 0.4 * R.rms_norm(zz ** 2, one, 1e-5) + 0.25 * R.rms_norm(zz ** 3, one, 1e-5) + 0.1
    assert _relative(got.float().cpu(), want) < (1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows, outputs, width", [(1, 3, 8), (70, 11, 96), (300, 9, 200), (300, 5, 3500), (260, 70, 6500)])
def test_router_logits_are_32_bit_products(dtype, rows, outputs, width):
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(rows + width)
    x = torch.randn(rows, width, generator=generator).to(dtype)
    w = torch.randn(outputs, width, generator=generator)
    got = ops.router_logits(x.cuda(), w.cuda(), torch.empty(rows, outputs, device="cuda"))
    assert _relative(got.cpu(), x.double() @ w.double().T) < 2e-6
    # logits and choice in one kernel give what the two kernels give
    experts, top = max(1, outputs - 2), min(3, outputs)
    correction = 0.3 * torch.randn(outputs, generator=generator)
    apart = ops.route_top(got, correction.cuda(), experts, top, torch.empty(rows, experts, device="cuda"), torch.empty(rows, device="cuda"))
    fused = ops.route(x.cuda(), w.cuda(), correction.cuda(), experts, top, torch.empty(rows, experts, device="cuda"), torch.empty(rows, device="cuda"))
    scores = torch.softmax((x.double() @ w.double().T), dim=-1)
    for one, other in zip(apart, fused):
        close = (one - other).abs() < 1e-5
        # (a choice may differ where two corrected scores are closer than the two sums' rounding)
        assert float(close.float().mean()) > 0.995, float(close.float().mean())
    chosen = torch.topk(scores + correction.double(), top, dim=-1).indices
    total = fused[0].cpu().double().sum(dim=1) + fused[1].cpu().double()  # a row's weights, identity outputs included
    assert float(((total - scores.gather(1, chosen).sum(dim=1)).abs() < 1e-5).float().mean()) > 0.995


@pytest.mark.parametrize("experts, identity, top", [(5, 1, 2), (3, 0, 1), (9, 2, 3), (70, 3, 4), (1, 0, 1), (2, 2, 4)])
def test_the_router_chooses_by_corrected_scores_and_weighs_by_plain_ones(experts, identity, top):
    """The correction is large against the scores' differences, so it decides who is chosen; the weights are the
    scores without it, not renormalised; the identity outputs' weights are summed apart."""
    from nnis_amd.kernels import ops

    generator = torch.Generator().manual_seed(experts)
    n, rows = experts + identity, 40
    logits = torch.randn(rows, n, generator=generator)
    correction = 0.5 * torch.randn(n, generator=generator)
    gates, keep = ops.route_top(logits.cuda(), correction.cuda(), experts, top, torch.empty(rows, experts, device="cuda"),
                                torch.empty(rows, device="cuda"))
    scores = torch.softmax(logits.double(), dim=-1)
    chosen = torch.topk(scores + correction.double(), top, dim=-1).indices
    want = torch.zeros(rows, n, dtype=torch.float64).scatter(1, chosen, scores.gather(1, chosen))
    assert torch.topk(scores, top, dim=-1).indices.sort(dim=1).values.ne(chosen.sort(dim=1).values).any() or n == top  # the correction matters
    assert float((gates.cpu().double() - want[:, :experts]).abs().max()) < 1e-6
    assert float((keep.cpu().double() - want[:, experts:].sum(dim=1)).abs().max()) < 1e-6
    bare, _ = ops.route_top(logits.cuda(), None, experts, top, torch.empty(rows, experts, device="cuda"), torch.empty(rows, device="cuda"))
    plain = torch.topk(scores, top, dim=-1).indices
    want = torch.zeros(rows, n, dtype=torch.float64).scatter(1, plain, scores.gather(1, plain))
    assert float((bare.cpu().double() - want[:, :experts]).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, inner, experts, top, identity", [(64, 24, 5, 2, 1), (48, 40, 3, 1, 0), (96, 16, 9, 3, 2), (40, 8, 2, 3, 1)])
def test_routed_feed_forward_alone(dtype, width, inner, experts, top, identity):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    part = build_part("feed_forward", dict(kind="routed", width=width, inner=inner, experts=experts, top=top, identity=identity,
                                           router="router", correction="correction", up="e{}.up", down="e{}.down"))
    plain_w, part_w = _weights(part, dtype, 3, scale={"router": 4.0, "correction": 0.5, **{f"e{e}.up": 8.0 for e in range(experts)},
                                                      **{f"e{e}.down": 8.0 for e in range(experts)}})
    part.bind(part_w, rt)
    generator = torch.Generator().manual_seed(5)
    x = torch.randn(70, width, generator=generator).to(torch.bfloat16).double()
    rnd = R.identity if dtype == "float32" else R.bf16_round
    want, chosen = R.routed_feed_forward(x, plain_w, {"experts": experts, "top": top, "identity": identity}, rnd)
    picked = set(chosen.flatten().tolist())
    assert len(picked) > (experts + identity) // 2 and (not identity or max(picked) >= experts)  # many outputs are chosen, an identity one among them
    got = part.forward(x.to(rt.dtype).cuda(), None, rt)
    _close(got, want, dtype, "routed feed-forward")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, inner", [(64, 136), (40, 36), (256, 640)])
def test_poly_norm_feed_forward_alone(dtype, width, inner):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    part = build_part("feed_forward", dict(kind="poly_norm", width=width, inner=inner, eps=1e-5, up="up", down="down", act="act"))
    plain_w, part_w = _weights(part, dtype, 4, scale={"up": 10.0, "down": 10.0})
    part.bind(part_w, rt)
    x = torch.randn(33, width, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).double()
    want = R.poly_norm_feed_forward(x, plain_w, 1e-5, R.identity if dtype == "float32" else R.bf16_round)
    _close(part.forward(x.to(rt.dtype).cuda(), None, rt), want, dtype, "PolyNorm feed-forward")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, channels", [(64, 72), (40, 8), (96, 300)])
def test_min_gru_alone(dtype, width, channels):
    """Whole prompts (one long enough to be cut into pieces that run side by side), portions down to two tokens, single
    tokens; three unequal sequences in every step, their states apart."""
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    mixer = build_part("mixer", dict(kind="min_gru", width=width, channels=channels, z="z", z_bias="z.b", x="x", x_bias="x.b", g="g", o="o"))
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"z": 12.0, "x": 12.0, "g": 12.0, "z.b": 10.0, "x.b": 10.0, "o": 5.0})
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    generator = torch.Generator().manual_seed(5)
    lengths = [200, 3, 67]
    xs = [torch.randn(n, width, generator=generator).to(torch.bfloat16).double() for n in lengths]
    rnd = R.identity if dtype == "float32" else R.bf16_round
    want = [R.min_gru(x, plain_w, rnd)[0] for x in xs]
    u = xs[0] @ plain_w["x"].T + plain_w["x.b"]
    assert float((u >= 0).double().mean()) > 0.2 and float((u < 0).double().mean()) > 0.2  # both forms of the candidate occur
    for cuts in ([[200], [3], [67]], [[61, 63, 64, 66, 128, 130, 131, 200], [1, 2, 3], [2, 4, 64, 65, 66, 67]],
                 [[150] + list(range(151, 201)), [3], [60] + list(range(61, 68))]):
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"minGRU {cuts[0][:2]} length {n}")


def _attention_part(sizes, width, eps=1e-5, reach=1024, rt=None):
    from nnis_amd.parts import build_part

    positions, name = {}, None
    rot = sizes.get("rot")
    if rot:
        scaling = rot.get("scaling")
        name = "r"
        positions[name] = build_part("position", {"kind": "rotary_pairs", "rot_dim": rot["dims"], "theta": rot["base"], "max_positions": None,
                                                  "angles": "float64", "scaling": None if scaling is None else
                                                  (scaling["factor"], scaling["low"], scaling["high"], scaling["original"])})
        positions[name].bind({}, rt)
        positions[name].reach(reach)
    mask = sizes.get("mask") or {}
    return build_part("mixer", dict(kind="gated_window_attention", width=width, heads=sizes["heads"], kv_heads=sizes["kv_heads"],
                                    head_dim=sizes["dim"], value_dim=sizes["vdim"], scale=sizes["scale"], eps=eps,
                                    softcap=sizes.get("softcap"), window=mask.get("size"), pool=mask.get("pool"), position=name,
                                    q="q", k="k", v="v", o="o", gate="g", q_norm="q.norm", k_norm="k.norm", sink="sink"), positions=positions)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, softcap, rot, window, pool, width", [
    (4, 2, 32, 16, 15.0, (32, 5000.0, (4.0, 1.0, 2.0, 64)), 37, 8, 64), (3, 1, 16, 48, 30.0, (8, 100.0), 70, 24, 48),
    (2, 2, 32, 16, None, None, 9, 1, 96), (6, 2, 24, 40, 40.0, (16, 1e4), 33, 16, 40), (2, 1, 16, 16, 20.0, (16, 1e4), 64, 64, 56),
    (2, 2, 32, 16, 12.0, (32, 300.0), 130, 3, 56), (3, 3, 16, 16, 20.0, (6, 50.0), None, None, 48), (2, 1, 20, 12, None, (20, 1e3), 11, 4, 40)])
def test_gated_window_attention_alone(dtype, heads, kv_heads, dim, vdim, softcap, rot, window, pool, width):
    """Grouped heads, values of their own size, normed and rotated queries and keys, capped scores, a window with pooled
    blocks, a sink large enough to take a good part of the weight, gates that matter.  Whole prompts; then portions down
    to two tokens and single tokens across the borders of pages, of the window and of the blocks."""
    rt = runtime(dtype)
    sizes = attention(heads, kv_heads, dim, vdim, scale=0.4, softcap=softcap, rot=rot, window=window, pool=pool)
    mixer = _attention_part(sizes, width, rt=rt)
    plain_w, part_w = _weights(mixer, dtype, 3, scale={"sink": 30.0, "g": 20.0, "v": 5.0, "o": 5.0})
    for w in (plain_w, part_w):  # norm weights large enough for a sharp softmax
        w["q.norm"], w["k.norm"] = w["q.norm"] * 3.0, w["k.norm"] * 3.0
    mixer.check(rt)
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=1024, max_positions=512)
    generator = torch.Generator().manual_seed(5)
    lengths = [200, 3, 67]
    xs = [torch.randn(n, width, generator=generator).to(torch.bfloat16).double() for n in lengths]
    rnd = R.identity if dtype == "float32" else R.bf16_round
    want = [R.pooled_window_attention(x, plain_w, sizes, 1e-5, None, rnd)[0] for x in xs]
    for cuts in ([[200], [3], [67]], [[61, 63, 64, 66, 128, 130, 131, 200], [1, 2, 3], [2, 4, 64, 65, 66, 67]],
                 [[150] + list(range(151, 201)), [3], [60] + list(range(61, 68))]):
        got = _run_in_steps(lambda x, ctx: mixer.forward(x, ctx, cache.view(0), rt), cache, rt, xs, cuts)
        for g, w, n in zip(got, want, lengths):
            _close(g, w, dtype, f"gated window attention {cuts[0][:2]} length {n}", bf16=4e-2)


def _reading_attention(dtype, window, pool, width=32, dim=32, vdim=16):
    """One head without rotation whose queries read the input's first eight channels and whose keys read the next
    eight, so that a token whose key channels are set takes all the weight of a query whose query channels are set.
    The keys also read channel 16, which ``_quiet_input`` sets to one in every token: the norm of a key then leaves an
    unmarked token's eight channels as small as they were, where without it they would be noise of a mark's size."""
    rt = runtime(dtype)
    sizes = attention(1, 1, dim, vdim, scale=4.0, window=window, pool=pool)
    mixer = _attention_part(sizes, width, rt=rt)
    plain_w, part_w = _weights(mixer, dtype, 11, scale={"v": 20.0, "o": 20.0})
    reads = {"q": torch.zeros(dim, width, dtype=torch.float64), "k": torch.zeros(dim, width, dtype=torch.float64)}
    reads["q"][:8, :8] = torch.eye(8, dtype=torch.float64)
    reads["k"][:8, 8:16] = torch.eye(8, dtype=torch.float64)
    reads["k"][8, 16] = 1.0
    for name in ("q", "k"):
        plain_w[name] = reads[name]
        part_w[name] = reads[name].to(part_w[name].dtype).cuda()
    for name in ("q.norm", "k.norm"):
        plain_w[name] = torch.ones(dim, dtype=torch.float64)
        part_w[name] = torch.ones(dim, dtype=part_w[name].dtype, device="cuda")
    mixer.bind(part_w, rt)
    cache = cache_for([mixer.cache_request()], rt, max_tokens=2048, max_positions=1024)
    return rt, sizes, mixer, plain_w, cache


def _quiet_input(n, width, generator, mark, last):
    x = (0.002 * torch.randn(n, width, generator=generator)).to(torch.bfloat16).double()
    x[:, 16] = 1.0
    x[mark, 8:16] = 8.0  # the norm makes a marked key and the last query of size 2 a channel: a score of 4 * 32, against scores near 0
    x[last, :8] = 8.0
    return x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window, pool", [(37, 8), (64, 16), (70, 1), (9, 24)])
def test_the_edges_of_the_window_and_of_a_block_decide(dtype, window, pool):
    """The marked token stands just inside the window (seen as itself), just outside it in a block that is not yet
    wholly outside (not seen at all), and in the last block that is (seen as a pool-th of its block's mean); the last
    token comes in a prompt, in a portion, and alone.  The output tells the three apart."""
    rt, sizes, mixer, plain_w, cache = _reading_attention(dtype, window, pool)
    width, n = 32, 180
    last_block = (n - window) // pool - 1  # the last block b with b * pool + pool - 1 <= n - 1 - window
    places = {"inside": n - window, "seen block": last_block * pool + pool - 1, "seen block's first": last_block * pool}
    if (n - window) % pool:
        places["outside, block not complete"] = n - window - 1
    generator = torch.Generator().manual_seed(1)
    share = {}
    for what, place in places.items():
        x = _quiet_input(n, width, generator, place, n - 1)
        want = R.pooled_window_attention(x, plain_w, sizes, 1e-5)[0]
        without = x.clone()
        without[place, 8:16] = x[0, 8:16] if place else 0.0
        share[what] = _relative(R.pooled_window_attention(without, plain_w, sizes, 1e-5)[0][n - 1], want[n - 1])
        for cuts in ([n], [n - 3, n], [n - 1, n], [100] + list(range(101, n + 1))):
            got = _run_in_steps(lambda h, ctx: mixer.forward(h, ctx, cache.view(0), rt), cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"mark {what} at {place} (window {window}, blocks of {pool}), cuts {cuts[:2]}", bf16=3e-2)
            _close(got, want, dtype, f"mark {what} at {place}, all tokens, cuts {cuts[:2]}", bf16=3e-2)
    assert share["inside"] > 0.3 and share["seen block"] > 0.3 and share["seen block's first"] > 0.3, share  # seen: the mark decides
    assert share.get("outside, block not complete", 0.0) < 1e-6, share  # not seen: it changes nothing


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_block_counts(dtype):
    """The marked token lies hundreds of tokens back, in the first, second, a page's last and next page's first pooled
    entry (blocks of 2: entries 63 and 64 are positions 126 to 129) and far beyond: its block takes the weight."""
    rt, sizes, mixer, plain_w, cache = _reading_attention(dtype, 20, 2)
    width, n = 32, 700
    generator = torch.Generator().manual_seed(2)
    for far in (0, 1, 2, 127, 128, 500):
        x = _quiet_input(n, width, generator, far, n - 1)
        want = R.pooled_window_attention(x, plain_w, sizes, 1e-5)[0]
        without = x.clone()
        without[far, 8:16] = x[300, 8:16]
        assert _relative(R.pooled_window_attention(without, plain_w, sizes, 1e-5)[0][n - 1], want[n - 1]) > 0.3
        for cuts in ([n], [n - 1, n], [650] + list(range(651, n + 1))):
            got = _run_in_steps(lambda h, ctx: mixer.forward(h, ctx, cache.view(0), rt), cache, rt, [x], [cuts])[0]
            _close(got[n - 1], want[n - 1], dtype, f"far block at {far}, cuts {cuts[:2]}", bf16=3e-2)


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def _sharpen(folder):
    """A random model's weights are too small for its mixers to matter.  Norm weights of queries and keys are scaled so
    that attention is sharp (a key left out or one too many shows); sinks, gates, biases and routers so that each of
    them matters; corrections so that they decide choices; the head so that logits are of order one."""
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key in tensors:
        if key.endswith((".q.norm", ".k.norm")):
            factor = 3.0
        elif key.endswith((".mix.sink", ".mix.g", ".mlp.router")):
            factor = 20.0
        elif key.endswith((".mix.z", ".mix.x", ".mix.v", ".mix.o", ".up", ".down")):
            factor = 7.0
        elif key.endswith((".b", ".correction")) or key == "head":
            factor = 10.0
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
    return {name: _folder(tmp_path_factory.mktemp(f"robopel_{name}"), config, seed) for name, (config, seed) in ROBOPEL_CONFIGS.items()}


def _ids(count, vocab, seed):
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()


class Yardstick:
    """What the engine may differ from the plain 64-bit logits by, as root mean square relative to the logits' own: in
    32-bit, rounding (5e-5 over a prompt, 2e-4 at a single position); in bfloat16, three times what rounding the plain model's activations to bfloat16 does on the same
    tokens (a single position: four times the worst position's)."""

    def __init__(self, plain):
        self.plain, self.known = plain, {}
        self.least = (0.0, 0.0)
        self.least = self.twin(_ids(64, plain.config["vocab"], 999))[1:]

    def twin(self, ids):
        key = tuple(ids)
        if key not in self.known:
            want, twin = self.plain.logits(ids), self.plain.logits(ids, R.bf16_round)
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
@pytest.mark.parametrize("name", sorted(ROBOPEL_CONFIGS))
def test_the_stream_after_every_layer(folders, name, dtype):
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.parts.lazy import PreparedRows

    plain = R.PlainRobopel(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=256)
    ids = _ids(90, ROBOPEL_CONFIGS[name][0]["vocab"], 8)
    want, twin = [], []
    plain.logits(ids, stream_after=want)
    plain.logits(ids, R.bf16_round, stream_after=twin)  # what rounding to bfloat16 alone does to the stream behind each layer
    seen = []
    for block in engine.model.layers:
        def watched(stream, ctx, view, rt, following=None, inner=block.forward):
            out = inner(stream, ctx, view, rt, following=following)
            seen.append((out.x if isinstance(out, PreparedRows) else out[0]).clone())
            return out
        block.forward = watched
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, ids, [0])])
    assert len(seen) == len(want) == len(ROBOPEL_CONFIGS[name][0]["layers"])
    for run, (got, expected, rounded) in enumerate(zip(seen, want, twin)):
        assert _relative(got.cpu(), expected) < (1e-5 if dtype == "float32" else max(1e-2, 3.0 * _relative(rounded, expected))), f"layer {run}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(ROBOPEL_CONFIGS))
def test_prompts_whole_in_portions_and_token_by_token(folders, name, dtype):
    config = ROBOPEL_CONFIGS[name][0]
    plain = R.PlainRobopel(folders[name])
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
@pytest.mark.parametrize("name", ["A", "C"])
def test_unequal_batches_equal_each_request_alone(folders, name, dtype):
    """Requests of different lengths start together, are decoded together and end one after the other; their slots,
    pages and states go to requests that start later.  Every logit equals the plain model's on that request alone."""
    from nnis_amd.engine.batch import StepEntry

    config = ROBOPEL_CONFIGS[name][0]
    plain = R.PlainRobopel(folders[name])
    engine = nnis_amd.load_engine(folders[name], dtype=dtype, max_tokens=64 * 9, max_slots=4)
    yard = Yardstick(plain)
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
        assert engine.free_slots() == 4 and engine.free_pages() == 9


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_across_windows_pages_and_pooled_pages(tmp_path, dtype):
    """330 tokens one by one behind a prompt of 3: windows of 5 and 70 tokens pass over decoded tokens; five page borders
    are crossed, and with blocks of 2 and of 1 tokens the pooled blocks' pages fill up and new ones begin (at 128 and 256
    tokens; at every 64)."""
    config = robopel(vocab=200, width=64, scale=4.0, layers=[
        layer("attention", attention(2, 1, 16, 16, scale=0.3, softcap=20.0, rot=(16, 1e4), window=5, pool=2), dense(40)),
        layer("mingru", {"width": 48}, moe(4, 2, 16, identity=1)),
        layer("attention", attention(2, 1, 16, 16, scale=0.3, rot=(16, 1e4), window=70, pool=1, kv_from=0))])
    folder = _folder(tmp_path / "m", config, 7)
    plain = R.PlainRobopel(folder)
    engine = nnis_amd.load_engine(folder, dtype=dtype, max_tokens=512)
    ids = _ids(330, config["vocab"], 4)
    slot = engine.start_sequence()
    got = _collect(engine, slot, ids, [3] + list(range(4, 331)))
    yard = Yardstick(plain)
    yard.check(got, ids, dtype, "long decoding")
    yard.check(got[-1], ids, dtype, "long decoding, the last token", rows=len(ids) - 1)


@pytest.mark.parametrize("name", sorted(ROBOPEL_CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name):
    """``nnis_amd.generate``: the library's scheduler, batches and selection on the device.  In 32-bit the tokens are
    the plain model's, unless two logits are closer than rounding."""
    config = ROBOPEL_CONFIGS[name][0]
    plain = R.PlainRobopel(folders[name])
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
    plain = R.PlainRobopel(folders["B"])
    assert [int(t) for t in done.stdout.strip().splitlines()[-1].split(",")] == plain.greedy([5, 17, 3], 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_runner_replays_schedules(folders, tmp_path, dtype):
    """The same requests whole, with their last tokens one by one, and in unequal batches whose slots are used again,
    through ``bin/trace_run`` in a cache too small to hold the schedules side by side."""
    config = ROBOPEL_CONFIGS["A"][0]
    plain = R.PlainRobopel(folders["A"])
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
    """No embedding scale, no cap, no rotation, no window (so no pooled blocks), no identity outputs, a layer without a
    feed-forward: the sink, the norms of queries and keys and the gates stay."""
    config = robopel(vocab=120, width=48, layers=[
        layer("attention", attention(2, 1, 16, 32, scale=0.3), moe(3, 2, 24)),
        layer("mingru", {"width": 40}),
        layer("attention", attention(2, 1, 16, 32, scale=0.2, window=30, kv_from=0), dense(56))])
    folder = _folder(tmp_path / "bare", config, 41)
    plain = R.PlainRobopel(folder)
    engine = nnis_amd.load_engine(folder, dtype=dtype, max_tokens=512)
    ids = _ids(100, config["vocab"], 6)
    slot = engine.start_sequence()
    got = _collect(engine, slot, ids, [70] + list(range(71, 101)))
    Yardstick(plain).check(got, ids, dtype, "a model without the optional mechanisms")


HEAD_SIZES = [(32, 16), (16, 48), (24, 40), (16, 16)]  # attention modules that are built beforehand


def test_other_sizes_drawn_from_a_seed(tmp_path):
    """Configurations whose every size is drawn at random, in 32-bit against the plain model: prompt, a portion, single tokens."""
    import random

    for seed in range(6):
        r = random.Random(seed)
        layers, owners = [], []
        for index in range(r.randint(1, 5)):
            mlp = r.choice([None, dense(r.randint(8, 90)), moe(r.randint(1, 6), 1, r.randint(4, 40), identity=r.choice([None, 0, 1, 3]))])
            if mlp and mlp["kind"] == "moe":
                mlp["router"]["top"] = r.randint(1, mlp["router"]["experts"] + (mlp["router"].get("identity") or 0))
            if r.random() < 0.6:
                window = r.choice([None, r.randint(1, 90)])
                pool = r.choice([None, r.randint(1, 40)]) if window else None
                if owners and r.random() < 0.5:
                    source = r.choice(owners)
                    base = layers[source]["mixer"]
                    mixer = attention(base["heads"], base["kv_heads"], base["dim"], base["vdim"], scale=r.uniform(0.05, 0.5),
                                      softcap=r.choice([None, r.uniform(5.0, 50.0)]), window=window, pool=pool, kv_from=source)
                    if "rot" in base:
                        mixer["rot"] = copy.deepcopy(base["rot"])
                else:
                    dim, vdim = r.choice(HEAD_SIZES)
                    rot = r.choice([None, (2 * r.randint(1, dim // 2), r.choice([50.0, 1e4, 1e6])),
                                    (dim, 1e4, (r.uniform(2.0, 16.0), 1.0, r.uniform(2.0, 8.0), r.choice([16, 64, 1024])))])
                    mixer = attention(r.randint(1, 3) * (k := r.randint(1, 2)), k, dim, vdim, scale=r.uniform(0.05, 0.5),
                                      softcap=r.choice([None, r.uniform(5.0, 50.0)]), rot=rot, window=window, pool=pool)
                    owners.append(index)
                layers.append(layer("attention", mixer, mlp))
            else:
                layers.append(layer("mingru", {"width": r.randint(1, 120)}, mlp))
        config = robopel(vocab=r.randint(20, 400), width=4 * r.randint(3, 30), layers=layers, scale=r.choice([None, 1.0, r.uniform(0.5, 20.0)]),
                         eps=r.choice([1e-5, 1e-6, 1e-3]))
        folder = _folder(tmp_path / f"m{seed}", config, seed)
        plain = R.PlainRobopel(folder)
        engine = nnis_amd.load_engine(folder, dtype="float32", max_tokens=256)
        ids = _ids(80, config["vocab"], seed)
        want = plain.logits(ids)
        slot = engine.start_sequence()
        got = _collect(engine, slot, ids, [66, 70] + list(range(71, 81)))
        assert _relative(got, want) < 5e-5, f"seed {seed}: {config}"
