"""Decode and prefill throughput of the Llama engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Default run: the SmolLM2-135M layer sizes (30 layers, hidden 576, 9 query and 3
key/value heads of 64, inner 1536, vocabulary 49152, tied head) with random
weights, a batch of 8 sequences whose prompts are uniform in [128, 2048]
tokens, in a cache sized for 8192 tokens per sequence.  A step is one decode
step of the whole batch through the generation path: token ids in, the model,
greedy selection on the device, token ids out to the host (which reads a
step's tokens while the next step, fed from the device, is under way, as the
generation loop does for greedy batches).  ``value`` is decoded tokens per
second over exactly K steps between two synchronisations; ``step_ms`` gives
the median, the least and the most of the steps' own times, taken with events
on the stream.  The prefill figure is one step over a 2,048-token prompt: the
time of a shape seen before (replayed from a captured graph where the engine
keeps one) and, beside it, of a shape seen for the first time.

``points`` holds, beside decode at batch 1 and 64 of the same shape, the same
four measurements at the SmolLM2-1.7B and TinyLlama-1.1B layer sizes (all
layers), each with the fraction of its roofline, and the TinyLlama workload
of 64 unequal prompts (16 to 1,024 tokens, prefilled in one step, decoded
until every sequence holds 2,048 tokens) run through ``nnis_amd.generate``.
For the SmolLM2 shapes there are further points at long contexts: decode at
batch 8 and 64 over prompts of 7,800 to 8,000 tokens (``*_ctx8k``) and a prompt
of 8,192 tokens in one step (``*_prefill_8192``).  A decode point is the
median of three windows of K steps, one after the other on the same batch; a
prefill figure is the median of seven runs of a shape seen before.
``--workload tinyllama-ragged`` runs that workload alone.

``--workload zifunex`` measures the Zifunex design (attention and a selective
scan side by side, gated linear attention, several residual streams) at two
sets of layer sizes of a real model's kind, each beside a Llama of the same
width, layers, heads, inner size and vocabulary: a prompt of 2,048 tokens in
one step and decode at batch 1, 8 and 64, all in one JSON line.

``--workload mutedra`` does the same for the Mutedra design (attention in a
window with kept first tokens, a bias by distance and a sink; attention over a
cached latent, plain and with a rotated part, a sink and gates; norms without
statistics before and after every sublayer).

``--workload robopel`` measures the Robopel design (attention with normed and
rotated heads, a window with pooled blocks, a sink and gated heads, some layers
reading an earlier layer's keys; minGRU; PolyNorm and routed feed-forwards;
norms on the sublayers' outputs only) beside a Mutedra of windowed-attention
layers of the same width, layers, heads, window, inner size and vocabulary.

``--workload mafalorn`` measures the Mafalorn design (retention; grouped
attention whose values are its keys beside the gated delta rule; attention
over a cached latent in a window with a gate element by element; experts chosen
among groups; RMS norms before and after every sublayer) beside a Zifunex of
the same width, layers, heads, state sizes, inner size and vocabulary.

Peaks used for the fractions are the published MI355X ones: HBM 8 TB/s; dense
matrix rate 2.5 PFLOP/s for bfloat16, 157.3 TFLOP/s for 32-bit.
"""

import argparse
import json
import os
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}
NAMES = {"smollm2-135m": "SmolLM2-135M", "smollm2-1.7b": "SmolLM2-1.7B", "tinyllama-1.1b": "TinyLlama-1.1B", "llama-8b": "Llama-8B"}
POINT_SHAPES = ("smollm2-135m", "smollm2-1.7b", "tinyllama-1.1b")  # the shapes whose figures go into `points` beside the headline's


def step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots."""
    h, nq, nkv, hd = (config[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim"))
    inner, vocab, layers = config["intermediate_size"], config["vocab_size"], config["num_hidden_layers"]
    per_token = 2 * ((nq + 2 * nkv) * hd * h + nq * hd * h + 3 * h * inner)
    total = 0
    for n in tokens_per_sequence:
        total += layers * (per_token * n + 2 * 2 * nq * hd * n * (n + 1) // 2)
    return total + 2 * wanted_rows * h * vocab


class Shape:
    """One model shape with random weights, loaded once; engines of any cache size share its weights."""

    def __init__(self, name, layers, dtype, seed, folder, config=None, context=None):
        """``config``: a config.json of any registered architecture instead of the preset ``name``; ``context``: how
        long its sequences may get here, where the configuration names no last position."""
        import nnis_amd
        from nnis_amd.api import load_model
        from nnis_amd.config import preset

        self.name = name
        self.config = preset(name) if config is None else config
        self.layers_of_model = self.config.get("num_hidden_layers")
        if layers:
            self.config["num_hidden_layers"] = layers
        self.dtype = dtype
        started = time.perf_counter()
        nnis_amd.write_random_model(folder, self.config, seed=seed)
        self.model, self.rt = load_model(folder, dtype=dtype)
        self.load_seconds = time.perf_counter() - started
        self.folder = folder
        self.context = context or self.config["max_position_embeddings"]
        self.vocab = self.model.spec.vocab_size

    def engine(self, max_tokens, max_slots=None):
        from nnis_amd.engine.step import Engine

        return Engine(self.model, self.rt, max_tokens=max_tokens, max_slots=max_slots)


PROMPT_STEP_MOST_TOKENS = 16384  # a batch's prompts go in one step up to this many tokens, in several beyond


def decode_run(shape, rng, batch, steps, warmup, prompt_min, prompt_max, windows=1):
    """Prefills ``batch`` prompts (in one step where they are 16k tokens or fewer between them), then times
    ``windows`` windows of ``steps`` decode steps each, one after the other, and reports the median window.
    Returns a dict."""
    import torch

    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.sampling.device import DeviceSelector

    longest = min(prompt_max, shape.context - (windows + 1) * steps - warmup - 1)
    shortest = max(1, min(prompt_min, longest))
    lengths = rng.integers(shortest, longest + 1, size=batch).tolist()
    engine = shape.engine(batch * shape.context, max_slots=batch)  # every sequence may grow to the model's context
    selector = DeviceSelector(engine)
    slots = [engine.start_sequence() for _ in range(batch)]
    prompts = [rng.integers(0, shape.vocab, size=n).tolist() for n in lengths]
    rows, group, held = [], [], 0
    for slot, prompt in zip(slots, prompts):
        if group and held + len(prompt) > PROMPT_STEP_MOST_TOKENS:
            rows.append(engine.step([StepEntry(s, p, None) for s, p in group]))
            group, held = [], 0
        group.append((slot, prompt))
        held += len(prompt)
    rows.append(engine.step([StepEntry(s, p, None) for s, p in group]))
    logits = rows[0] if len(rows) == 1 else torch.cat(rows)
    greedy = [None] * batch
    sync = torch.cuda.synchronize
    if engine.use_graphs:
        # as the generation loop runs greedy batches: a step ahead of the host, which reads a
        # step's tokens while the next step, fed from the device, is under way
        pending = selector.select_start(logits, slots, greedy)

        def one_step(pending):
            following = selector.select_start(engine.step_from_device(slots, pending.device), slots, greedy)
            pending.result()
            return following

        def finish(pending):
            pending.result()
    else:
        pending = selector.select(logits, slots, greedy)

        def one_step(tokens):
            logits = engine.step_view([StepEntry(s, [t], None) for s, t in zip(slots, tokens)])
            return selector.select(logits, slots, greedy)

        def finish(tokens):
            pass

    for _ in range(warmup):
        pending = one_step(pending)
    finish(pending)
    # the graphs of the lengths that the timed steps (and the pass with events) reach are captured before the clock
    # starts: as the sequences grow a step may cross into another plan of the attention, whose first use costs 8 ms
    reached = max(engine.length(s) for s in slots)
    for ahead in range(1, min((windows + 1) * steps + 1, shape.context - reached) + 1):
        engine.prepare_decode(batch, reached + ahead)
    timed = []
    for _ in range(windows):
        sync()
        start = time.perf_counter()
        for _ in range(steps):
            pending = one_step(pending)
        finish(pending)
        sync()
        seconds = time.perf_counter() - start
        # (seconds, tokens held on average over the window's steps)
        timed.append((seconds, sum(engine.length(s) for s in slots) - batch * steps / 2.0))
    seconds, context_tokens = sorted(timed)[len(timed) // 2]
    # the steps' own times, in a pass of its own (an event on the stream after every step costs the step a little)
    spread = min(steps, shape.context - max(engine.length(s) for s in slots) - 1)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(spread + 1)]
    marks[0].record()
    for index in range(spread):
        pending = one_step(pending)
        marks[index + 1].record()
    finish(pending)
    sync()
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(spread)) or [1000.0 * seconds / steps]
    step_bytes = engine.model.step_weight_bytes() + engine.cache.bytes_per_token() * context_tokens
    del engine, selector
    torch.cuda.empty_cache()
    per_step = seconds / steps
    return {
        "tokens_per_second": batch * steps / seconds, "ms_per_step": 1000.0 * per_step, "lengths": lengths,
        "prompt_min": shortest, "prompt_max": longest, "gbs": step_bytes / per_step / 1e9,
        "step_ms": {"median": round(each[len(each) // 2], 4), "min": round(each[0], 4), "max": round(each[-1], 4)},
    }


def prefill_run(shape, rng, tokens=2048):
    """One prompt of ``tokens`` tokens in one step, logits at the last place: the first time its shape comes
    and once it has come before."""
    import torch

    from nnis_amd.engine.batch import StepEntry

    tokens = min(tokens, shape.context)
    engine = shape.engine(tokens)
    prompt = rng.integers(0, shape.vocab, size=tokens).tolist()
    warm = rng.integers(0, shape.vocab, size=max(1, tokens // 2 - 7)).tolist()
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, warm, None)])  # another shape: kernels loaded, buffers made
    engine.end_sequence(slot)
    times = []
    for _ in range(10):
        slot = engine.start_sequence()
        torch.cuda.synchronize()
        start = time.perf_counter()
        engine.step([StepEntry(slot, prompt, None)])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - start)
        engine.end_sequence(slot)
    del engine
    torch.cuda.empty_cache()
    seconds = sorted(times[3:])[3]  # the median of seven runs of a shape that has come before (and is captured, where it is)
    flops = {"Zifunex": zifunex_step_flops, "Mutedra": mutedra_step_flops, "Robopel": robopel_step_flops,
             "Mafalorn": mafalorn_step_flops}.get(shape.config.get("architecture"), step_flops)(
        shape.config, [tokens], 1)
    return {"value": round(tokens / seconds, 1), "tokens": tokens, "ms": round(1000.0 * seconds, 3),
            "frac": round(flops / seconds / FLOP_PEAK[shape.dtype], 5), "first_ms": round(1000.0 * times[0], 3)}


def ragged_run(shape, rng, sequences=64, shortest=16, longest=1024):
    """BASELINE's fifth configuration through the generation loop: ``sequences`` prompts of unequal lengths in
    one step, each decoded greedily until it holds the model's context; the live set shrinks as they end."""
    import torch

    from nnis_amd.engine.generate import GenerationRequest, generate

    total = shape.context
    lengths = rng.integers(shortest, min(longest, total - 1) + 1, size=sequences).tolist()
    prompts = [rng.integers(0, shape.vocab, size=n).tolist() for n in lengths]
    engine = shape.engine(sequences * total, max_slots=sequences)
    generate(engine, [GenerationRequest(p[:16], 2, ()) for p in prompts[:4]])  # kernels loaded

    def timed(requests):
        torch.cuda.synchronize()
        start = time.perf_counter()
        results = generate(engine, requests, max_batch=sequences)
        torch.cuda.synchronize()
        return time.perf_counter() - start, results

    first, _ = timed([GenerationRequest(p, 1, ()) for p in prompts])  # the prompts' step and one selection
    whole, results = timed([GenerationRequest(p, total - len(p), ()) for p in prompts])
    generated = sum(len(r.tokens) for r in results)
    assert all(len(r.tokens) == total - n for r, n in zip(results, lengths))
    del engine
    torch.cuda.empty_cache()
    decode_seconds = max(whole - first, 1e-9)
    return {
        "sequences": sequences, "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "prefill_tokens_per_second": round(sum(lengths) / first, 1), "prefill_ms": round(1000.0 * first, 2),
        "decode_tokens_per_second": round((generated - sequences) / decode_seconds, 1),
        "decode_steps": total - min(lengths) - 1, "seconds": round(whole, 3),
    }


# Zifunex at layer sizes of a real model's kind.  Per set: width, inner size of the feed-forwards, (query heads, key/value
# heads, key channels, value channels) of the attention, (channels, states, rank of the step sizes, taps) of the scan,
# (heads, key channels, value channels, rank of the decays) of the gated linear attention, streams.  Eight layers: two
# of attention and scan side by side for one of gated linear attention (which has no feed-forward), twice, then two more.
ZIFUNEX_SETS = {
    "w1024": dict(width=1024, ff=2816, attention=(16, 4, 64, 64), scan=(2048, 16, 64, 4), gla=(4, 128, 256, 32), streams=2),
    "w2048": dict(width=2048, ff=5632, attention=(16, 4, 128, 64), scan=(4096, 16, 128, 4), gla=(8, 128, 256, 32), streams=2),
}
ZIFUNEX_LAYERS = "PPGPPGPP"
ZIFUNEX_VOCAB = 32000
ZIFUNEX_CONTEXT = 8192  # how far a sequence of these measurements may grow (the design names no last position)


def zifunex_config(sizes):
    heads, kv_heads, dim, vdim = sizes["attention"]
    inner, states, dt_rank, taps = sizes["scan"]
    g_heads, g_dim, g_vdim, g_rank = sizes["gla"]
    side_by_side = {"type": "parallel", "mlp": {"kind": "dense", "ff": sizes["ff"]}, "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"dims": dim, "base": 10000.0},
                 "scale": dim ** -0.5, "softcap": 30.0},
        "right": {"inner": inner, "state": states, "dt_rank": dt_rank, "conv": taps}}}
    linear = {"type": "gla", "mlp": None, "mixer": {"heads": g_heads, "dim": g_dim, "vdim": g_vdim, "tau": 16.0, "rank": g_rank}}
    return {"architecture": "Zifunex", "vocab": ZIFUNEX_VOCAB, "width": sizes["width"], "streams": sizes["streams"], "norm": {"eps": 1e-5},
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 1000003, "mul_cur": 31}},
            "layers": [side_by_side if kind == "P" else linear for kind in ZIFUNEX_LAYERS]}


def llama_twin_config(sizes):
    """The closest model the library had: a Llama of the same width, layers, inner size and vocabulary, its heads those
    of the attention with the value's channels (so that the attention's outputs are as wide)."""
    from nnis_amd.config import preset

    heads, kv_heads, dim, vdim = sizes["attention"]
    return preset("tinyllama-1.1b", num_hidden_layers=len(ZIFUNEX_LAYERS), hidden_size=sizes["width"], num_attention_heads=heads,
                  num_key_value_heads=kv_heads, head_dim=max(dim, vdim), intermediate_size=sizes["ff"], vocab_size=ZIFUNEX_VOCAB,
                  max_position_embeddings=ZIFUNEX_CONTEXT, tie_word_embeddings=False)


def zifunex_step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots (projections, attention, the two recurrences)."""
    w = config["width"]
    total = 0
    for n in tokens_per_sequence:
        for layer in config["layers"]:
            if layer["type"] == "parallel":
                a, r = layer["mixer"]["left"], layer["mixer"]["right"]
                per_token = ((a["heads"] + a["kv_heads"]) * a["dim"] + a["kv_heads"] * a["vdim"]) * w + a["heads"] * a["vdim"] * w
                per_token += 2 * r["inner"] * w + (r["dt_rank"] + 2 * r["state"]) * r["inner"] + r["dt_rank"] * r["inner"] + r["inner"] * w
                per_token += 3 * r["inner"] * r["state"] + r["conv"] * r["inner"]
                total += 2 * per_token * n + 2 * a["heads"] * (a["dim"] + a["vdim"]) * n * (n + 1) // 2
            else:
                g = layer["mixer"]
                hd, he = g["heads"] * g["dim"], g["heads"] * g["vdim"]
                per_token = (2 * hd + 2 * he) * w + g["rank"] * (w + hd) + he * w + 2 * g["heads"] * g["dim"] * g["vdim"]
                total += 2 * per_token * n
            if layer["mlp"] is not None:
                total += 2 * 3 * w * layer["mlp"]["ff"] * n
    return total + 2 * wanted_rows * w * config["vocab"]


# Mutedra at two sets of layer sizes: W = attention in a window, L = attention over a latent, R = the same with a rotated
# part, a sink and gates; every layer with a feed-forward; one pass over all layers (its entry adds the pass's vector).
MUTEDRA_SETS = {
    "w1024": dict(width=1024, ff=2816, attention=(16, 4, 64, 64), window=(512, 4), bias=(128, 32), latent=(16, 64, 64, 384, 128, 32)),
    "w2048": dict(width=2048, ff=5632, attention=(16, 4, 128, 128), window=(1024, 4), bias=(128, 32), latent=(16, 128, 128, 768, 192, 64)),
}
MUTEDRA_LAYERS = "WLWRWLWR"


def mutedra_config(sizes):
    heads, kv_heads, dim, vdim = sizes["attention"]
    l_heads, l_dim, l_vdim, q_rank, kv_rank, rot = sizes["latent"]
    mlp = {"kind": "dense", "ff": sizes["ff"]}
    kinds = {
        "W": {"type": "attention", "mlp": mlp, "mixer": {
            "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "bias_max": sizes["bias"][0],
            "bias_buckets": sizes["bias"][1], "mask": {"size": sizes["window"][0], "keep_first": sizes["window"][1]}}},
        "L": {"type": "latent_attention", "mlp": mlp, "mixer": {
            "heads": l_heads, "dim": l_dim, "vdim": l_vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": l_dim ** -0.5}},
        "R": {"type": "latent_attention_2", "mlp": mlp, "mixer": {
            "heads": l_heads, "dim": l_dim, "vdim": l_vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": (l_dim + rot) ** -0.5,
            "rot_dim": rot, "rot": {"dims": rot, "base": 10000.0}}},
    }
    return {"architecture": "Mutedra", "vocab": ZIFUNEX_VOCAB, "width": sizes["width"], "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
            "logit_softcap": 30.0, "layers": [kinds[kind] for kind in MUTEDRA_LAYERS], "loop": {"start": 0, "stop": len(MUTEDRA_LAYERS), "times": 1}}


def mutedra_step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots, as the library computes them (the heads' key
    and value maps folded into the projections around the latent; a window's keys only as far as it reaches)."""
    w = config["width"]
    total = 0
    for n in tokens_per_sequence:
        for layer in config["layers"]:
            m = layer["mixer"]
            if layer["type"] == "attention":
                per_token = ((m["heads"] + m["kv_heads"]) * m["dim"] + m["kv_heads"] * m["vdim"]) * w + m["heads"] * m["vdim"] * w
                reach = m["mask"]["size"] + m["mask"]["keep_first"]
                keys = n * (n + 1) // 2 if n <= reach else reach * (reach + 1) // 2 + (n - reach) * reach
                total += 2 * per_token * n + 2 * m["heads"] * (m["dim"] + m["vdim"]) * keys
            else:
                rot = m.get("rot_dim", 0)
                per_token = (m["q_rank"] + m["kv_rank"] + rot) * w + m["heads"] * (m["kv_rank"] + rot) * m["q_rank"] + m["heads"] * m["kv_rank"] * w
                total += 2 * per_token * n + 2 * m["heads"] * (2 * m["kv_rank"] + rot) * n * (n + 1) // 2
            if layer["mlp"] is not None:
                total += 2 * 3 * w * layer["mlp"]["ff"] * n
    return total + 2 * wanted_rows * w * config["vocab"]


def mutedra_twin_config(sizes):
    """The closest model the library had: a Llama of the same width, layers, inner size and vocabulary, its heads those of
    the windowed attention."""
    from nnis_amd.config import preset

    heads, kv_heads, dim, vdim = sizes["attention"]
    return preset("tinyllama-1.1b", num_hidden_layers=len(MUTEDRA_LAYERS), hidden_size=sizes["width"], num_attention_heads=heads,
                  num_key_value_heads=kv_heads, head_dim=max(dim, vdim), intermediate_size=sizes["ff"], vocab_size=ZIFUNEX_VOCAB,
                  max_position_embeddings=ZIFUNEX_CONTEXT, tie_word_embeddings=False)


# Robopel at two sets of layer sizes: A = attention with keys of its own and a PolyNorm feed-forward, K = attention that
# reads the keys of the A before it, G = minGRU with a routed feed-forward (experts, chosen, identity outputs, inner
# size of an expert).  Windows with pooled blocks of 64 tokens; a bent rotation of the whole head.
ROBOPEL_SETS = {
    "w1024": dict(width=1024, ff=2816, attention=(16, 4, 64, 64), window=(512, 64), gru=1024, moe=(8, 2, 1, 704)),
    "w2048": dict(width=2048, ff=5632, attention=(16, 4, 128, 128), window=(1024, 64), gru=2048, moe=(8, 2, 1, 1408)),
}
ROBOPEL_LAYERS = "AGKGAGKG"


def robopel_config(sizes):
    heads, kv_heads, dim, vdim = sizes["attention"]
    experts, top, identity, expert_ff = sizes["moe"]
    layers, owner = [], None
    for index, kind in enumerate(ROBOPEL_LAYERS):
        if kind == "G":
            layers.append({"type": "mingru", "mixer": {"width": sizes["gru"]}, "mlp": {
                "kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "identity": identity}}})
            continue
        mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": 30.0,
                 "rot": {"dims": dim, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 2048}},
                 "mask": {"size": sizes["window"][0], "pool": sizes["window"][1]}}
        if kind == "K":
            mixer["kv_from"] = owner
        else:
            owner = index
        layers.append({"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": sizes["ff"]}})
    return {"architecture": "Robopel", "vocab": ZIFUNEX_VOCAB, "width": sizes["width"], "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
            "layers": layers}


def robopel_step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots: the projections, a window's keys and the
    pooled blocks before it, and of the experts those that a token has chosen (the library multiplies all of them)."""
    w = config["width"]
    total = 0
    for n in tokens_per_sequence:
        for layer in config["layers"]:
            m = layer["mixer"]
            if layer["type"] == "attention":
                own = 0 if m.get("kv_from") is not None else m["kv_heads"] * (m["dim"] + m["vdim"])
                per_token = (m["heads"] * m["dim"] + own + 2 * m["heads"] * m["vdim"]) * w
                size, pool = m["mask"]["size"], m["mask"]["pool"]
                keys = sum(min(i + 1, size) + max(0, i + 1 - size) // pool for i in range(n))
                total += 2 * per_token * n + 2 * m["heads"] * (m["dim"] + m["vdim"]) * keys
            else:
                total += 2 * 4 * m["width"] * w * n
            mlp = layer["mlp"]
            if mlp is not None and mlp["kind"] == "dense":
                total += 2 * 2 * w * mlp["ff"] * n
            elif mlp is not None:
                router = mlp["router"]
                total += 2 * (2 * w * mlp["expert"]["ff"] * router["top"] + (router["experts"] + router["identity"]) * w) * n
    return total + 2 * wanted_rows * w * config["vocab"]


def robopel_twin_config(sizes):
    """The closest model the library had: a Mutedra of windowed-attention layers (a sink, kept first tokens, a bias by
    distance) with gated feed-forwards, of the same width, layers, heads, window, inner size and vocabulary."""
    heads, kv_heads, dim, vdim = sizes["attention"]
    layer = {"type": "attention", "mlp": {"kind": "dense", "ff": sizes["ff"]}, "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "bias_max": 128, "bias_buckets": 32,
        "mask": {"size": sizes["window"][0], "keep_first": 4}}}
    return {"architecture": "Mutedra", "vocab": ZIFUNEX_VOCAB, "width": sizes["width"], "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
            "logit_softcap": 30.0, "layers": [layer] * len(ROBOPEL_LAYERS), "loop": {"start": 0, "stop": len(ROBOPEL_LAYERS), "times": 1}}


# Mafalorn at two sets of layer sizes: R = retention, P = attention whose values are its keys beside the gated delta
# rule, L = attention over a latent in a window; every layer with experts chosen among two groups.  Per set: retention
# (heads, key channels, value channels), the softmax side (query heads, key/value heads, channels, turned channels), the
# delta rule (value heads, query/key heads, key channels, value channels, taps), the latent (heads, plain key
# channels, turned channels, value channels, latent, window), experts (experts, chosen, identity outputs, inner size).
MAFALORN_SETS = {
    "w1024": dict(width=1024, retention=(4, 128, 256), softmax=(16, 4, 64, 64), delta=(8, 4, 64, 128, 4), latent=(16, 64, 32, 64, 128, 512),
                  moe=(8, 2, 2, 352)),
    "w2048": dict(width=2048, retention=(8, 128, 256), softmax=(16, 4, 128, 64), delta=(16, 8, 128, 128, 4), latent=(16, 128, 64, 128, 192, 1024),
                  moe=(8, 2, 2, 704)),
}
MAFALORN_LAYERS = "RPRLRPRL"


def mafalorn_config(sizes):
    r_heads, r_dim, r_vdim = sizes["retention"]
    heads, kv_heads, dim, turned = sizes["softmax"]
    d_heads, d_qk, d_dim, d_vdim, taps = sizes["delta"]
    l_heads, l_dim, l_rot, l_vdim, rank, window = sizes["latent"]
    experts, top, identity, expert_ff = sizes["moe"]
    mlp = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "identity": identity,
                                                                  "groups": {"count": 2, "keep": 1}}}
    kinds = {
        "R": {"type": "retention", "mlp": mlp, "mixer": {
            "heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": [1.0 - 2.0 ** (-5 - h) for h in range(r_heads)],
            "rot": {"dims": r_dim, "base": 10000.0}}},
        "P": {"type": "parallel", "mlp": mlp, "mixer": {
            "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                     "rot": {"dims": turned, "base": 10000.0, "scaling": {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}}},
            "right": {"heads": d_heads, "kv_heads": d_qk, "dim": d_dim, "vdim": d_vdim, "conv": taps},
            "left_scale": 0.7, "right_scale": 0.7}},
        "L": {"type": "latent_attention", "mlp": mlp, "mixer": {
            "heads": l_heads, "dim": l_dim, "rot_dim": l_rot, "vdim": l_vdim, "kv_rank": rank, "scale": (l_dim + l_rot) ** -0.5,
            "rot": {"dims": l_rot, "base": 10000.0}, "mask": {"size": window}}},
    }
    return {"architecture": "Mafalorn", "vocab": ZIFUNEX_VOCAB, "width": sizes["width"], "norm": {"eps": 1e-6}, "logit_scale": 0.5,
            "layers": [kinds[kind] for kind in MAFALORN_LAYERS]}


def mafalorn_step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots: the projections, the two recurrences, the
    softmax side's keys, a window's latents, and of the experts those that a token has chosen (the library multiplies
    all of them)."""
    w = config["width"]
    total = 0
    for n in tokens_per_sequence:
        for layer in config["layers"]:
            m = layer["mixer"]
            if layer["type"] == "retention":
                hd, he = m["heads"] * m["dim"], m["heads"] * m["vdim"]
                total += 2 * ((2 * hd + 3 * he) * w + 2 * m["heads"] * m["dim"] * m["vdim"]) * n
            elif layer["type"] == "parallel":
                a, r = m["left"], m["right"]
                per_token = (2 * a["heads"] + a["kv_heads"]) * a["dim"] * w
                per_token += (2 * r["kv_heads"] * r["dim"] + 3 * r["heads"] * r["vdim"] + 2 * r["heads"]) * w + 3 * r["heads"] * r["dim"] * r["vdim"]
                total += 2 * per_token * n + 2 * a["heads"] * 2 * a["dim"] * n * (n + 1) // 2
            else:
                per_token = (m["heads"] * (m["dim"] + m["rot_dim"]) + m["kv_rank"] + m["rot_dim"] + 2 * m["heads"] * m["vdim"]) * w
                per_token += m["heads"] * m["kv_rank"] * (m["dim"] + m["vdim"])
                size = (m.get("mask") or {}).get("size") or n
                keys = sum(min(i + 1, size) for i in range(n))
                total += 2 * per_token * n + 2 * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"]) * keys
            mlp = layer["mlp"]
            if mlp is not None:
                router = mlp["router"]
                total += 2 * (3 * w * mlp["expert"]["ff"] * router["top"] + (router["experts"] + router.get("identity", 0)) * w) * n
    return total + 2 * wanted_rows * w * config["vocab"]


def mafalorn_twin_config(sizes):
    """The closest model the library had: a Zifunex whose gated linear attention has retention's heads, whose attention
    has the softmax side's, whose scan stands where the delta rule and the latent do, and whose feed-forward's inner
    size is all the experts' together: the same width, layers and vocabulary."""
    r_heads, r_dim, r_vdim = sizes["retention"]
    heads, kv_heads, dim, _ = sizes["softmax"]
    experts, _, _, expert_ff = sizes["moe"]
    twin = dict(width=sizes["width"], ff=experts * expert_ff, attention=(heads, kv_heads, dim, dim), scan=(2 * sizes["width"], 16, sizes["width"] // 16, 4),
                gla=(r_heads, r_dim, r_vdim, 32), streams=1)
    config = zifunex_config(twin)
    side_by_side, linear = config["layers"][0], config["layers"][2]
    config["layers"] = [linear if kind == "R" else side_by_side for kind in MAFALORN_LAYERS]
    return config


def design_run(args, rng, design, sets, config_of, twin_of, twin="llama"):
    """Each set of sizes: the design's model and its Llama twin, a prompt of 2,048 tokens and decode at batch 1, 8, 64."""
    import torch

    out = {}
    for name, sizes in sets.items():
        for which, config in ((design, config_of(sizes)), (twin, twin_of(sizes))):
            torch.cuda.empty_cache()
            with tempfile.TemporaryDirectory() as folder:
                shape = Shape(f"{which}-{name}", 0, args.dtype, args.seed, folder, config=config, context=ZIFUNEX_CONTEXT)
                record = {"prefill_2048": prefill_run(shape, rng)}
                for batch in (1, 8, 64):
                    run = decode_run(shape, rng, batch, args.steps, args.warmup, args.prompt_min, args.prompt_max, windows=3)
                    record[f"decode_b{batch}"] = {"tokens_per_second": round(run["tokens_per_second"], 1), "ms_per_step": round(run["ms_per_step"], 4),
                                                  "hbm_frac": round(run["gbs"] / HBM_PEAK_GBS, 4)}
                record["step_weight_mb"] = round(shape.model.step_weight_bytes() / 1e6, 1)
                out[f"{which}-{name}"] = record
                del shape
    return out


def environment():
    import torch

    from nnis_amd.kernels import lib

    env = {"gpu": torch.cuda.get_device_name(0), "rocm": getattr(torch.version, "hip", None), "torch": torch.__version__,
           "kernels": lib.module_filename("core")}  # (named after a hash of the kernels' sources and flags)
    try:
        env["commit"] = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short=12", "HEAD"], capture_output=True, text=True,
                                       timeout=10).stdout.strip() or None
    except (OSError, subprocess.SubprocessError):
        env["commit"] = None
    if not env["commit"]:
        env["commit"] = os.environ.get("NNIS_COMMIT") or None  # a copy of the tree without its history: whoever made it may say
    return env


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", default="smollm2-135m", choices=sorted(NAMES), help="layer sizes of the model")
    parser.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all of them)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--no-points", action="store_true", help="only the headline: no further batches, shapes or workload")
    parser.add_argument("--no-other-shapes", action="store_true", help="points of the headline's shape only")
    parser.add_argument("--prompt-min", type=int, default=128, help="shortest prompt of the decode batches")
    parser.add_argument("--prompt-max", type=int, default=2048, help="longest prompt of the decode batches (within the context)")
    parser.add_argument("--workload", choices=["tinyllama-ragged", "zifunex", "mutedra", "robopel", "mafalorn"], help="run this workload alone")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import numpy as np

    rng = np.random.default_rng(args.seed)
    if args.workload == "zifunex":
        models = design_run(args, rng, "zifunex", ZIFUNEX_SETS, zifunex_config, llama_twin_config)
        head = models["zifunex-w2048"]["decode_b8"]
        print(json.dumps({
            "metric": "Zifunex at two sets of layer sizes beside a Llama of the same sizes: prefill of 2,048 tokens, decode at batch 1, 8, 64",
            "value": head["tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": head["ms_per_step"], "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights from a seed, uniform-random token ids",
            "config": {"model": "Zifunex, 8 layers of width 2048 (decode at batch 8)", "sets": ZIFUNEX_SETS, "layers": ZIFUNEX_LAYERS,
                       "vocab": ZIFUNEX_VOCAB, "context": ZIFUNEX_CONTEXT, "prompt_min": args.prompt_min, "prompt_max": args.prompt_max},
            "models": models, "env": environment()}))
        return 0
    if args.workload == "mutedra":
        models = design_run(args, rng, "mutedra", MUTEDRA_SETS, mutedra_config, mutedra_twin_config)
        head = models["mutedra-w2048"]["decode_b8"]
        print(json.dumps({
            "metric": "Mutedra at two sets of layer sizes beside a Llama of the same sizes: prefill of 2,048 tokens, decode at batch 1, 8, 64",
            "value": head["tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": head["ms_per_step"], "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights from a seed, uniform-random token ids",
            "config": {"model": "Mutedra, 8 layers of width 2048 (decode at batch 8)", "sets": MUTEDRA_SETS, "layers": MUTEDRA_LAYERS,
                       "vocab": ZIFUNEX_VOCAB, "context": ZIFUNEX_CONTEXT, "prompt_min": args.prompt_min, "prompt_max": args.prompt_max},
            "models": models, "env": environment()}))
        return 0
    if args.workload == "robopel":
        models = design_run(args, rng, "robopel", ROBOPEL_SETS, robopel_config, robopel_twin_config, twin="mutedra")
        head = models["robopel-w2048"]["decode_b8"]
        print(json.dumps({
            "metric": "Robopel at two sets of layer sizes beside a Mutedra of windowed attention of the same sizes: prefill of 2,048 tokens, decode at batch 1, 8, 64",
            "value": head["tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": head["ms_per_step"], "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights from a seed, uniform-random token ids",
            "config": {"model": "Robopel, 8 layers of width 2048 (decode at batch 8)", "sets": ROBOPEL_SETS, "layers": ROBOPEL_LAYERS,
                       "vocab": ZIFUNEX_VOCAB, "context": ZIFUNEX_CONTEXT, "prompt_min": args.prompt_min, "prompt_max": args.prompt_max},
            "models": models, "env": environment()}))
        return 0
    if args.workload == "mafalorn":
        models = design_run(args, rng, "mafalorn", MAFALORN_SETS, mafalorn_config, mafalorn_twin_config, twin="zifunex")
        head = models["mafalorn-w2048"]["decode_b8"]
        print(json.dumps({
            "metric": "Mafalorn at two sets of layer sizes beside a Zifunex of the same sizes: prefill of 2,048 tokens, decode at batch 1, 8, 64",
            "value": head["tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": head["ms_per_step"], "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights from a seed, uniform-random token ids",
            "config": {"model": "Mafalorn, 8 layers of width 2048 (decode at batch 8)", "sets": MAFALORN_SETS, "layers": MAFALORN_LAYERS,
                       "vocab": ZIFUNEX_VOCAB, "context": ZIFUNEX_CONTEXT, "prompt_min": args.prompt_min, "prompt_max": args.prompt_max},
            "models": models, "env": environment()}))
        return 0
    with tempfile.TemporaryDirectory() as folder:
        if args.workload == "tinyllama-ragged":
            shape = Shape("tinyllama-1.1b", args.layers, args.dtype, args.seed, folder)
            ragged = ragged_run(shape, rng)
            print(json.dumps({
                "metric": "TinyLlama-1.1B shape: 64 prompts of 16..1024 tokens in one step, decoded to 2048 tokens each",
                "value": ragged["decode_tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
                "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
                "data": "synthetic: random weights N(0, 0.02) from a seed, uniform-random token ids",
                "config": {"model": "TinyLlama-1.1B shape (Llama)", "layers": shape.config["num_hidden_layers"],
                           "layers_of_model": shape.layers_of_model, "global_batch": 64, "seq_len": shape.context},
                "workload": ragged, "env": environment()}))
            return 0

        shape = Shape(args.shape, args.layers, args.dtype, args.seed, folder)
        head = decode_run(shape, rng, args.batch, args.steps, args.warmup, args.prompt_min, args.prompt_max)
        prefill = prefill_run(shape, rng)
        points = {}

        def point_run(shape, batch, prompt_min=args.prompt_min, prompt_max=args.prompt_max):
            """A point beside the headline: the median of three windows on one batch."""
            return decode_run(shape, rng, batch, args.steps, args.warmup, prompt_min, prompt_max, windows=3)

        def long_points(shape, prefix):
            """Contexts near the model's end: decode over prompts of 7,800 to 8,000 tokens, and a prompt of 8,192."""
            if shape.context < 8192:
                return
            for batch in (8, 64):
                run = point_run(shape, batch, 7800, 8000)
                points[f"{prefix}decode_b{batch}_ctx8k"] = round(run["tokens_per_second"], 1)
                points[f"{prefix}decode_b{batch}_ctx8k_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
            long_prefill = prefill_run(shape, rng, tokens=8192)
            points[f"{prefix}prefill_8192"] = long_prefill["value"]
            points[f"{prefix}prefill_8192_frac"] = long_prefill["frac"]

        if not args.no_points:
            for batch in (1, 64):
                run = point_run(shape, batch)
                points[f"decode_b{batch}"] = round(run["tokens_per_second"], 1)
                points[f"decode_b{batch}_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
            long_points(shape, "")
        config, layers, layers_of_model = shape.config, shape.config["num_hidden_layers"], shape.layers_of_model
        del shape
    if not args.no_points and not args.no_other_shapes:
        import torch

        for other in POINT_SHAPES:
            if other == args.shape:
                continue
            torch.cuda.empty_cache()
            with tempfile.TemporaryDirectory() as folder:
                shape = Shape(other, 0, args.dtype, args.seed, folder)
                for batch in (1, 8, 64):
                    run = point_run(shape, batch)
                    points[f"{other}_decode_b{batch}"] = round(run["tokens_per_second"], 1)
                    points[f"{other}_decode_b{batch}_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
                other_prefill = prefill_run(shape, rng)
                points[f"{other}_prefill_{other_prefill['tokens']}"] = other_prefill["value"]
                points[f"{other}_prefill_{other_prefill['tokens']}_frac"] = other_prefill["frac"]
                long_points(shape, f"{other}_")
                if other == "tinyllama-1.1b":
                    ragged = ragged_run(shape, rng)
                    points["tinyllama-1.1b_ragged64_prefill"] = ragged["prefill_tokens_per_second"]
                    points["tinyllama-1.1b_ragged64_decode"] = ragged["decode_tokens_per_second"]
                del shape

    record = {
        "metric": f"decode tok/s at batch {args.batch} ({NAMES[args.shape]} shape); prefill tok/s at {prefill['tokens']} tokens; "
                  "decode at batch 1 and 64, and the other shapes, in points",
        "value": round(head["tokens_per_second"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02) from a seed, uniform-random token ids",
        "config": {
            "model": f"{NAMES[args.shape]} shape (Llama)", "layers": layers, "layers_of_model": layers_of_model,
            "hidden": config["hidden_size"], "heads": config["num_attention_heads"], "kv_heads": config["num_key_value_heads"],
            "head_dim": config["head_dim"], "inner": config["intermediate_size"], "vocab": config["vocab_size"],
            "tied_head": config["tie_word_embeddings"], "context": config["max_position_embeddings"],
            "global_batch": args.batch, "seq_len": config["max_position_embeddings"], "prompt_min": head["prompt_min"],
            "prompt_max": head["prompt_max"], "mean_prompt": round(float(np.mean(head["lengths"])), 1),
            "parallelism": "single GPU", "sampling": "greedy on device",
        },
        "step_ms": head["step_ms"],
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(head["gbs"] / HBM_PEAK_GBS, 5)},
        "points": points,
        "env": environment(),
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
