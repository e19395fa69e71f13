"""Mafalorn, plainly: one function a mechanism over whole sequences in 64-bit,
written from the design's equations and sharing nothing with the library.

Notation.  x: the residual stream [tokens, width].  R(v, w) = v / sqrt(mean(v^2)
+ eps) * w.  A layer is x <- x + R(mixer(R(x, a1)), b1), then, where it has a
feed-forward, x <- x + R(ff(R(x, a2)), b2): every sublayer is normed on its
way in and on its way out.  ``rnd`` rounds where an engine that keeps
activations in bfloat16 rounds them (the identity by default).
"""

import json
import math
import os

import torch
from safetensors.torch import load_file


def identity(x):
    return x


def bf16_round(x):
    return x.to(torch.bfloat16).to(x.dtype)


def rms_norm(v, w, eps):
    out = v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return out if w is None else out * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def frequencies(rot):
    """f_i = base^(-2i / dims) for the pairs of a rotation, and the factor on cosine and sine.  With ``scaling``
    (factor, original, fast, slow) a frequency whose turns within ``original`` positions are few is divided by
    ``factor``, one with many stays, and those between are blended by a ramp over the pair's index."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    scaling = rot.get("scaling")
    if scaling is None:
        return torch.tensor(f, dtype=torch.float64), 1.0
    factor, original = scaling["factor"], scaling["original"]

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(scaling["fast"])), 0)
    hi = min(math.ceil(index_of(scaling["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def turn(x, positions, rot, layout):
    """x [tokens, heads, dim]: the first rot.dims channels of a head turn by position * f_i; ``layout`` "halves"
    pairs channel i with i + dims / 2, "neighbours" channel 2i with 2i + 1."""
    f, magnitude = frequencies(rot)
    dims = rot["dims"]
    angle = positions.double()[:, None] * f[None, :]
    c = (torch.cos(angle) * magnitude)[:, None, :].to(x.dtype)
    s = (torch.sin(angle) * magnitude)[:, None, :].to(x.dtype)
    out = x.clone()
    if layout == "halves":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def retention(h, w, sizes, eps, rnd=identity, first=0, state=None):
    """Linear attention with one fixed decay a head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; q and k turned
    (halves), k times dim^(-1/2); each head's o over its root mean square, times silu(Wg h), through Wo.
    Returns (out, state [heads, dim, vdim])."""
    n = h.shape[0]
    heads, dim, vdim = sizes["heads"], sizes["dim"], sizes["vdim"]
    positions = torch.arange(first, first + n)
    q, k = rnd(h @ w["q"].T).view(n, heads, dim), rnd(h @ w["k"].T).view(n, heads, dim)
    if sizes.get("rot") is not None:
        q, k = turn(q, positions, sizes["rot"], "halves"), turn(k, positions, sizes["rot"], "halves")
    k = k * dim ** -0.5
    v = rnd(h @ w["v"].T).view(n, heads, vdim)
    gate = silu(rnd(h @ w["g"].T))
    decay = torch.tensor(sizes["decay"], dtype=h.dtype)[:, None, None]
    S = torch.zeros(heads, dim, vdim, dtype=h.dtype) if state is None else state
    rows = []
    for t in range(n):
        S = decay * S + k[t][:, :, None] * v[t][:, None, :]
        rows.append(torch.einsum("hde,hd->he", S, q[t]))
    o = rms_norm(torch.stack(rows), None, eps).reshape(n, heads * vdim)
    return rnd(o * gate) @ w["o"].T, S


def softmax_attention(h, w, sizes, rnd=identity):
    """Grouped causal attention whose values are the keys as projected (before their rotation); rotation by halves
    with the scaled frequencies; one sigmoid gate a head.  w: q, k, g, o."""
    n = h.shape[0]
    heads, groups, dim = sizes["heads"], sizes["kv_heads"], sizes["dim"]
    positions = torch.arange(n)
    q = rnd(h @ w["q"].T).view(n, heads, dim)
    k = rnd(h @ w["k"].T).view(n, groups, dim)
    v = k
    if sizes.get("rot") is not None:
        q, k = rnd(turn(q, positions, sizes["rot"], "halves")), rnd(turn(k, positions, sizes["rot"], "halves"))
    gate = sigmoid(h @ w["g"].T)
    out = torch.zeros(n, heads, v.shape[-1], dtype=h.dtype)
    causal = positions[:, None] >= positions[None, :]
    for head in range(heads):
        g = head // (heads // groups)
        score = (q[:, head] @ k[:, g].T) * sizes["scale"]
        score = score.masked_fill(~causal, -math.inf)
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, g]
    out = out * gate[:, :, None]
    return rnd(out.reshape(n, -1)) @ w["o"].T


def short_convolution(x, taps):
    """x [tokens, channels], taps [channels, count]: causal per channel, the last tap on the token itself, zeros before."""
    count = taps.shape[1]
    padded = torch.cat([x.new_zeros(count - 1, x.shape[1]), x], dim=0)
    out = torch.zeros_like(x)
    for j in range(count):
        out = out + padded[j:j + x.shape[0]] * taps[:, j]
    return out


def gated_delta_rule(h, w, sizes, eps, rnd=identity):
    """Per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with q, k (kv_heads x dim) and v (heads x
    vdim) through a short convolution and silu, q and k made unit vectors (q also times dim^(-1/2)), beta =
    sigmoid(Wb h), g = exp(-exp(A_log) softplus(Wa h + dt_bias)); o over its root mean square times ``norm`` times
    silu(Wg h), through Wo."""
    n = h.shape[0]
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = rnd(silu(rnd(short_convolution(rnd(h @ w["q"].T), w["q.conv"])))).view(n, groups, dim)
    k = rnd(silu(rnd(short_convolution(rnd(h @ w["k"].T), w["k.conv"])))).view(n, groups, dim)
    v = rnd(silu(rnd(short_convolution(rnd(h @ w["v"].T), w["v.conv"])))).view(n, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    gate = silu(rnd(h @ w["g"].T)).view(n, heads, vdim)
    S = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    rows = []
    for t in range(n):
        row = []
        for head in range(heads):
            kk, qq = k[t, head // (heads // groups)], q[t, head // (heads // groups)]
            s = g[t, head] * S[head]
            u = beta[t, head] * (v[t, head] - s.T @ kk)
            S[head] = s + kk[:, None] * u[None, :]
            row.append(S[head].T @ qq)
        rows.append(torch.stack(row))
    o = rms_norm(torch.stack(rows), w["norm"], eps) * gate
    return rnd(o.reshape(n, heads * vdim)) @ w["o"].T


def parallel(h, w, sizes, eps, rnd=identity):
    left = softmax_attention(h, {k[5:]: v for k, v in w.items() if k.startswith("left.")}, sizes["left"], rnd)
    right = gated_delta_rule(h, {k[6:]: v for k, v in w.items() if k.startswith("right.")}, sizes["right"], eps, rnd)
    return sizes["left_scale"] * left + sizes["right_scale"] * right


def latent_attention(h, w, sizes, eps, rnd=identity):
    """A token keeps c = R(first kv_rank rows of Wdkv h, dkv.norm) and one key part of rot_dim channels, turned
    (neighbours); head by head k = [Uk c | that part], v = Uv c, q = [plain | turned]; a window of mask.size tokens;
    the heads' outputs times sigmoid(Wg h) element by element, through Wo."""
    n = h.shape[0]
    heads, dim, rot_dim, vdim, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    positions = torch.arange(n)
    q = rnd(h @ w["q"].T).view(n, heads, dim + rot_dim)
    down = h @ w["dkv"].T
    c = rnd(rms_norm(down[:, :rank], w["dkv.norm"], eps))
    shared = down[:, rank:].view(n, 1, rot_dim)
    q_plain, q_rot, k_rot = q[..., :dim], q[..., dim:], rnd(shared)
    if rot_dim:
        rot = dict(sizes["rot"], dims=rot_dim)
        q_rot, k_rot = turn(q_rot, positions, rot, "neighbours"), rnd(turn(shared, positions, rot, "neighbours"))
    k = (c @ w["uk"].T).view(n, heads, dim)
    v = (c @ w["uv"].T).view(n, heads, vdim)
    seen = positions[:, None] >= positions[None, :]
    mask = sizes.get("mask")
    if mask is not None:
        seen = seen & (positions[:, None] - positions[None, :] < mask["size"])
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        score = (q_plain[:, head] @ k[:, head].T + q_rot[:, head] @ k_rot[:, 0].T) * sizes["scale"]
        out[:, head] = torch.softmax(score.masked_fill(~seen, -math.inf), dim=-1) @ v[:, head]
    gate = sigmoid(h @ w["g"].T)
    return rnd(out.reshape(n, -1) * gate) @ w["o"].T


def chosen_outputs(s, correction, top, groups):
    """The indices of the ``top`` largest of s + correction among the outputs of the best ``keep`` of ``count`` equal
    groups of neighbours (a group's mark is its largest corrected score); the lower index on a tie."""
    choice = s + correction
    outputs = choice.shape[0]
    allowed = torch.ones(outputs, dtype=torch.bool)
    if groups is not None:
        count, keep = groups["count"], groups["keep"]
        size = outputs // count
        marks = choice.view(count, size).max(dim=1).values
        order = sorted(range(count), key=lambda i: (-marks[i].item(), i))[:keep]
        allowed = torch.zeros(outputs, dtype=torch.bool)
        for i in order:
            allowed[i * size:(i + 1) * size] = True
    ranked = sorted((i for i in range(outputs) if allowed[i]), key=lambda i: (-choice[i].item(), i))
    return ranked[:top]


def experts(h, w, mlp, rnd=identity):
    """s = softmax(Wr h) over experts and identity outputs; the chosen outputs' s weigh down_e(silu(gate_e h) * up_e h),
    or h itself for an identity output; not renormalised."""
    router = mlp["router"]
    count, identity_outputs = router["experts"], router.get("identity") or 0
    s = torch.softmax(h @ w["router"].T, dim=-1)
    correction = w["correction"] if "correction" in w else torch.zeros(count + identity_outputs, dtype=h.dtype)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e in chosen_outputs(s[t], correction, router["top"], router.get("groups")):
            if e >= count:
                out[t] += s[t, e] * h[t]
            else:
                inner = rnd(silu(rnd(h[t] @ w[f"e{e}.gate"].T)) * rnd(h[t] @ w[f"e{e}.up"].T))
                out[t] += s[t, e] * (inner @ w[f"e{e}.down"].T)
    return out


MIXERS = {"retention": retention, "parallel": parallel, "latent_attention": latent_attention}


def forward(config, weights, tokens, rnd=identity, layers_out=None):
    """Logits [tokens, vocab] of one sequence.  ``layers_out``: a list that receives the stream after every layer."""
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        own = {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}
        mix = {k[4:]: v for k, v in own.items() if k.startswith("mix.")}
        h = rnd(rms_norm(x, own["norm1"], eps))
        kind = layer["type"]
        if kind == "retention":
            y = retention(h, mix, layer["mixer"], eps, rnd)[0]
        else:
            y = MIXERS[kind](h, mix, layer["mixer"], eps, rnd)
        x = x + rms_norm(y, own["norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rnd(rms_norm(x, own["norm2"], eps))
            y = experts(h, {k[4:]: v for k, v in own.items() if k.startswith("mlp.")}, layer["mlp"], rnd)
            x = x + rms_norm(y, own["norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rnd(rms_norm(x, w["final.norm"], eps))
    return (h @ w["head"].T) * config.get("logit_scale", 1.0)


def load(folder):
    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    return config, load_file(os.path.join(folder, "model.safetensors"))


class PlainMafalorn:
    """The whole model over one sequence from its first token, from a folder with config.json and model.safetensors."""

    def __init__(self, folder):
        self.config, self.weights = load(folder)

    def logits(self, ids, rnd=identity, stream_after=None):
        """Logits [tokens, vocab]; ``stream_after`` (a list) gets the stream after every layer."""
        return forward(self.config, self.weights, list(ids), rnd, stream_after)

    def greedy(self, ids, count):
        ids, out = list(ids), []
        for _ in range(count):
            out.append(int(self.logits(ids)[-1].argmax()))
            ids.append(out[-1])
        return out
