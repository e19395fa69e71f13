"""Robopel, plainly: one function a mechanism over whole sequences in 64-bit,
written from the design's equations and sharing nothing with the library.

Notation.  x: the residual stream [tokens, width].  R(v, w) = v / sqrt(mean(v^2)
+ eps) * w.  A layer is x <- x + R(mixer(x), 1 + w1), then, where it has a
feed-forward, x <- x + R(ff(x), 1 + w2): the sublayers read the stream itself
and only their outputs are normed.  ``rnd`` rounds where an engine that keeps
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
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps) * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def min_gru(h, w, rnd=identity, state=None):
    """h [tokens, width].  w: z, z.b, x, x.b, g, o.  Element by element S_t = (1 - z_t) S_(t-1) + z_t c_t with
    z = sigmoid(Wz h + bz), c = u + 1/2 where u >= 0 and sigmoid(u) below, u = Wx h + bx; out = Wo (S_t * silu(Wg h)).
    Returns (out, last state)."""
    z = sigmoid(rnd(h @ w["z"].T + w["z.b"]))
    u = rnd(h @ w["x"].T + w["x.b"])
    c = torch.where(u >= 0, u + 0.5, sigmoid(u))
    gate = silu(rnd(h @ w["g"].T))
    s = torch.zeros(z.shape[1], dtype=h.dtype) if state is None else state
    rows = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * c[t]
        rows.append(s)
    out = rnd(torch.stack(rows) * gate) @ w["o"].T if rows else h.new_zeros(0, w["o"].shape[0])
    return out, s


def scaled_frequencies(dims, base, scaling):
    """f_i = base^(-2i / dims), each bent by its wavelength l = 2 pi / f: kept where l < original / high, divided by
    factor where l > original / low, between the two a blend by s = (original / l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            length = 2.0 * math.pi / f
            factor, low, high, original = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
            if length < original / high:
                pass
            elif length > original / low:
                f = f / factor
            else:
                s = (original / length - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def turn_neighbours(x, positions, frequencies):
    """x [tokens, heads, dim]: of the first 2 * len(frequencies) channels of a head, channel 2i turns with 2i + 1 by
    position * frequencies[i]; the others stay."""
    n = 2 * frequencies.shape[0]
    angle = positions.double()[:, None] * frequencies[None, :]
    c, s = torch.cos(angle)[:, None, :].to(x.dtype), torch.sin(angle)[:, None, :].to(x.dtype)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def keys_and_values(h, w, sizes, eps, rnd=identity, first=0):
    """What the cache holds of h's tokens: keys [tokens, kv_heads, dim] normed per head and turned, values as projected."""
    n = h.shape[0]
    groups, dim, vdim = sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    k = rnd(h @ w["k"].T).view(n, groups, dim)
    v = rnd(h @ w["v"].T).view(n, groups, vdim)
    k = rms_norm(k, w["k.norm"], eps)
    rot = sizes.get("rot")
    if rot is not None:
        k = turn_neighbours(k, torch.arange(first, first + n), scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling")))
    return rnd(k), v


def pooled_window_attention(h, w, sizes, eps, kv=None, rnd=identity):
    """h [tokens, width].  w: q, q.norm, sink, g, o and, unless ``kv`` brings another layer's cache, k, k.norm, v.
    Query i sees the keys j with 0 <= i - j < size and, for every block b of P tokens with b P + P - 1 <= i - size, one
    key and one value that are the block's means; all of them and the sink (exp(sink_h) in the denominator, no value)
    share one softmax of scores cap * tanh(q . k * scale / cap); the heads' outputs times sigmoid(Wg h) go through Wo.
    Returns (out, (keys, values))."""
    n = h.shape[0]
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = rms_norm(rnd(h @ w["q"].T).view(n, heads, dim), w["q.norm"], eps)
    rot = sizes.get("rot")
    if rot is not None:
        q = turn_neighbours(q, torch.arange(n), scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling")))
    q = rnd(q)
    if kv is None:
        kv = keys_and_values(h, w, sizes, eps, rnd)
    k, v = kv
    mask = sizes.get("mask")
    size = mask["size"] if mask else n + 1
    pool = mask.get("pool") if mask else None
    blocks = n // pool if pool else 0
    if blocks:
        pk = rnd(k[:blocks * pool].view(blocks, pool, groups, dim).mean(dim=1))
        pv = rnd(v[:blocks * pool].view(blocks, pool, groups, vdim).mean(dim=1))
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    near = (j <= i) & (i - j < size)
    b = torch.arange(blocks)[None, :]
    far = (b * pool + pool - 1 <= i - size) if blocks else torch.zeros(n, 0, dtype=torch.bool)
    cap = sizes.get("softcap")
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for head in range(heads):
        group = head // (heads // groups)
        s = q[:, head] @ k[:, group].T * sizes["scale"]
        seen, values = near, v[:, group]
        if blocks:
            s = torch.cat([s, q[:, head] @ pk[:, group].T * sizes["scale"]], dim=1)
            seen, values = torch.cat([near, far], dim=1), torch.cat([values, pv[:, group]], dim=0)
        if cap:
            s = cap * torch.tanh(s / cap)
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        sink = w["sink"][head] if "sink" in w else None
        top = s.max(dim=1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink)
        e = torch.exp(s - top)
        below = e.sum(dim=1, keepdim=True)
        if sink is not None:
            below = below + torch.exp(sink - top)
        out[:, head] = (e / below) @ values
    out = rnd(out.reshape(n, heads * vdim))
    if "g" in w:
        out = rnd(out * sigmoid(rnd(h @ w["g"].T)))
    return out @ w["o"].T, kv


def poly_norm_feed_forward(h, w, eps, rnd=identity):
    """Wdown act(Wup h), act(z) = a N(z) + b N(z^2) + c N(z^3) + e with powers element by element and N a division by
    the root mean square over the inner size."""
    z = rnd(h @ w["up"].T)
    a, b, c, e = [float(value) for value in w["act"]]
    one = torch.ones(z.shape[-1], dtype=z.dtype)
    act = a * rms_norm(z, one, eps) + b * rms_norm(z * z, one, eps) + c * rms_norm(z * z * z, one, eps) + e
    return rnd(act) @ w["down"].T


def routed_feed_forward(h, w, router, rnd=identity):
    """Scores s = softmax(Wrouter h) over experts + identity outputs; the ``top`` largest of s + correction are
    chosen; the output is the sum of s_e expert_e(h) over the chosen, an expert being Wdown relu(Wup h)^2 and each of
    the last ``identity`` outputs h itself.  Returns (out, chosen [tokens, top])."""
    experts, lazy, top = router["experts"], router.get("identity", 0), router["top"]
    s = torch.softmax(h @ w["router"].T, dim=-1)
    choice = s + w["correction"] if "correction" in w else s
    chosen = torch.topk(choice, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            if e >= experts:
                out[t] += s[t, e] * h[t]
            else:
                inner = torch.relu(rnd(w[f"e{e}.up"] @ h[t])) ** 2
                out[t] += s[t, e] * rnd(w[f"e{e}.down"] @ rnd(inner))
    return out, chosen


def _sub(weights, prefix):
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


class PlainRobopel:
    """The whole model over one sequence from its first token, from a folder with config.json and model.safetensors."""

    def __init__(self, folder):
        with open(os.path.join(folder, "config.json")) as handle:
            self.config = json.load(handle)
        self.w = {name: (value.double() if value.is_floating_point() else value)
                  for name, value in load_file(os.path.join(folder, "model.safetensors")).items()}

    def logits(self, ids, rnd=identity, stream_after=None):
        """Logits [tokens, vocab]; ``stream_after`` (a list) gets the stream after every layer."""
        cfg, w = self.config, self.w
        eps = cfg["norm"]["eps"]
        x = w["embed"][torch.as_tensor(list(ids), dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
        caches = {}
        for index, layer in enumerate(cfg["layers"]):
            prefix = f"l{index}."
            mix = _sub(w, prefix + "mix.")
            h = rnd(x)
            if layer["type"] == "mingru":
                y, _ = min_gru(h, mix, rnd)
            else:
                source = layer["mixer"].get("kv_from")
                y, caches[index] = pooled_window_attention(h, mix, layer["mixer"], eps, None if source is None else caches[source], rnd)
            x = x + rms_norm(y, 1.0 + w[prefix + "norm1"], eps)
            mlp = layer.get("mlp")
            if mlp is not None:
                h = rnd(x)
                if mlp["kind"] == "dense":
                    y = poly_norm_feed_forward(h, _sub(w, prefix + "mlp."), eps, rnd)
                else:
                    y, _ = routed_feed_forward(h, _sub(w, prefix + "mlp."), mlp["router"], rnd)
                x = x + rms_norm(y, 1.0 + w[prefix + "norm2"], eps)
            if stream_after is not None:
                stream_after.append(x.clone())
        return rms_norm(x, 1.0 + w["final.norm"], eps) @ w["head"].T

    def greedy(self, ids, count):
        ids, out = list(ids), []
        for _ in range(count):
            out.append(int(self.logits(ids)[-1].argmax()))
            ids.append(out[-1])
        return out
