"""RMSNorm with a per-channel weight: y = x / sqrt(mean(x^2) + eps) * w
(/root/reference/crates/nnis-model/src/kernels.rs:15-48); with ``offset`` the
stored weight lies around zero and the gain is offset + w."""

from __future__ import annotations

import torch

from ..weights.random_init import register_init_rule
from .base import Norm, TensorSpec, register_part


class RMSNorm(Norm):
    graph_safe = True
    fusable_rms = True  # ``weight`` and ``eps`` are all a projection kernel needs to apply this norm itself

    def __init__(self, width: int, eps: float, weight: str, offset: float = 0.0):
        """``offset``: the gain is offset + weight (a weight stored around zero has an offset of 1); the sum is made
        once, in 32-bit, when the weights are bound, and such a norm is not taken into a projection's kernel."""
        self.width = int(width)
        self.eps = float(eps)
        self.weight_name = weight
        self.offset = float(offset)
        self.weight = None
        if self.offset:
            self.fusable_rms = False

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.width,), init="small" if self.offset else "gain")]

    def bind(self, weights, rt):
        self.weight = weights[self.weight_name].contiguous()
        if self.offset:
            self.weight = (self.weight.float() + self.offset).contiguous()

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def _out(self, x, rt, rows):
        count = x.shape[0] if rows is None else rows.shape[0]
        return rt.empty(count, self.width)

    def forward(self, x, rt, rows=None):
        return rt.ops.rmsnorm(x, self.weight, self.eps, self._out(x, rt, rows), rows=rows)

    def add_forward(self, residual, delta, rt, rows=None):
        return rt.ops.rmsnorm(residual, self.weight, self.eps, self._out(residual, rt, rows), delta=delta, rows=rows)

    def post_step(self, x, y, rt, share=None):
        """x += this norm of y, in place in the 32-bit stream; returns the new rows in the activation type (the stream
        itself under a 32-bit runtime): what a sublayer that reads the stream un-normed takes next.  ``share``: (a
        factor per row, rows): y stands for y + factor * rows (a sublayer's share of its own input, left to this kernel)."""
        if rt.dtype == torch.float32:
            rt.ops.rms_post_step(x, y, self.weight, 0.0, self.eps, share=share)
            return x
        return rt.ops.rms_post_step(x, y, self.weight, 0.0, self.eps, h=rt.empty(x.shape[0], self.width), share=share)


register_init_rule("small", lambda spec, generator, dtype: (0.1 * torch.randn(tuple(spec.shape), generator=generator)).to(dtype),
                   replace=True)
register_part("norm", "rms", RMSNorm)


class NoNorm(Norm):
    """The stream's rows as they are, in the activation type: what a sublayer
    reads that is normed on its way out only.  Under a 32-bit runtime that is
    the stream itself."""

    graph_safe = True

    def __init__(self, width: int):
        self.width = int(width)

    def forward(self, x, rt, rows=None):
        if rows is None and x.dtype == rt.dtype:
            return x
        count = x.shape[0] if rows is None else rows.shape[0]
        return rt.ops.cast_rows(x, rt.empty(count, self.width), rows)

    def add_forward(self, residual, delta, rt, rows=None):
        raise NotImplementedError("a stream that is read as it is has nothing left to add")


register_part("norm", "none", NoNorm)


class LayerNorm(Norm):
    """Layer norm with weight and bias: (x - mean) / sqrt(var + eps) * w + b, the
    variance being the mean squared deviation; ``centred=False`` leaves the mean
    in (an RMS norm, then with an optional bias).

    It also reads a residual kept as several streams ``[streams, tokens,
    width]``: what it norms is then u = sum_s take[s] x_s, ``take`` a tensor of
    the checkpoint, or the plain sum of the streams without one.  The streams'
    update by the sublayer before (``update_forward``) runs in the same kernel."""

    graph_safe = True

    def __init__(self, width: int, eps: float, weight: str, bias: str = None, centred: bool = True, streams: int = 1,
                 take: str = None):
        self.width, self.eps, self.centred, self.streams = int(width), float(eps), bool(centred), int(streams)
        self.weight_name, self.bias_name, self.take_name = weight, bias, take
        self.weight = self.bias = self.take = None

    def tensors(self):
        out = [TensorSpec(self.weight_name, (self.width,), init="gain")]
        if self.bias_name:
            out.append(TensorSpec(self.bias_name, (self.width,)))
        if self.take_name:
            out.append(TensorSpec(self.take_name, (self.streams,), init="stream_share"))
        return out

    def bind(self, weights, rt):
        self.weight = weights[self.weight_name].contiguous()
        self.bias = weights[self.bias_name].contiguous() if self.bias_name else None
        self.take = weights[self.take_name].float().contiguous() if self.take_name else None  # (the coefficients are kept in 32-bit)

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.weight, self.bias) if t is not None)

    def _streams(self, x):
        return x if x.dim() == 3 else x.unsqueeze(0)

    def forward(self, x, rt, rows=None):
        count = x.shape[-2] if rows is None else rows.shape[0]
        return rt.ops.stream_step(self._streams(x), rt.empty(count, self.width), take=self.take, weight=self.weight, bias=self.bias,
                                  eps=self.eps, centred=self.centred, rows=rows)

    def update_forward(self, x, y, mix, gain, rt):
        """x_t <- sum_s mix[s, t] x_s + gain[t] y for every stream, in place, and then this norm of the new streams."""
        return rt.ops.stream_step(x, rt.empty(x.shape[-2], self.width), y=y, mix=mix, gain=gain, take=self.take, weight=self.weight,
                                  bias=self.bias, eps=self.eps, centred=self.centred)

    def add_forward(self, residual, delta, rt, rows=None):
        import torch

        one = torch.ones(1, dtype=torch.float32, device=residual.device)
        if rows is None:
            return self.update_forward(self._streams(residual), delta, one, one, rt)
        rt.ops.stream_step(self._streams(residual), y=delta, mix=one, gain=one)
        return self.forward(residual, rt, rows=rows)


register_part("norm", "layer", LayerNorm)


class TanhNorm(Norm):
    """A norm without statistics: y = tanh(alpha x) * w + b, ``alpha`` one
    learned number, ``w`` and ``b`` per channel.  Nothing of a row is summed,
    so it rides in any kernel that touches the row once: ``ops.tanh_norm_step``
    takes a sublayer's output through one such norm into the stream and the
    stream through another into the next sublayer's input.  ``triple()`` is
    what that kernel needs of a norm."""

    graph_safe = True

    def __init__(self, width: int, weight: str, bias: str, alpha: str):
        self.width = int(width)
        self.weight_name, self.bias_name, self.alpha_name = weight, bias, alpha
        self.weight = self.bias = None
        self.alpha = 1.0

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.width,), init="gain"), TensorSpec(self.bias_name, (self.width,)),
                TensorSpec(self.alpha_name, (), init="tanh_alpha")]

    def bind(self, weights, rt):
        self.weight = weights[self.weight_name].contiguous()
        self.bias = weights[self.bias_name].to(self.weight.dtype).contiguous()
        self.alpha = float(weights[self.alpha_name].float().item())  # (a kernel argument: read once, when the model is loaded)

    def weight_bytes(self):
        return 2 * self.weight.numel() * self.weight.element_size()

    def triple(self):
        return self.alpha, self.weight, self.bias

    def forward(self, x, rt, rows=None):
        count = x.shape[0] if rows is None else rows.shape[0]
        out = rt.empty(count, self.width)
        if x.dtype == torch.float32:
            return rt.ops.tanh_norm_step(x, following=self.triple(), h=out, rows=rows)
        return rt.ops.tanh_norm_step(None, y=x, following=self.triple(), h=out, rows=rows)  # rows in the activation type

    def add_forward(self, residual, delta, rt, rows=None):
        """``delta``: a tensor, or a ``PostNormed`` (its norm then runs in the same kernel if it is of this kind)."""
        from .lazy import PostNormed

        post = None
        if isinstance(delta, PostNormed):
            if hasattr(delta.norm, "triple"):
                delta, post = delta.y, delta.norm.triple()
            else:
                delta = delta.materialize(rt)
        count = residual.shape[0] if rows is None else rows.shape[0]
        return rt.ops.tanh_norm_step(residual, x_out=residual if rows is None else None, y=delta, post=post,
                                     following=self.triple(), h=rt.empty(count, self.width), rows=rows)


# what a random model draws for alpha: around one half, so that tanh bends the stream's larger entries
register_init_rule("tanh_alpha", lambda spec, generator, dtype: (0.5 + 0.05 * torch.randn(tuple(spec.shape), generator=generator)).to(dtype),
                   replace=True)
register_part("norm", "dynamic_tanh", TanhNorm)
