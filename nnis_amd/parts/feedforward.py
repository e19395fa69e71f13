"""Gated feed-forward: down( act(gate x) * up x ), act = SiLU
(/root/reference/crates/nnis-model/src/runtime.rs:1054-1087;
/root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28), the tanh form
of GELU, or ReLU.  Gate and up are one fused projection whose first ``inner`` output
columns are the gate."""

from __future__ import annotations

import torch

from ..errors import InvalidInput, Unsupported
from ..weights.random_init import register_init_rule
from .base import FeedForward, TensorSpec, register_part
from .linear import Projection


class GatedFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, width, inner, gate, up, down, activation="silu"):
        if activation not in ("silu", "gelu_tanh", "relu"):
            raise Unsupported(f"gated feed-forward activation {activation!r}; silu, gelu_tanh and relu are built")
        self.activation = activation
        self.width, self.inner = int(width), int(inner)
        self.names = {"gate": gate, "up": up, "down": down}
        self.gate_up = None
        self.down = None

    def tensors(self):
        return [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]

    def bind(self, weights, rt):
        if rt.dtype == torch.bfloat16:
            rt.ops.unit_rows(rt.device)  # (made here, outside any captured step)
        self.gate_up = Projection(torch.cat([weights[self.names["gate"]], weights[self.names["up"]]], dim=0), rt)
        self.down = Projection(weights[self.names["down"]], rt)

    def weight_bytes(self):
        return self.gate_up.weight_bytes() + self.down.weight_bytes()

    takes_pending_norm = True
    adds_to_residual = True

    def forward(self, x, ctx, rt, into=None):
        from .lazy import PendingNorm

        if isinstance(x, PendingNorm) and self.activation == "silu" and x.can_fuse(self.gate_up.weight):
            # (residual sum,) norm, both projections and the gating in one kernel
            hidden = x.fused(self.gate_up.weight, rt.empty(x.rows, self.inner), rt.ops.EPILOGUE_SILU)
        else:
            if isinstance(x, PendingNorm):
                x = x.materialize()
            ops = rt.ops
            if (rt.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and isinstance(self.gate_up.weight, ops.PackedWeight)
                    and 0 < x.shape[0] <= ops.UNIT_ROWS_MOST and x.is_contiguous() and x.data_ptr() % 16 == 0):
                # both projections with the gating in their epilogue, on rows that are normed already
                hidden = ops.gated_linear(x, self.gate_up.weight, rt.empty(x.shape[0], self.inner), self.activation)
            else:
                gate_up = self.gate_up(x, rt)
                hidden = ops.gated_act(gate_up, rt.empty(x.shape[0], self.inner), self.activation)
        if into is not None and into.can_take(hidden, self.down.weight):
            return into.take(hidden, self.down.weight)  # the down projection adds to the stream itself
        return self.down(hidden, rt)


register_part("feed_forward", "gated", GatedFeedForward)


class PolyNormFeedForward(FeedForward):
    """down(act(up x)) with act(z) = a N(z) + b N(z^2) + c N(z^3) + e: powers element by element, N a division of a
    token's inner row by its root mean square (eps inside the root); (a, b, c, e) are the four numbers of ``act``.
    The statistics and the polynomial are 32-bit."""

    graph_safe = True

    def __init__(self, width, inner, eps, up, down, act):
        self.width, self.inner, self.eps = int(width), int(inner), float(eps)
        self.names = {"up": up, "down": down, "act": act}
        self.up = self.down = self.coefficients = None

    def tensors(self):
        return [TensorSpec(self.names["up"], (self.inner, self.width)), TensorSpec(self.names["down"], (self.width, self.inner)),
                TensorSpec(self.names["act"], (4,), init="poly_coefficients")]

    def bind(self, weights, rt):
        self.up = Projection(weights[self.names["up"]], rt)
        self.down = Projection(weights[self.names["down"]], rt)
        self.coefficients = weights[self.names["act"]].float().contiguous()

    def weight_bytes(self):
        return self.up.weight_bytes() + self.down.weight_bytes() + 16

    def forward(self, x, ctx, rt):
        z = self.up(x, rt)
        return self.down(rt.ops.poly_norm(z, self.coefficients, self.eps, rt.empty(x.shape[0], self.inner)), rt)


class RoutedFeedForward(FeedForward):
    """A mixture of ``experts`` small feed-forwards, down_e(relu(up_e x)^2) or (``activation="silu_gated"``)
    down_e(silu(gate_e x) * up_e x), of which a token uses ``top``:

        s = softmax(W_r x) over experts + identity outputs       32-bit
        chosen = the ``top`` largest of s + correction           (the lower index on a tie)
        out = sum over chosen e of s_e * expert_e(x),            expert_e(x) = x for the last ``identity`` outputs

    The weights are the scores themselves, not renormalised; ``correction`` (a tensor's name or None) enters the
    choice only.  ``groups`` (count, keep): the outputs, identity outputs included, form ``count`` equal groups of
    neighbours; a group's mark is its largest corrected score, and only outputs of the ``keep`` groups with the largest
    marks can be chosen.  The experts' up projections are one product over all experts, gated row by row with the
    scores (zero for the experts not chosen) before one down projection over all of them."""

    graph_safe = True

    def __init__(self, width, inner, experts, top, router, up, down, identity=0, correction=None, activation="relu_squared", gate=None,
                 groups=None):
        """``up``, ``down`` and ``gate``: names with ``{}`` in the expert's place."""
        self.width, self.inner, self.experts, self.top, self.identity = int(width), int(inner), int(experts), int(top), int(identity or 0)
        if min(self.width, self.inner, self.experts, self.top) <= 0 or self.identity < 0 or self.top > self.experts + self.identity:
            raise InvalidInput(f"a router of {experts} experts and {identity} identity outputs cannot choose {top}")
        if activation not in ("relu_squared", "silu_gated") or (activation == "silu_gated") != (gate is not None):
            raise InvalidInput(f"experts are relu_squared, or silu_gated with gate projections; got {activation!r}")
        self.activation = activation
        self.groups = None
        if groups is not None and int(groups[0]) > 1:
            count, keep = int(groups[0]), int(groups[1])
            outputs = self.experts + self.identity
            if outputs % count or not 1 <= keep <= count or self.top > keep * (outputs // count):
                raise InvalidInput(f"{outputs} router outputs in {count} equal groups of which {keep} are kept cannot choose {top}")
            self.groups = (count, keep)
        self.names = {"router": router, "up": up, "down": down, "correction": correction, "gate": gate}

    def tensors(self):
        n, outputs = self.names, self.experts + self.identity
        out = [TensorSpec(n["router"], (outputs, self.width), init="router")]
        if n["correction"]:
            out.append(TensorSpec(n["correction"], (outputs,), init="small"))
        for e in range(self.experts):
            if n["gate"]:
                out.append(TensorSpec(n["gate"].format(e), (self.inner, self.width)))
            out += [TensorSpec(n["up"].format(e), (self.inner, self.width)), TensorSpec(n["down"].format(e), (self.width, self.inner))]
        return out

    def check(self, rt):
        if self.experts + self.identity > rt.ops.ROUTE_MOST_OUTPUTS or self.width > rt.ops.ROUTE_MOST_CHANNELS:
            raise Unsupported(f"the router kernels take up to {rt.ops.ROUTE_MOST_OUTPUTS} outputs of rows of up to "
                              f"{rt.ops.ROUTE_MOST_CHANNELS} channels, got {self.experts + self.identity} and {self.width}")

    def bind(self, weights, rt):
        n = self.names
        self.router = weights[n["router"]].float().contiguous()  # its logits are a 32-bit product under either runtime
        self.correction = weights[n["correction"]].float().contiguous() if n["correction"] else None
        # one product over all experts: expert by expert its up rows (behind its gate rows, where it has them)
        rows = [weights[name.format(e)] for e in range(self.experts) for name in ((n["gate"], n["up"]) if n["gate"] else (n["up"],))]
        self.up = Projection(torch.cat(rows, dim=0), rt)
        self.down = Projection(torch.cat([weights[n["down"].format(e)] for e in range(self.experts)], dim=1), rt)

    def weight_bytes(self):
        return self.up.weight_bytes() + self.down.weight_bytes() + self.router.numel() * 4

    can_leave_share = True  # ``forward(..., share_later=True)`` leaves the identity outputs' share to a consumer that adds it in a kernel of its own

    def forward(self, x, ctx, rt, share_later=False):
        """With ``share_later`` and identity outputs: returns (y, (keep, x)), where the output is y + keep[row] * x[row]."""
        tokens = x.shape[0]
        gates, keep = rt.empty(tokens, self.experts, dtype=torch.float32), rt.empty(tokens, dtype=torch.float32)
        if self.width <= rt.ops.ROUTE_FUSED_MOST_CHANNELS:
            rt.ops.route(x, self.router, self.correction, self.experts, self.top, gates, keep, groups=self.groups)
        else:
            logits = rt.ops.router_logits(x, self.router, rt.empty(tokens, self.experts + self.identity, dtype=torch.float32))
            rt.ops.route_top(logits, self.correction, self.experts, self.top, gates, keep, groups=self.groups)
        z = self.up(x, rt)
        y = self.down(rt.ops.routed_act(z, gates, rt.empty(tokens, self.experts * self.inner), self.activation), rt)
        if self.identity and share_later:
            return y, (keep, x)
        if self.identity:
            rt.ops.rows_axpy(y, x, keep)
        return y


# what a random model draws: coefficients of a size that matters, router rows that spread the scores
register_init_rule("poly_coefficients", lambda spec, generator, dtype: (0.5 + 0.25 * torch.randn(tuple(spec.shape), generator=generator)).to(dtype),
                   replace=True)
register_init_rule("router", lambda spec, generator, dtype: (0.3 * torch.randn(tuple(spec.shape), generator=generator)).to(dtype), replace=True)
register_part("feed_forward", "poly_norm", PolyNormFeedForward)
register_part("feed_forward", "routed", RoutedFeedForward)
