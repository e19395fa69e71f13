"""Mixers that carry a state of fixed size from token to token instead of
keys and values: the selective scan, gated linear attention, retention, the
gated delta rule and the minGRU.  Their state
lives in the cache's per-slot regions (``StateRequest``), in 32-bit, zero when
a sequence starts; a step reads it at each sequence's first row and leaves it
behind the last, so a prompt gives the same in one step, in portions or token
by token.  Projections and the short convolution run in the activation type;
step sizes, decays, exponentials, the recurrences and the per-head norm are
32-bit under either runtime.
"""

from __future__ import annotations

import torch

from ..errors import InvalidInput, Unsupported
from ..weights.random_init import register_init_rule
from .base import Mixer, StateRequest, TensorSpec, register_part
from .linear import Projection


class SelectiveScan(Mixer):
    """Mamba's mixer.  With C channels, N states, R the rank of the step sizes:

        [x | z] = W_in h                                  x, z: C each
        x <- silu(conv(x) + b_conv)                       causal, per channel, ``taps`` wide, last tap on the token
        [dt | B | C] = W_x x                              R, N, N
        dt <- softplus(W_dt dt + b_dt)                    one step size a channel
        S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,   A = -exp(A_log)
        y_c = sum_n S[c, n] C_n + D_c x_c
        out = W_o (y * silu(z))

    State per sequence: S [C, N] and the convolution's last ``taps`` - 1 inputs."""

    graph_safe = True

    def __init__(self, width, channels, states, dt_rank, taps, w_in, conv, conv_bias, w_x, w_dt, dt_bias, a_log, d, w_out):
        self.width, self.channels, self.states = int(width), int(channels), int(states)
        self.dt_rank, self.taps = int(dt_rank), int(taps)
        if min(self.channels, self.states, self.dt_rank, self.taps) <= 0:
            raise InvalidInput("a selective scan needs positive sizes")
        self.names = dict(w_in=w_in, conv=conv, conv_bias=conv_bias, w_x=w_x, w_dt=w_dt, dt_bias=dt_bias, a_log=a_log, d=d, w_out=w_out)

    def tensors(self):
        C, N, R, n = self.channels, self.states, self.dt_rank, self.names
        return [
            TensorSpec(n["w_in"], (2 * C, self.width)),
            TensorSpec(n["conv"], (C, self.taps), init="conv_taps"),
            TensorSpec(n["conv_bias"], (C,)),
            TensorSpec(n["w_x"], (R + 2 * N, C)),
            TensorSpec(n["w_dt"], (C, R), init="step_matrix"),
            TensorSpec(n["dt_bias"], (C,), init="step_bias"),
            TensorSpec(n["a_log"], (C, N), init="log_rates"),
            TensorSpec(n["d"], (C,), init="gain"),
            TensorSpec(n["w_out"], (self.width, C)),
        ]

    def check(self, rt):
        if self.states > 128 or self.taps > 16:
            raise Unsupported(f"the scan kernels take up to 128 states and 16 taps, got {self.states} and {self.taps}")

    def bind(self, weights, rt):
        n, R = self.names, self.dt_rank
        self.w_in = Projection(weights[n["w_in"]], rt)
        self.conv = weights[n["conv"]].contiguous()
        self.conv_bias = weights[n["conv_bias"]].contiguous()
        # the low-rank step sizes and the read/write vectors leave separate projections: each output is then a matrix of its own
        self.w_dt_low = Projection(weights[n["w_x"]][:R].contiguous(), rt)
        self.w_bc = Projection(weights[n["w_x"]][R:].contiguous(), rt)
        self.w_dt = Projection(weights[n["w_dt"]], rt)
        self.dt_bias = weights[n["dt_bias"]].float().contiguous()
        self.A = (-torch.exp(weights[n["a_log"]].float())).contiguous()  # the rates, 32-bit, made once
        self.D = weights[n["d"]].float().contiguous()
        self.w_out = Projection(weights[n["w_out"]], rt)

    def weight_bytes(self):
        small = sum(t.numel() * t.element_size() for t in (self.conv, self.conv_bias, self.dt_bias, self.A, self.D))
        return small + sum(p.weight_bytes() for p in (self.w_in, self.w_dt_low, self.w_bc, self.w_dt, self.w_out))

    def cache_request(self):
        return (StateRequest((self.channels, self.states)), StateRequest((self.taps - 1, self.channels)))

    def forward(self, x, ctx, view, rt):
        scan_state, conv_state = view
        if scan_state.read_only:
            raise Unsupported("a selective scan cannot read another layer's state")
        tokens, C = x.shape[0], self.channels
        xz = self.w_in(x, rt)
        xc = rt.ops.conv_silu(xz, C, self.conv, self.conv_bias, conv_state.state if self.taps > 1 else None, ctx, rt.empty(tokens, C))
        low = self.w_dt_low(xc, rt)
        dt_pre = self.w_dt(low, rt, out_dtype=torch.float32)
        bc = self.w_bc(xc, rt, out_dtype=torch.float32)
        y = rt.ops.selective_scan(xc, dt_pre, bc, xz[:, C:], self.A, self.D, self.dt_bias, scan_state.state, ctx, rt.empty(tokens, C))
        return self.w_out(y, rt)


class GatedLinearAttention(Mixer):
    """Linear attention whose state decays per key channel.  With H heads, d key and e value channels a head:

        q = W_q h / sqrt(d),  k = W_k h,  v = W_v h
        alpha = sigmoid(W_a2 (W_a1 h) + b_a2)^(1 / tau)        per head and key channel
        S <- diag(alpha) S + k v^T,   o = S^T q                 per head, S [d, e]
        out = W_o (concat_h(o / rms(o) * w_norm) * silu(W_g h))

    the norm of a head's o over its e channels with a weight shared by the heads."""

    graph_safe = True

    def __init__(self, width, heads, key_dim, value_dim, tau, eps, q, k, v, g, o, norm, a1, a2, a2_bias, decay_rank=None):
        self.width, self.heads, self.key_dim, self.value_dim = int(width), int(heads), int(key_dim), int(value_dim)
        self.tau, self.eps = float(tau), float(eps)
        if min(self.heads, self.key_dim, self.value_dim) <= 0 or not self.tau > 0.0:
            raise InvalidInput("gated linear attention needs positive sizes and a positive tau")
        self.names = dict(q=q, k=k, v=v, g=g, o=o, norm=norm, a1=a1, a2=a2, a2_bias=a2_bias)
        # the inner size of the decays' two projections: None takes whatever the checkpoint's tensors have
        self.rank = None if decay_rank is None else int(decay_rank)

    def tensors(self):
        H, d, e, n = self.heads, self.key_dim, self.value_dim, self.names
        return [
            TensorSpec(n["q"], (H * d, self.width)),
            TensorSpec(n["k"], (H * d, self.width)),
            TensorSpec(n["v"], (H * e, self.width)),
            TensorSpec(n["g"], (H * e, self.width)),
            TensorSpec(n["o"], (self.width, H * e)),
            TensorSpec(n["norm"], (e,), init="gain"),
            TensorSpec(n["a1"], (self.rank, self.width)),
            TensorSpec(n["a2"], (H * d, self.rank)),
            TensorSpec(n["a2_bias"], (H * d,), init="decay_bias"),
        ]

    def check(self, rt):
        if self.key_dim > 256:
            raise Unsupported(f"the gated linear attention kernel takes up to 256 key channels a head, got {self.key_dim}")

    def bind(self, weights, rt):
        n = self.names
        # queries, keys, values and gates leave one projection; their columns are read in place
        self.qkvg = Projection(torch.cat([weights[n[key]] for key in ("q", "k", "v", "g")], dim=0), rt)
        if weights[n["a1"]].shape[0] != weights[n["a2"]].shape[1]:
            raise InvalidInput(f"{n['a1']} and {n['a2']} do not meet: {tuple(weights[n['a1']].shape)} and {tuple(weights[n['a2']].shape)}")
        self.a1 = Projection(weights[n["a1"]], rt)
        self.a2 = Projection(weights[n["a2"]], rt)
        self.a2_bias = weights[n["a2_bias"]].float().contiguous()
        self.norm = weights[n["norm"]].contiguous()
        self.out = Projection(weights[n["o"]], rt)

    def weight_bytes(self):
        return (sum(p.weight_bytes() for p in (self.qkvg, self.a1, self.a2, self.out))
                + self.a2_bias.numel() * 4 + self.norm.numel() * self.norm.element_size())

    def cache_request(self):
        return StateRequest((self.heads, self.key_dim, self.value_dim))

    def forward(self, x, ctx, view, rt):
        if view.read_only:
            raise Unsupported("gated linear attention cannot read another layer's state")
        H, d, e = self.heads, self.key_dim, self.value_dim
        tokens = x.shape[0]
        qkvg = self.qkvg(x, rt)
        logits = self.a2(self.a1(x, rt), rt, out_dtype=torch.float32)
        rt.ops.gla_decays(logits, self.a2_bias, self.tau)  # the decays' logarithms, once for all heads' blocks
        q, k = qkvg[:, :H * d], qkvg[:, H * d:2 * H * d]
        v, g = qkvg[:, 2 * H * d:2 * H * d + H * e], qkvg[:, 2 * H * d + H * e:]
        o = rt.ops.gla_scan(q, k, v, logits, d ** -0.5, view.state, ctx, H, rt.empty(tokens, H * e, dtype=torch.float32))
        gated = rt.ops.head_norm_gate(o, g, self.norm, self.eps, H, rt.empty(tokens, H * e))
        return self.out(gated, rt)


class Retention(Mixer):
    """Linear attention with one fixed decay a head and no softmax or denominator.  With H heads, d key and e value
    channels a head:

        q = rot(W_q h),  k = rot(W_k h) / sqrt(d),  v = W_v h      rot: the first channels of a head turned by the position
        S <- decay_h S + k v^T,   o = S^T q                        per head, S [d, e]
        out = W_o (concat_h(o / rms(o)) * silu(W_g h))

    the norm of a head's o over its e channels without a weight.  The state is that of gated linear attention and so
    is the kernel, with the decay a constant of the head and the rotation done while it stages queries and keys;
    rotation, state and norm are 32-bit under either runtime."""

    graph_safe = True

    def __init__(self, width, heads, key_dim, value_dim, decay, eps, q, k, v, g, o, position=None, positions=None):
        self.width, self.heads, self.key_dim, self.value_dim = int(width), int(heads), int(key_dim), int(value_dim)
        self.eps = float(eps)
        self.decay = [float(value) for value in decay]
        if min(self.heads, self.key_dim, self.value_dim) <= 0 or len(self.decay) != self.heads or not all(0.0 < d <= 1.0 for d in self.decay):
            raise InvalidInput("retention needs positive sizes and one decay in (0, 1] for every head")
        self.names = dict(q=q, k=k, v=v, g=g, o=o)
        self.position = None
        if position is not None:
            if positions is None or position not in positions:
                raise InvalidInput(f"retention names position encoding {position!r}, which the model does not define")
            self.position = positions[position]
            if getattr(self.position, "pairing", None) != "halves" or self.position.rot_dim > self.key_dim:
                raise InvalidInput("retention turns channel i with channel i + rot_dim / 2 of a head: the position encoding must say so and fit")
        self.qkvg = self.out = self.head_decay = None

    def tensors(self):
        H, d, e, n = self.heads, self.key_dim, self.value_dim, self.names
        return [TensorSpec(n["q"], (H * d, self.width)), TensorSpec(n["k"], (H * d, self.width)), TensorSpec(n["v"], (H * e, self.width)),
                TensorSpec(n["g"], (H * e, self.width)), TensorSpec(n["o"], (self.width, H * e))]

    def check(self, rt):
        if self.key_dim > 256:
            raise Unsupported(f"the retention kernel takes up to 256 key channels a head, got {self.key_dim}")

    def bind(self, weights, rt):
        n = self.names
        self.qkvg = Projection(torch.cat([weights[n[key]] for key in ("q", "k", "v", "g")], dim=0), rt)
        self.out = Projection(weights[n["o"]], rt)
        decay = torch.tensor(self.decay, dtype=torch.float64)
        self.head_decay = torch.stack([decay, torch.log(decay)]).to(torch.float32).to(rt.device).contiguous()

    def weight_bytes(self):
        return self.qkvg.weight_bytes() + self.out.weight_bytes()

    def cache_request(self):
        return StateRequest((self.heads, self.key_dim, self.value_dim))

    def forward(self, x, ctx, view, rt):
        if view.read_only:
            raise Unsupported("retention cannot read another layer's state")
        H, d, e = self.heads, self.key_dim, self.value_dim
        tokens = x.shape[0]
        rows = self.qkvg(x, rt)
        q, k = rows[:, :H * d], rows[:, H * d:2 * H * d]
        v, g = rows[:, 2 * H * d:2 * H * d + H * e], rows[:, 2 * H * d + H * e:]
        tables = self.position.rotary() if self.position is not None else None
        rotation = (tables.cos, tables.sin, tables.rot_dim) if tables is not None else None
        # (the keys' factor 1 / sqrt(d) rides on the queries: o is linear in both)
        o = rt.ops.gla_scan(q, k, v, None, d ** -0.5, view.state, ctx, H, rt.empty(tokens, H * e, dtype=torch.float32),
                            head_decay=self.head_decay, rotation=rotation)
        gated = rt.ops.head_norm_gate(o, g, None, self.eps, H, rt.empty(tokens, H * e))
        return self.out(gated, rt)


class GatedDeltaRule(Mixer):
    """The gated delta rule.  With H value heads of e channels on G query/key heads of d channels (value head h uses
    query/key head h // (H / G)):

        q, k, v = silu(conv(W_q h)), silu(conv(W_k h)), silu(conv(W_v h))     causal, per channel, ``taps`` wide, no bias
        q <- q / sqrt(sum q^2 + 1e-6) / sqrt(d),   k <- k / sqrt(sum k^2 + 1e-6)          per head
        beta = sigmoid(W_b h),   g = exp(-exp(A_log) softplus(W_a h + dt_bias))           one each a value head
        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q                   per head, S [d, e]
        out = W_o (concat_h(o / rms(o) * w_norm) * silu(W_g h))

    State per sequence: S, kept column by column as [H, e, d], and the convolution's last ``taps`` - 1 inputs.  Queries, keys, values and the gate
    leave one projection and one convolution; beta's and the decay's logits leave a second projection in 32-bit; unit
    vectors, beta, decays, the recurrence and the norm are 32-bit under either runtime."""

    graph_safe = True

    def __init__(self, width, heads, qk_heads, key_dim, value_dim, taps, eps, q, k, v, q_conv, k_conv, v_conv, b, a, a_log, dt_bias,
                 norm, g, o):
        self.width, self.heads, self.qk_heads = int(width), int(heads), int(qk_heads)
        self.key_dim, self.value_dim, self.taps, self.eps = int(key_dim), int(value_dim), int(taps), float(eps)
        if min(self.heads, self.qk_heads, self.key_dim, self.value_dim, self.taps) <= 0 or self.heads % self.qk_heads:
            raise InvalidInput("the gated delta rule needs positive sizes and value heads that divide among the query/key heads")
        self.names = dict(q=q, k=k, v=v, q_conv=q_conv, k_conv=k_conv, v_conv=v_conv, b=b, a=a, a_log=a_log, dt_bias=dt_bias,
                          norm=norm, g=g, o=o)
        self.channels = 2 * self.qk_heads * self.key_dim + self.heads * self.value_dim  # what the convolution runs over

    def tensors(self):
        H, G, d, e, n = self.heads, self.qk_heads, self.key_dim, self.value_dim, self.names
        return [
            TensorSpec(n["q"], (G * d, self.width)), TensorSpec(n["q_conv"], (G * d, self.taps), init="conv_taps"),
            TensorSpec(n["k"], (G * d, self.width)), TensorSpec(n["k_conv"], (G * d, self.taps), init="conv_taps"),
            TensorSpec(n["v"], (H * e, self.width)), TensorSpec(n["v_conv"], (H * e, self.taps), init="conv_taps"),
            TensorSpec(n["b"], (H, self.width)), TensorSpec(n["a_log"], (H,), init="small"), TensorSpec(n["norm"], (e,), init="gain"),
            TensorSpec(n["a"], (H, self.width)), TensorSpec(n["dt_bias"], (H,), init="small"),
            TensorSpec(n["g"], (H * e, self.width)), TensorSpec(n["o"], (self.width, H * e)),
        ]

    def check(self, rt):
        if self.key_dim > 256 or self.taps > 16:
            raise Unsupported(f"the gated delta rule's kernels take up to 256 key channels a head and 16 taps, got {self.key_dim} and {self.taps}")

    def bind(self, weights, rt):
        n = self.names
        self.qkvg = Projection(torch.cat([weights[n[key]] for key in ("q", "k", "v", "g")], dim=0), rt)
        self.conv = torch.cat([weights[n[key]] for key in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.ba = Projection(torch.cat([weights[n["b"]], weights[n["a"]]], dim=0), rt)
        self.rate = torch.exp(weights[n["a_log"]].float()).contiguous()  # 32-bit, made once
        self.dt_bias = weights[n["dt_bias"]].float().contiguous()
        self.norm = weights[n["norm"]].contiguous()
        self.out = Projection(weights[n["o"]], rt)

    def weight_bytes(self):
        small = sum(t.numel() * t.element_size() for t in (self.conv, self.rate, self.dt_bias, self.norm))
        return small + sum(p.weight_bytes() for p in (self.qkvg, self.ba, self.out))

    def cache_request(self):
        # (the matrix state lies column by column: a value channel's key rows are consecutive)
        return (StateRequest((self.heads, self.value_dim, self.key_dim)), StateRequest((self.taps - 1, self.channels)))

    def forward(self, x, ctx, view, rt):
        state, conv_state = view
        if state.read_only:
            raise Unsupported("the gated delta rule cannot read another layer's state")
        H, e, tokens = self.heads, self.value_dim, x.shape[0]
        rows = self.qkvg(x, rt)
        ba = self.ba(x, rt, out_dtype=torch.float32)
        qkv = rt.ops.conv_silu(rows, self.channels, self.conv, None, conv_state.state if self.taps > 1 else None, ctx,
                               rt.empty(tokens, self.channels))
        o = rt.ops.gated_delta(qkv, ba, self.rate, self.dt_bias, self.key_dim ** -0.5, state.state, ctx, H, self.qk_heads, self.key_dim,
                               e, rt.empty(tokens, H * e, dtype=torch.float32))
        gated = rt.ops.head_norm_gate(o, rows[:, self.channels:], self.norm, self.eps, H, rt.empty(tokens, H * e))
        return self.out(gated, rt)


class MinGRU(Mixer):
    """A gated recurrence whose gates read the current token only.  With C channels:

        z = sigmoid(W_z h + b_z),   u = W_x h + b_x,   c = u + 1/2 where u >= 0, sigmoid(u) below
        S <- (1 - z) S + z c                              element by element
        out = W_o (S * silu(W_g h))

    State per sequence: S [C], 32-bit, zero at the start.  The three projections of the input are one product; the
    gates, the candidate and the recurrence are 32-bit under either runtime."""

    graph_safe = True

    def __init__(self, width, channels, z, z_bias, x, x_bias, g, o):
        self.width, self.channels = int(width), int(channels)
        if min(self.width, self.channels) <= 0:
            raise InvalidInput("a minGRU needs positive sizes")
        self.names = dict(z=z, z_bias=z_bias, x=x, x_bias=x_bias, g=g, o=o)

    def tensors(self):
        C, n = self.channels, self.names
        return [TensorSpec(n["z"], (C, self.width)), TensorSpec(n["z_bias"], (C,), init="small"),
                TensorSpec(n["x"], (C, self.width)), TensorSpec(n["x_bias"], (C,), init="small"),
                TensorSpec(n["g"], (C, self.width)), TensorSpec(n["o"], (self.width, C))]

    def bind(self, weights, rt):
        n = self.names
        self.zxg = Projection(torch.cat([weights[n[key]] for key in ("z", "x", "g")], dim=0), rt)
        self.z_bias = weights[n["z_bias"]].float().contiguous()
        self.x_bias = weights[n["x_bias"]].float().contiguous()
        self.out = Projection(weights[n["o"]], rt)

    def weight_bytes(self):
        return self.zxg.weight_bytes() + self.out.weight_bytes() + 8 * self.channels

    def cache_request(self):
        return StateRequest((self.channels,))

    def forward(self, x, ctx, view, rt):
        if view.read_only:
            raise Unsupported("a minGRU cannot read another layer's state")
        rows = self.zxg(x, rt)
        y = rt.ops.min_gru(rows, self.z_bias, self.x_bias, view.state, ctx, rt.empty(x.shape[0], self.channels))
        return self.out(y, rt)


class SideBySide(Mixer):
    """Several mixers that read the same input; each output is divided by its
    root mean square over the model width and multiplied by a weight of its
    own, and the result is the mean of these -- or, with ``scales`` in the
    weights' place, the outputs are added as they are, each times its factor.
    The cache gives each branch what it asks for; the view is the tuple of
    their views.

    The branches do not depend on one another: the first runs on the stream
    the step is on, the others on a second stream of the same priority that
    forks from it and joins it again (also inside a captured step, where the
    fork and the join become edges of the graph), with scratch of their own
    (``ops.lane``) -- in steps of few rows; a long prompt's kernels fill the
    chip one after the other."""

    BESIDE_MOST_ROWS = 256  # steps of up to this many rows run the branches on two streams

    def __init__(self, width, eps, branches, weights=None, positions=None, scales=None):
        from .base import build_part

        if (weights is None) == (scales is None):
            raise InvalidInput("branches side by side are normed and weighted (weights), or added with a factor each (scales)")
        if not 1 <= len(branches) <= 4 or len(weights if scales is None else scales) != len(branches):
            raise InvalidInput("one to four branches side by side, each with a weight or a factor")
        self.width, self.eps = int(width), float(eps)
        self.branches = [build_part("mixer", description, positions=positions) for description in branches]
        self.scales = None if scales is None else [float(value) for value in scales]
        self.weight_names = list(weights or [])
        self.weights = None
        self.graph_safe = all(getattr(branch, "graph_safe", False) for branch in self.branches)
        self._beside = None  # the second stream, made at the first step

    def tensors(self):
        out = [spec for branch in self.branches for spec in branch.tensors()]
        return out + [TensorSpec(name, (self.width,), init="gain") for name in self.weight_names]

    def bind(self, weights, rt):
        for branch in self.branches:
            branch.bind(weights, rt)
        self.weights = [weights[name].contiguous() for name in self.weight_names]

    def weight_bytes(self):
        return sum(branch.weight_bytes() for branch in self.branches) + sum(w.numel() * w.element_size() for w in self.weights)

    def check(self, rt):
        for branch in self.branches:
            branch.check(rt)

    def cache_request(self):
        return tuple(branch.cache_request() for branch in self.branches)

    def decode_plan(self, batch, longest, rt):
        plans = tuple(branch.decode_plan(batch, longest, rt) for branch in self.branches)
        return None if all(plan is None for plan in plans) else plans

    def prompt_plan(self, batch, rows, longest, rt):
        plans = tuple(branch.prompt_plan(batch, rows, longest, rt) for branch in self.branches)
        return None if all(plan is None for plan in plans) else plans

    def held_buffers(self, rt):
        return [buffer for branch in self.branches for buffer in branch.held_buffers(rt)]

    def _run(self, branch, x, ctx, branch_view, rt):
        if self.scales is None and getattr(branch, "can_leave_bias", False):
            return branch.forward(x, ctx, branch_view, rt, bias_later=True), branch.output_bias
        return branch.forward(x, ctx, branch_view, rt), None

    def forward(self, x, ctx, view, rt):
        count = len(self.branches)
        results = [None] * count
        # (side by side pays for steps of few rows, whose kernels leave most of the chip idle: a decode step at batch 8
        # of 6 such layers of width 2,048 took 0.879 ms on one stream and 0.829 ms on two; a prompt of 2,048 tokens
        # 4.84 ms on one and 5.03 ms on two)
        if count > 1 and x.is_cuda and x.shape[0] <= self.BESIDE_MOST_ROWS:
            if self._beside is None:
                self._beside = torch.cuda.Stream(device=x.device)
            main = torch.cuda.current_stream(x.device)
            self._beside.wait_stream(main)  # fork: what made x is done before the branches beside start
            with torch.cuda.stream(self._beside), rt.ops.lane(1):
                for index in range(1, count):
                    results[index] = self._run(self.branches[index], x, ctx, view[index], rt)
            results[0] = self._run(self.branches[0], x, ctx, view[0], rt)
            main.wait_stream(self._beside)  # join
        else:
            for index in range(count):
                results[index] = self._run(self.branches[index], x, ctx, view[index], rt)
        outputs, biases = [r[0] for r in results], [r[1] for r in results]
        if self.scales is not None:
            return rt.ops.branch_sum(outputs, self.scales, rt.empty(x.shape[0], self.width))
        return rt.ops.branch_mean(outputs, self.weights, biases, self.eps, rt.empty(x.shape[0], self.width))


def _noise(spec, generator):
    return torch.randn(tuple(spec.shape), generator=generator, dtype=torch.float32)


# what a random model of these mixers draws: taps and step sizes large enough to matter, rates spread over the
# states, decays near one
register_init_rule("conv_taps", lambda spec, generator, dtype: (0.3 * _noise(spec, generator)).to(dtype), replace=True)
register_init_rule("step_matrix", lambda spec, generator, dtype: (0.3 * _noise(spec, generator)).to(dtype), replace=True)
register_init_rule("step_bias", lambda spec, generator, dtype: (-2.0 + 0.5 * _noise(spec, generator)).to(dtype), replace=True)
register_init_rule(
    "log_rates",
    lambda spec, generator, dtype: (torch.log(torch.arange(1, spec.shape[-1] + 1, dtype=torch.float32)).expand(tuple(spec.shape))
                                    + 0.1 * _noise(spec, generator)).to(dtype), replace=True)
register_init_rule("decay_bias", lambda spec, generator, dtype: (2.0 + _noise(spec, generator)).to(dtype), replace=True)

register_part("mixer", "selective_scan", SelectiveScan)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "retention", Retention)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
register_part("mixer", "min_gru", MinGRU)
register_part("mixer", "side_by_side", SideBySide)
