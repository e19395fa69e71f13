"""The pre-norm arrangement of a layer:
x += mixer(norm1(x)); x += feed_forward(norm2(x))
(/root/reference/crates/nnis-model/src/runtime.rs:945-1095).

The residual stream is kept in 32-bit as a pair (x, pending): ``pending`` is a
part's output not yet added.  The sum is taken by the next norm in the same
kernel that normalises, and a mixer or feed-forward that starts with a
projection may take sum and norm into that projection's kernel
(``PendingNorm``), so the stream is read and written once per part.  A part
that ends with a projection (``adds_to_residual``) may go further and add its
output to the stream in that projection's kernel, which then also prepares
the norm that follows (``ResidualInto``); the block names that norm -- its own
second one, or the first of the block that comes next (``following``).
"""

from __future__ import annotations

import torch

from ..errors import InvalidInput
from ..weights.random_init import register_init_rule
from .base import Block, TensorSpec, build_part, register_part
from .lazy import PendingNorm, PostNormed, PreparedRows, PreparedStreams, ResidualInto, TanhInto


def _joined(plans):
    """The parts' plans as one: None where none of them plans anything, the
    plan itself where one part does (the mixer, as a rule)."""
    plans = tuple(plan for plan in plans if plan is not None)
    return None if not plans else (plans[0] if len(plans) == 1 else plans)


class PreNormBlock(Block):
    def __init__(self, width, norm1, mixer, norm2, feed_forward, positions=None):
        self.width = int(width)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer, positions=positions)
        self.norm2 = build_part("norm", norm2)
        self.feed_forward = build_part("feed_forward", feed_forward)
        self._parts = [self.norm1, self.mixer, self.norm2, self.feed_forward]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self._parts)

    def tensors(self):
        return [spec for part in self._parts for spec in part.tensors()]

    def bind(self, weights, rt):
        for part in self._parts:
            part.bind(weights, rt)

    def weight_bytes(self):
        return sum(part.weight_bytes() for part in self._parts)

    def cache_request(self):
        return self.mixer.cache_request()

    def check(self, rt):
        for part in self._parts:
            part.check(rt)

    def decode_plan(self, batch, longest, rt):
        return _joined(part.decode_plan(batch, longest, rt) for part in self._parts)

    def prompt_plan(self, batch, rows, longest, rt):
        return _joined(part.prompt_plan(batch, rows, longest, rt) for part in self._parts)

    def held_buffers(self, rt):
        return [buffer for part in self._parts for buffer in part.held_buffers(rt)]

    @property
    def entry_norm(self):
        """The norm a stream meets first here: a block before this one may prepare it."""
        return self.norm1

    def _run(self, part, normed, args, then, rt):
        """Runs a mixer or feed-forward on a pending norm; returns the pending
        norm ``then`` of the stream with the part's output (or, without
        ``then``, the stream and the output not yet added)."""
        given = normed if getattr(part, "takes_pending_norm", False) else normed.materialize()
        if then is not None and getattr(part, "adds_to_residual", False):
            out = part.forward(given, *args, into=ResidualInto(normed, then, rt))
        else:
            out = part.forward(given, *args)
        if isinstance(out, PendingNorm):
            return out
        if then is None:
            return normed.residual, out
        return then.defer(normed.residual, out, rt)

    def forward(self, stream, ctx, view, rt, following=None):
        """stream: (x, pending), or this block's first norm, pending, from the
        block before.  following: the next block's first norm, if that block
        takes it pending; then the return value is that pending norm, else the
        pair (x, pending)."""
        if isinstance(stream, PendingNorm):
            if stream.norm is not self.norm1:
                raise ValueError("the pending norm handed to a block is not the block's own first norm")
            normed = stream
        else:
            x, pending = stream
            normed = self.norm1.defer(x, pending, rt)
        normed = self._run(self.mixer, normed, (ctx, view, rt), self.norm2, rt)
        return self._run(self.feed_forward, normed, (ctx, rt), following, rt)


class HyperConnectionBlock(Block):
    """A pre-norm layer over a residual kept as ``streams`` streams x_1 .. x_s
    (all equal to the embedding at the start; their sum is the model's output).
    A sublayer, the mixer or the feed-forward, reads a weighted sum of the
    streams and writes into all of them:

        u = sum_s take[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s mix[s, t] x_s + gain[t] y

    ``take`` belongs to the norm (a norm over streams reads them itself);
    ``mix`` [from, to] and ``gain`` are this block's, one pair a sublayer.  The
    update and the norm that comes next (this block's second, or the first of
    the block behind it) are one kernel.  Without a feed-forward the layer has
    the first sublayer only."""

    def __init__(self, width, streams, norm1, mixer, connect1, norm2=None, feed_forward=None, connect2=None, positions=None):
        self.width, self.streams = int(width), int(streams)
        if (feed_forward is None) != (norm2 is None) or (feed_forward is None) != (connect2 is None):
            raise InvalidInput("a feed-forward comes with its norm and its connections, or none of the three")
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer, positions=positions)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self.connections = [connect1] + ([connect2] if connect2 is not None else [])
        self._parts = [part for part in (self.norm1, self.mixer, self.norm2, self.feed_forward) if part is not None]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self._parts)
        self._mix = self._gain = None

    def tensors(self):
        out = [spec for part in self._parts for spec in part.tensors()]
        for connect in self.connections:
            out.append(TensorSpec(connect["mix"], (self.streams, self.streams), init="stream_mix"))
            out.append(TensorSpec(connect["gain"], (self.streams,), init="stream_share"))
        return out

    def bind(self, weights, rt):
        for part in self._parts:
            part.bind(weights, rt)
        # the connections' coefficients are kept in 32-bit whatever they are stored in
        self._mix = [weights[connect["mix"]].float().contiguous() for connect in self.connections]
        self._gain = [weights[connect["gain"]].float().contiguous() for connect in self.connections]

    def weight_bytes(self):
        return sum(part.weight_bytes() for part in self._parts)

    def cache_request(self):
        return self.mixer.cache_request()

    def check(self, rt):
        for part in self._parts:
            part.check(rt)
        if not 1 <= self.streams <= 8:
            raise InvalidInput(f"the streams' kernels take 1 to 8 streams, got {self.streams}")

    def decode_plan(self, batch, longest, rt):
        return _joined(part.decode_plan(batch, longest, rt) for part in self._parts)

    def prompt_plan(self, batch, rows, longest, rt):
        return _joined(part.prompt_plan(batch, rows, longest, rt) for part in self._parts)

    def held_buffers(self, rt):
        return [buffer for part in self._parts for buffer in part.held_buffers(rt)]

    @property
    def entry_norm(self):
        return self.norm1

    def forward(self, stream, ctx, view, rt, following=None):
        """stream: (x, None) with x [streams, tokens, width], or this block's first
        norm already run by the block before (``PreparedStreams``).  following: the
        next block's first norm; if it reads these streams it is run here and handed on."""
        if isinstance(stream, PreparedStreams):
            if stream.norm is not self.norm1:
                raise ValueError("the rows handed to a block are not those of the block's own first norm")
            x, h = stream.x, stream.h
        else:
            x, pending = stream
            if pending is not None:
                raise InvalidInput("a block over several streams takes them with nothing left to add")
            if x.dim() == 2:
                if self.streams != 1:
                    raise InvalidInput(f"a block over {self.streams} streams was handed a single one")
                x = x.unsqueeze(0)
            h = self.norm1.forward(x, rt)
        y = self.mixer.forward(h, ctx, view, rt)
        if self.feed_forward is not None:
            h = self.norm2.update_forward(x, y, self._mix[0], self._gain[0], rt)
            y = self.feed_forward.forward(h, ctx, rt)
        mix, gain = self._mix[-1], self._gain[-1]
        if following is not None and hasattr(following, "update_forward") and getattr(following, "streams", 0) == self.streams:
            return PreparedStreams(following, x, following.update_forward(x, y, mix, gain, rt))
        rt.ops.stream_step(x, y=y, mix=mix, gain=gain)
        return x, None


class PrePostNormBlock(Block):
    """A layer that norms each sublayer on the way in and on the way out:

        x <- x + post1(mixer(norm1(x)));   x <- x + post2(feed_forward(norm2(x)))

    (the second line only with a feed-forward).  With norms that need no
    statistics (``TanhNorm``) everything between two sublayers -- the norm on
    the way out, the sum into the 32-bit stream, the next norm on the way in --
    is one kernel, and the layer's last output is handed on not yet normed
    (``PostNormed``), so that whoever takes the stream next does the same in
    its own first kernel; with other norms each step is the norm's own."""

    takes_post_normed = True

    def __init__(self, width, norm1, post1, mixer, norm2=None, post2=None, feed_forward=None, positions=None):
        self.width = int(width)
        if (feed_forward is None) != (norm2 is None) or (feed_forward is None) != (post2 is None):
            raise InvalidInput("a feed-forward comes with its two norms, or none of the three")
        self.norm1 = build_part("norm", norm1)
        self.norm1.rows_may_be_prepared = True  # the block before may run this norm in its own last kernel (``PreparedRows``)
        self.post1 = build_part("norm", post1)
        self.mixer = build_part("mixer", mixer, positions=positions)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.post2 = build_part("norm", post2) if post2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self._parts = [part for part in (self.norm1, self.post1, self.mixer, self.norm2, self.post2, self.feed_forward) if part is not None]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self._parts)

    def tensors(self):
        return [spec for part in self._parts for spec in part.tensors()]

    def bind(self, weights, rt):
        for part in self._parts:
            part.bind(weights, rt)

    def weight_bytes(self):
        return sum(part.weight_bytes() for part in self._parts)

    def cache_request(self):
        return self.mixer.cache_request()

    def check(self, rt):
        for part in self._parts:
            part.check(rt)

    def decode_plan(self, batch, longest, rt):
        return _joined(part.decode_plan(batch, longest, rt) for part in self._parts)

    def prompt_plan(self, batch, rows, longest, rt):
        return _joined(part.prompt_plan(batch, rows, longest, rt) for part in self._parts)

    def held_buffers(self, rt):
        return [buffer for part in self._parts for buffer in part.held_buffers(rt)]

    @property
    def entry_norm(self):
        return self.norm1

    @staticmethod
    def _run(part, args, x, post, following, rt):
        """The part's output, or -- where its last projection took the way out into its own kernel -- ``following``'s rows."""
        if following is not None and getattr(part, "adds_to_residual", False):
            return part.forward(*args, into=TanhInto(x, post, following, rt))
        return part.forward(*args)

    @staticmethod
    def _rms_pair(post, following) -> bool:
        """Whether both are plain RMS norms of one eps and one weight type: their step between two sublayers is one kernel."""
        return (getattr(post, "fusable_rms", False) and getattr(following, "fusable_rms", False) and post.eps == following.eps
                and post.weight is not None and following.weight is not None and post.weight.dtype == following.weight.dtype)

    @classmethod
    def _hands_rms_rows(cls, post, following) -> bool:
        """Whether the next block's first norm may be run here: an RMS pair, and a block behind it that takes the rows."""
        return following is not None and getattr(following, "rows_may_be_prepared", False) and cls._rms_pair(post, following)

    @classmethod
    def _between(cls, x, y, post, following, rt, share=None):
        """x += post(y) in place; returns following(x).  ``share``: (a factor per row, rows): y stands for y + factor * rows."""
        if hasattr(post, "triple") and hasattr(following, "triple") and share is None:
            return rt.ops.tanh_norm_step(x, x_out=x, y=y, post=post.triple(), following=following.triple(),
                                         h=rt.empty(x.shape[0], x.shape[1]))
        if cls._rms_pair(post, following) and y.is_contiguous():
            return rt.ops.rms_between(x, y, post.weight, following.weight, post.eps, h=rt.empty(x.shape[0], x.shape[1]), share=share)
        if share is not None:
            rt.ops.rows_axpy(y, share[1], share[0])
        return following.add_forward(x, post.forward(y, rt), rt)

    def forward(self, stream, ctx, view, rt, following=None):
        """stream: (x, pending) -- pending a tensor, a ``PostNormed`` or None -- or
        this block's first norm already run (``PreparedRows``).  following: the next
        block's first norm; run here and handed on if it is of the kind that this
        block's kernel takes, else the stream goes on as (x, ``PostNormed``)."""
        if isinstance(stream, PreparedRows):
            if stream.norm is not self.norm1:
                raise ValueError("the rows handed to a block are not those of the block's own first norm")
            x, h = stream.x, stream.h
        else:
            x, pending = stream
            if isinstance(pending, PostNormed) and not hasattr(self.norm1, "triple"):
                pending = pending.materialize(rt)
            h = self.norm1.forward(x, rt) if pending is None else self.norm1.add_forward(x, pending, rt)
        # A part that ends with a projection may take the way out -- its norm, the sum into the stream, the next norm on
        # the way in -- into that projection's kernel (``TanhInto``) and then returns the next part's rows, prepared.
        after_mixer = self.norm2 if self.feed_forward is not None else following
        y = self._run(self.mixer, (h, ctx, view, rt), x, self.post1, after_mixer, rt)
        post = self.post1
        share = None
        if self.feed_forward is not None:
            h = y.h if isinstance(y, PreparedRows) else self._between(x, y, self.post1, self.norm2, rt)
            if getattr(self.feed_forward, "can_leave_share", False) and self._hands_rms_rows(self.post2, following):
                # (a feed-forward that hands a share of its input through leaves that sum to the step's kernel)
                y = self.feed_forward.forward(h, ctx, rt, share_later=True)
                y, share = y if isinstance(y, tuple) else (y, None)
            else:
                y = self._run(self.feed_forward, (h, ctx, rt), x, self.post2, following, rt)
            post = self.post2
        if isinstance(y, PreparedRows):
            return y
        if following is not None and ((hasattr(post, "triple") and hasattr(following, "triple")) or self._hands_rms_rows(post, following)):
            return PreparedRows(following, x, self._between(x, y, post, following, rt, share=share))
        return x, PostNormed(y, post)


class PostNormBlock(Block):
    """A layer whose sublayers read the stream as it is and are normed on their way out only:

        x <- x + norm1(mixer(x));   x <- x + norm2(feed_forward(x))

    (the second line only with a feed-forward).  The norm on the way out, the sum into the 32-bit stream and the
    stream's rows in the activation type, which the next sublayer reads, are one kernel (``Norm.post_step``); the rows
    behind the layer's last sublayer are handed to a block of this kind that comes next (``PreparedRows``)."""

    def __init__(self, width, norm1, mixer, norm2=None, feed_forward=None, positions=None):
        self.width = int(width)
        if (feed_forward is None) != (norm2 is None):
            raise InvalidInput("a feed-forward comes with its norm, or neither")
        self.entry = build_part("norm", {"kind": "none", "width": self.width})  # how this block reads the stream
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer, positions=positions)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "post_step"):
                raise InvalidInput("a block that norms its sublayers' outputs needs norms that bring them into the stream (post_step)")
        self._parts = [part for part in (self.norm1, self.mixer, self.norm2, self.feed_forward) if part is not None]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self._parts)

    def tensors(self):
        return [spec for part in self._parts for spec in part.tensors()]

    def bind(self, weights, rt):
        for part in self._parts:
            part.bind(weights, rt)

    def weight_bytes(self):
        return sum(part.weight_bytes() for part in self._parts)

    def cache_request(self):
        return self.mixer.cache_request()

    def cache_request_beside(self):
        """What the mixer keeps of its own while its keys and values are another entry's (see ``Mixer.cache_request_beside``)."""
        return self.mixer.cache_request_beside() if hasattr(self.mixer, "cache_request_beside") else None

    def check(self, rt):
        for part in self._parts:
            part.check(rt)

    def decode_plan(self, batch, longest, rt):
        return _joined(part.decode_plan(batch, longest, rt) for part in self._parts)

    def prompt_plan(self, batch, rows, longest, rt):
        return _joined(part.prompt_plan(batch, rows, longest, rt) for part in self._parts)

    def held_buffers(self, rt):
        return [buffer for part in self._parts for buffer in part.held_buffers(rt)]

    @property
    def entry_norm(self):
        return self.entry

    def forward(self, stream, ctx, view, rt, following=None):
        """stream: (x, pending), or the stream with its rows made already (``PreparedRows`` of a norm of kind
        ``none``).  following: the next block's first norm; if that reads the stream as it is, the rows go with it."""
        if isinstance(stream, PreparedRows):
            if type(stream.norm) is not type(self.entry):
                raise ValueError("the rows handed to a block are not the stream's own")
            x, h = stream.x, stream.h
        else:
            x, pending = stream
            if isinstance(pending, PostNormed):
                pending = pending.materialize(rt)
            if pending is not None:
                raise InvalidInput("a block that reads the stream as it is takes it with nothing left to add")
            h = self.entry.forward(x, rt)
        h = self.norm1.post_step(x, self.mixer.forward(h, ctx, view, rt), rt)
        if self.feed_forward is not None:
            if getattr(self.feed_forward, "can_leave_share", False):
                # (a feed-forward that hands a share of its input through leaves that sum to the way out's kernel)
                y = self.feed_forward.forward(h, ctx, rt, share_later=True)
                y, share = y if isinstance(y, tuple) else (y, None)
                h = self.norm2.post_step(x, y, rt, share=share)
            else:
                h = self.norm2.post_step(x, self.feed_forward.forward(h, ctx, rt), rt)
        if following is not None and type(following) is type(self.entry):
            return PreparedRows(following, x, h)
        return x, None


def _noise(spec, generator):
    return torch.randn(tuple(spec.shape), generator=generator, dtype=torch.float32)


# what a random model draws for the connections: a mix near the identity, shares spread around one half
register_init_rule("stream_mix", lambda spec, generator, dtype: (torch.eye(spec.shape[0]) + 0.2 * _noise(spec, generator)).to(dtype), replace=True)
register_init_rule("stream_share", lambda spec, generator, dtype: (0.5 + 0.25 * _noise(spec, generator)).to(dtype), replace=True)

register_part("block", "pre_norm", PreNormBlock)
register_part("block", "hyper_connections", HyperConnectionBlock)
register_part("block", "pre_post_norm", PrePostNormBlock)
register_part("block", "post_norm", PostNormBlock)
