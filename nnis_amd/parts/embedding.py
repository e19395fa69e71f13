"""Token embedding (a row copy, /root/reference/crates/nnis-kernels/src/gather.rs:17-33)
and the output head (/root/reference/crates/nnis-model/src/runtime.rs:1109-1116),
which shares the embedding table when the checkpoint has no head of its own and
the configuration ties them
(/root/reference/crates/nnis-model/src/safetensors_loader.rs:755-786)."""

from __future__ import annotations

import torch

from .base import Part, StateRequest, TensorSpec, register_part
from .linear import Projection


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size, width, weight, scale=1.0):
        """``scale``: every row is multiplied by it on the way out (in 32-bit)."""
        self.vocab_size, self.width, self.weight_name, self.scale = int(vocab_size), int(width), weight, float(scale)
        self.table = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.vocab_size, self.width))]

    def bind(self, weights, rt):
        self.table = weights[self.weight_name].contiguous()

    def adopt_packed(self, source, packed) -> bool:
        """A part of the model has packed the tensor at ``source`` (address,
        shape) for the matrix cores.  If that tensor is this table (a tied
        head), rows are gathered from the packed copy from now on and the
        table in the checkpoint's order is let go: the table is kept once."""
        if isinstance(self.table, torch.Tensor) and source == (self.table.data_ptr(), tuple(self.table.shape)):
            self.table = packed
            return True
        return False

    def forward(self, ids, tokens, rt):
        """ids: int32 on the device -> the 32-bit residual stream [tokens, width]."""
        return rt.ops.embed(ids, self.table, rt.empty(tokens, self.width, dtype=torch.float32), self.scale)


class PairHashEmbedding(Part):
    """A token's row of the table plus a row of a second table chosen by the
    token and the one before it: row (before * mul_prev + token * mul_cur) %
    buckets, and row ``buckets`` (the last) for a sequence's first token.  The
    token before a step's first is part of the sequence's state: one integer
    per slot, which the cache keeps (``cache_request``).  ``copies`` > 1 gives
    the output as that many equal streams ``[copies, tokens, width]``."""

    graph_safe = True

    def __init__(self, vocab_size, width, weight, pairs, buckets, mul_prev, mul_cur, copies=1):
        self.vocab_size, self.width, self.weight_name, self.pairs_name = int(vocab_size), int(width), weight, pairs
        self.buckets, self.mul_prev, self.mul_cur, self.copies = int(buckets), int(mul_prev), int(mul_cur), int(copies)
        self.table = self.pairs = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.vocab_size, self.width)),
                TensorSpec(self.pairs_name, (self.buckets + 1, self.width))]

    def bind(self, weights, rt):
        self.table = weights[self.weight_name].contiguous()
        self.pairs = weights[self.pairs_name].contiguous()

    def cache_request(self):
        return StateRequest((), "int32")

    def forward_step(self, ids, ctx, view, rt):
        """ids: int32 on the device -> the 32-bit residual [copies, tokens, width] ([tokens, width] for one copy)."""
        out = rt.empty(self.copies, ctx.tokens, self.width, dtype=torch.float32)
        rt.ops.embed_pair(ids, ctx.tok_slot, ctx.tok_pos, self.table, self.pairs, self.mul_prev, self.mul_cur, view.state, out)
        return out if self.copies > 1 else out[0]


class LinearHead(Part):
    graph_safe = True

    def __init__(self, vocab_size, width, weight, tied_to=None, softcap=None, scale=None):
        """``softcap``: logits z leave as softcap * tanh(z / softcap).  ``scale``: logits are multiplied by it (before a cap)."""
        self.vocab_size, self.width, self.weight_name, self.tied_to = int(vocab_size), int(width), weight, tied_to
        self.softcap = None if not softcap else float(softcap)
        self.scale = None if scale is None or float(scale) == 1.0 else float(scale)
        self.projection = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.vocab_size, self.width), fallback=self.tied_to)]

    def bind(self, weights, rt):
        # a tied head is the same device tensor as the embedding table
        self.projection = Projection(weights[self.weight_name], rt)

    def packed_sources(self):
        return [(self.projection.packed_from, self.projection.weight)] if self.projection.packed_from else []

    def weight_bytes(self):
        return self.projection.weight_bytes()

    def forward(self, x, rt):
        """Logits are 32-bit whatever the storage type."""
        logits = self.projection(x, rt, out_dtype=torch.float32)
        if self.scale is not None:
            rt.ops.scale_rows(logits, self.scale)
        return logits if self.softcap is None else rt.ops.tanh_cap(logits, self.softcap)


register_part("embedding", "table", TokenEmbedding)
register_part("embedding", "table_pairs", PairHashEmbedding)
register_part("head", "linear", LinearHead)
