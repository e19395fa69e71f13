"""Attention over a cached latent.  A token keeps one vector c of ``kv_rank``
channels, the root-mean-square norm of a down projection of the mixer's input,
and, where the mixer rotates, one key part of ``rot_dim`` channels turned by
the token's position and shared by all heads.  Per head h, keys and values are
maps of the latent, k_h = Uk_h c and v_h = Uv_h c; queries go through a latent
of their own, c_q = norm(Dq x), q_h = Uq_h c_q = [plain part | rotated part]:

    score_h(i, j) = (q_h,plain(i) . k_h(j) + q_h,rot(i) . k_rot(j)) * scale
    y = O [ gate_h * sum_j p_h(i, j) v_h(j) ]_h

Nothing per head is ever made of a cached token.  q_plain . (Uk_h c) = (Uk_h^T
q_plain) . c, so the heads' key maps are folded into the query's up
projection, and sum_j p v_h(j) = Uv_h sum_j p c(j), so the value maps are
folded into the output projection (both once, when the weights are bound, in
64-bit).  What runs is attention of ``heads`` query heads of kv_rank + rot_dim
channels over ONE key/value head whose keys are [c | k_rot] and whose values
are c: the kernels of grouped attention, with values narrower than the keys.
The folded matrices are larger than the maps they replace where kv_rank
exceeds a head's own size (heads * kv_rank columns instead of heads * dim):
the price of reading each cached token once for all heads.

Options: a sink per head in the softmax's denominator (``sink``), a gate per
head, sigmoid of a projection of the mixer's input, on the head's output
(``gate``); queries that leave one projection of the mixer's input, without a
latent of their own (``q_rank`` None and ``q``: the key maps are then folded
into that projection); a sliding window (``window``); a gate element by
element on the concatenated heads' outputs (``channel_gate``): it stands
between the value maps and the output projection, so the maps are not folded
into the projection but run head by head behind the attention, gate included.
"""

from __future__ import annotations

import torch

from ..errors import InvalidInput
from .base import KVRequest, Mixer, TensorSpec, register_part
from .linear import Projection


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, width, heads, key_dim, value_dim, q_rank, kv_rank, scale, eps, dkv, dkv_norm, uk, uv, o, dq=None, dq_norm=None,
                 uq=None, q=None, rot_dim=0, position=None, sink=None, gate=None, positions=None, window=None, channel_gate=None):
        self.width, self.heads, self.key_dim, self.value_dim = int(width), int(heads), int(key_dim), int(value_dim)
        self.q_rank, self.kv_rank, self.rot_dim = int(q_rank or 0), int(kv_rank), int(rot_dim or 0)
        self.scale, self.eps = float(scale), float(eps)
        if min(self.width, self.heads, self.key_dim, self.value_dim, self.kv_rank) <= 0 or self.q_rank < 0 or not self.scale > 0.0:
            raise InvalidInput("attention over a latent needs positive sizes and a positive scale")
        if self.q_rank and (dq is None or dq_norm is None or uq is None or q is not None):
            raise InvalidInput("queries through a latent name its down projection, its norm and its up projection")
        if not self.q_rank and (q is None or dq is not None or uq is not None):
            raise InvalidInput("queries without a latent name their one projection")
        if gate is not None and channel_gate is not None:
            raise InvalidInput("the heads are gated one number a head or element by element, not both")
        self.names = {"dq": dq, "dq_norm": dq_norm, "uq": uq, "q": q, "dkv": dkv, "dkv_norm": dkv_norm, "uk": uk, "uv": uv, "o": o}
        self.sink_name, self.gate_name, self.channel_gate_name = sink, gate, channel_gate
        self.window = 0 if not window else int(window)
        self.value_maps = None  # [heads, value_dim, kv_rank] where the maps run behind the attention
        self.position = None
        if self.rot_dim:
            if self.rot_dim % 2 or positions is None or position not in positions:
                raise InvalidInput(f"a rotated key part of {rot_dim} channels needs an even size and a position encoding ({position!r})")
            self.position = positions[position]
            if getattr(self.position, "pairing", None) != "neighbours" or getattr(self.position, "rot_dim", None) != self.rot_dim:
                raise InvalidInput("the rotated part turns neighbouring channels, all of them: the position encoding must say so")
        self.head_width = self.kv_rank + self.rot_dim  # a query head as the attention sees it
        self.inputs = self.queries = self.out = None
        self.q_weight = self.c_weight = self.extras = None

    def tensors(self):
        h = self.heads
        if self.q_rank:
            out = [TensorSpec(self.names["dq"], (self.q_rank, self.width)),
                   TensorSpec(self.names["dq_norm"], (self.q_rank,), init="gain"),
                   TensorSpec(self.names["uq"], (h * (self.key_dim + self.rot_dim), self.q_rank))]
        else:
            out = [TensorSpec(self.names["q"], (h * (self.key_dim + self.rot_dim), self.width))]
        out += [
            TensorSpec(self.names["dkv"], (self.kv_rank + self.rot_dim, self.width)),
            TensorSpec(self.names["dkv_norm"], (self.kv_rank,), init="gain"),
            TensorSpec(self.names["uk"], (h * self.key_dim, self.kv_rank)),
            TensorSpec(self.names["uv"], (h * self.value_dim, self.kv_rank)),
            TensorSpec(self.names["o"], (self.width, h * self.value_dim)),
        ]
        if self.sink_name:
            out.append(TensorSpec(self.sink_name, (h,)))
        if self.gate_name:
            out.append(TensorSpec(self.gate_name, (h, self.width)))
        if self.channel_gate_name:
            out.append(TensorSpec(self.channel_gate_name, (h * self.value_dim, self.width)))
        return out

    def bind(self, weights, rt):
        h, dim, rot, rank = self.heads, self.key_dim, self.rot_dim, self.kv_rank
        kind = weights[self.names["uk"]].dtype
        # the down projections (and the gates' projection) read the same rows: one product, rows [dq | dkv | gate]
        gate_name = self.gate_name or self.channel_gate_name
        rows = ([weights[self.names["dq"]]] if self.q_rank else []) + [weights[self.names["dkv"]]] + ([weights[gate_name]] if gate_name else [])
        self.inputs = Projection(torch.cat(rows, dim=0), rt)
        # the heads' key maps into the queries' up projection (or, without a query latent, into the queries' one
        # projection): per head [Uk^T Uq_plain ; Uq_rot], rows of q_rank (of the model width)
        inner = self.q_rank or self.width
        uq = weights[self.names["uq" if self.q_rank else "q"]].double().view(h, dim + rot, inner)
        uk = weights[self.names["uk"]].double().view(h, dim, rank)
        folded = torch.cat([torch.einsum("hdk,hdq->hkq", uk, uq[:, :dim]), uq[:, dim:]], dim=1)
        self.queries = Projection(folded.reshape(h * self.head_width, inner).to(kind), rt)
        if self.channel_gate_name:
            # a gate element by element stands between the value maps and the output projection: both stay as they are
            self.value_maps = weights[self.names["uv"]].view(h, self.value_dim, rank).contiguous()
            self.out = Projection(weights[self.names["o"]], rt)
        else:
            # the heads' value maps into the output projection: columns per head O_h Uv_h
            uv = weights[self.names["uv"]].double().view(h, self.value_dim, rank)
            o = weights[self.names["o"]].double().view(self.width, h, self.value_dim)
            self.out = Projection(torch.einsum("whv,hvk->whk", o, uv).reshape(self.width, h * rank).to(kind), rt)
        self.c_weight = weights[self.names["dkv_norm"]].contiguous()
        self.q_weight = weights[self.names["dq_norm"]].contiguous() if self.q_rank else None
        if self.q_weight is not None:
            self.c_weight = self.c_weight.to(self.q_weight.dtype).contiguous()
        sink = weights[self.sink_name].float().contiguous() if self.sink_name else None
        self.extras = rt.ops.ScoreExtras(0, None, sink)

    def weight_bytes(self):
        maps = 0 if self.value_maps is None else self.value_maps.numel() * self.value_maps.element_size()
        return self.inputs.weight_bytes() + self.queries.weight_bytes() + self.out.weight_bytes() + maps

    def cache_request(self):
        return KVRequest(1, self.head_width, self.window or None, self.kv_rank if self.rot_dim else None)

    def check(self, rt):
        # (a latent wider than the matrix-core kernels carry still runs, on the row kernel)
        rt.ops.attention_check(self.head_width, self.kv_rank, rt.ops.ATTENTION_ROWS_MOST_CHANNELS)

    def _matrix_cores(self, rt) -> bool:
        return rt.ops.attention_on_matrix_cores(rt.dtype, rt.dtype, self.head_width, self.kv_rank, 0.0, self.extras)

    def decode_plan(self, batch, longest, rt):
        if not self._matrix_cores(rt):
            return None
        # (one key/value head makes few blocks: the keys are cut into runs by the rule of narrow outputs, from 9 pages on)
        return rt.ops.decode_plan(batch, 1, longest, width=min(1024, self.heads * self.kv_rank))

    def prompt_plan(self, batch, rows, longest, rt):
        if not self._matrix_cores(rt):
            return None
        return rt.ops.prefill_plan(longest, rows, self.heads, self.head_width, 1)

    def held_buffers(self, rt):
        held = rt.ops.decode_scratch_held(rt.device)
        return [] if held is None else [held]

    adds_to_residual = True

    def forward(self, x, ctx, view, rt, into=None):
        tokens = x.shape[0]
        ops = rt.ops
        gates = self.heads if self.gate_name else (self.heads * self.value_dim if self.channel_gate_name else 0)
        proj = self.inputs(x, rt, out_dtype=torch.float32)  # the norms read what the products summed, not a rounding of it
        cq = rt.empty(tokens, self.q_rank) if self.q_rank else None
        gate = rt.empty(tokens, gates, dtype=torch.float32) if gates else None
        tables = self.position.rotary() if self.position is not None else None
        writes = not view.read_only
        ops.latent_prepare(proj, self.q_rank, self.kv_rank, self.rot_dim, gates, self.q_weight, self.c_weight, self.eps,
                           tables.cos if tables else None, tables.sin if tables else None, ctx.tok_slot, ctx.tok_pos, cq,
                           view.k_pages if writes else None, view.v_pages if writes else None,
                           view.block_table if writes else None, gate)
        q = self.queries(cq if self.q_rank else x, rt)
        if self.rot_dim:
            ops.latent_rotate_q(q, self.heads, self.head_width, self.kv_rank, self.rot_dim, tables.cos, tables.sin, ctx.tok_pos)
        fast = self._matrix_cores(rt) and view.k_pages.dtype == torch.bfloat16
        step = ctx.step_tables(rt, None, view.block_table) if (ctx.decode and fast) else None
        plan = ctx.options.get("latent_attention")
        if plan is None and fast:
            plan = (self.decode_plan(ctx.batch, ctx.planned_len, rt) if ctx.decode
                    else self.prompt_plan(ctx.batch, ctx.planned_rows, ctx.planned_len, rt))
        mixed = ops.attention(q, rt.empty(tokens, self.heads * self.kv_rank), view, ctx, self.heads, 1, self.head_width, self.scale,
                              self.window, tables=step, plan=plan, value_dim=self.kv_rank, extras=self.extras)
        if self.value_maps is not None:
            # the heads' value maps, head by head, and the gate element by element in the same kernel
            mixed = ops.heads_linear(mixed, self.value_maps, gate, self.heads, rt.empty(tokens, self.heads * self.value_dim))
        elif gates:
            ops.head_scale(mixed, gate, self.heads)
        if into is not None and into.can_take(mixed, self.out.weight):
            return into.take(mixed, self.out.weight)  # the output projection adds to the stream itself
        return self.out(mixed, rt)


register_part("mixer", "latent_attention", LatentAttention)
