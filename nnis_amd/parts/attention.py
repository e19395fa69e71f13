"""Causal self-attention with grouped key/value heads over the cache
(/root/reference/crates/nnis-model/src/runtime.rs:959-1038; formula
/root/reference/crates/nnis-model/src/kernels.rs:66-125).  Queries, keys and
values come from one fused projection; queries and keys are rotated by the
position encoding handed in; keys and values go into the cache before the
scores are taken, so the same code runs whole prompts and single tokens.

Options beyond that formula, each off unless the description names it: biases
on the four projections; values (and a head's output) of another size than
the keys (``value_dim``); a scale of the scores other than 1 / sqrt(head_dim);
scores bent by a cap, s -> softcap * tanh(s / softcap), before the softmax;
a rotation of the first channels of a head only (the position encoding's
``rot_dim``); with a window, first tokens that stay visible to every later
query (``keep_first``); a learned bias by distance added to the scaled score
(``distance_bias``, ``bias_reach``); a sink in the softmax's denominator
(``sink``); values that are the keys as projected, before their rotation, with
no projection of their own (``values_from_keys``); a gate per head, sigmoid of
a projection of the mixer's input, on the head's output (``head_gate``).
"""

from __future__ import annotations

import math

import torch

from ..errors import InvalidInput
from .base import KVRequest, Mixer, TensorSpec, register_part
from .linear import Projection


def distance_bucket(n: int, buckets: int, reach: int) -> int:
    """The row of a table of ``buckets`` rows that a key ``n`` positions back
    reads: the distance itself in the first half of the table, then steps that
    widen with the logarithm of the distance, so that the last row is met at
    ``reach`` and holds for everything beyond."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (buckets - half))))


class CausalSelfAttention(Mixer):
    graph_safe = True

    def __init__(self, width, heads, kv_heads, head_dim, q, k, v, o, position=None, window=None, positions=None,
                 value_dim=None, scale=None, softcap=None, q_bias=None, k_bias=None, v_bias=None, o_bias=None,
                 keep_first=None, distance_bias=None, bias_reach=None, bias_buckets=None, sink=None, values_from_keys=False,
                 head_gate=None):
        """``keep_first``: with a ``window``, keys at positions below it stay
        visible.  ``distance_bias``: the name of a table [buckets, heads]; the
        scaled score of a key n positions back gets row ``distance_bucket(n,
        buckets, bias_reach)`` of its head's column added (the table's length
        is the checkpoint's; a random model names it as ``bias_buckets``).
        ``sink``: "zero" for a score of 0, or the name of a tensor [heads] of
        learned scores, that joins the softmax's denominator and has no value."""
        if heads % kv_heads != 0:
            raise InvalidInput(f"{heads} query heads do not divide into {kv_heads} key/value heads")
        self.width, self.heads, self.kv_heads, self.head_dim = int(width), int(heads), int(kv_heads), int(head_dim)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        if self.value_dim <= 0:
            raise InvalidInput(f"value_dim must be positive, got {value_dim}")
        self.values_from_keys = bool(values_from_keys)
        if self.values_from_keys and (self.value_dim != self.head_dim or v is not None or v_bias is not None):
            raise InvalidInput("values that are the keys have the keys' size and no projection of their own")
        self.gate_name, self.gate = head_gate, None
        self.softcap = 0.0 if not softcap else float(softcap)
        if self.softcap < 0.0:
            raise InvalidInput(f"the cap of the scores must be positive, got {softcap}")
        if (q_bias is None) != (k_bias is None) or ((q_bias is None) != (v_bias is None) and not values_from_keys):
            raise InvalidInput("the projections of queries, keys and values have biases all three or none")
        self.bias_names = {"q": q_bias, "k": k_bias, "v": v_bias, "o": o_bias}
        self.qkv_bias = None
        self.output_bias = None
        self.names = {"q": q, "k": k, "v": v, "o": o}
        self.window = None if not window else int(window)
        self.position = None
        if position is not None:
            if positions is None or position not in positions:
                raise InvalidInput(f"attention names position encoding {position!r}, which the model does not define")
            self.position = positions[position]
        self.scale = 1.0 / math.sqrt(self.head_dim) if scale is None else float(scale)  # runtime.rs:943
        if not self.scale > 0.0:
            raise InvalidInput(f"the scale of the scores must be positive, got {scale}")
        self.keep_first = 0 if not keep_first else int(keep_first)
        if self.keep_first < 0 or (self.keep_first and not self.window):
            raise InvalidInput(f"first tokens are kept visible ({keep_first}) beside a window only")
        self.bias_name, self.bias_reach = distance_bias, None if bias_reach is None else int(bias_reach)
        self.bias_buckets = None if bias_buckets is None else int(bias_buckets)
        if distance_bias is not None and (self.bias_reach is None or self.bias_reach < 1):
            raise InvalidInput(f"a bias by distance needs the distance at which its last row is met, got {bias_reach!r}")
        self.sink_name = sink
        self.extras = None  # ``ops.ScoreExtras``, made when the weights are bound
        self.qkv = None
        self.out = None

    def tensors(self):
        q_width, kv_width = self.heads * self.head_dim, self.kv_heads * self.head_dim
        v_width, o_width = self.kv_heads * self.value_dim, self.heads * self.value_dim
        out = [
            TensorSpec(self.names["q"], (q_width, self.width)),
            TensorSpec(self.names["k"], (kv_width, self.width)),
            TensorSpec(self.names["v"], (v_width, self.width)),
            TensorSpec(self.names["o"], (self.width, o_width)),
        ]
        if self.values_from_keys:
            del out[2]
        if self.gate_name:
            out.append(TensorSpec(self.gate_name, (self.heads, self.width)))
        for key, size in (("q", q_width), ("k", kv_width), ("v", v_width), ("o", self.width)):
            if self.bias_names[key]:
                out.append(TensorSpec(self.bias_names[key], (size,)))
        if self.bias_name:
            out.append(TensorSpec(self.bias_name, (self.bias_buckets, self.heads)))
        if self.sink_name and self.sink_name != "zero":
            out.append(TensorSpec(self.sink_name, (self.heads,)))
        return out

    def bind(self, weights, rt):
        # one projection for queries, keys and values: rows q heads, k heads, v heads
        rows = ("q", "k") if self.values_from_keys else ("q", "k", "v")
        self.qkv = Projection(torch.cat([weights[self.names[key]] for key in rows], dim=0), rt)
        self.out = Projection(weights[self.names["o"]], rt)
        if self.gate_name:
            self.gate = Projection(weights[self.gate_name], rt)
        if self.bias_names["q"]:
            self.qkv_bias = torch.cat([weights[self.bias_names[key]] for key in rows]).contiguous()
        if self.bias_names["o"]:
            self.output_bias = weights[self.bias_names["o"]].contiguous()
        bias = sink = None
        if self.bias_name:
            # the table by bucket becomes a table by distance, [heads, reach + 1] in 32-bit: the kernels index it by min(n, reach)
            table = weights[self.bias_name].float()
            buckets = table.shape[0]
            if buckets < 2 or self.bias_reach <= buckets // 2:
                raise InvalidInput(f"a bias table of {buckets} rows cannot reach a distance of {self.bias_reach}")
            rows = torch.tensor([distance_bucket(n, buckets, self.bias_reach) for n in range(self.bias_reach + 1)],
                                dtype=torch.long, device=table.device)
            bias = table[rows].t().contiguous()
        if self.sink_name:
            sink = (torch.zeros(self.heads, dtype=torch.float32, device=rt.device) if self.sink_name == "zero"
                    else weights[self.sink_name].float().contiguous())
        self.extras = rt.ops.ScoreExtras(self.keep_first, bias, sink)

    def weight_bytes(self):
        return self.qkv.weight_bytes() + self.out.weight_bytes() + (self.gate.weight_bytes() if self.gate is not None else 0)

    def cache_request(self):
        return KVRequest(self.kv_heads, self.head_dim, self.window, None if self.value_dim == self.head_dim else self.value_dim)

    def check(self, rt):
        rt.ops.attention_check(self.head_dim, self.value_dim)
        tables = self.position.rotary() if self.position is not None else None
        rot_dim = tables.rot_dim if tables is not None else getattr(self.position, "rot_dim", 0)
        if rot_dim > self.head_dim:
            raise InvalidInput(f"a rotation of {rot_dim} channels does not fit heads of {self.head_dim}")

    def _matrix_cores(self, rt) -> bool:
        return rt.ops.attention_on_matrix_cores(rt.dtype, rt.dtype, self.head_dim, self.value_dim, self.softcap, self.extras)

    @property
    def _plain(self) -> bool:
        """The formula without any of the options: what the fused kernels of the projections take."""
        return self.value_dim == self.head_dim and self.qkv_bias is None and not self.values_from_keys

    def decode_plan(self, batch, longest, rt):
        # (runs of the keys, waves of a block) of a step of single tokens with these sizes
        if not self._matrix_cores(rt):
            return None
        return rt.ops.decode_plan(batch, self.kv_heads, longest, width=self.heads * self.value_dim)

    def prompt_plan(self, batch, rows, longest, rt):
        # (waves of a block, columns a wave carries) of the matrix-core kernel; the 32-bit kernel has no plan
        if not self._matrix_cores(rt):
            return None
        return rt.ops.prefill_plan(longest, rows, self.heads, max(self.head_dim, self.value_dim), self.kv_heads)

    def held_buffers(self, rt):
        # the runs of a decode step's keys meet in a scratch that the kernels' wrapper keeps per device
        held = rt.ops.decode_scratch_held(rt.device)
        return [] if held is None else [held]

    takes_pending_norm = True
    adds_to_residual = True

    def _project_rotate_store(self, x, ctx, view, rt):
        """Queries [tokens, heads * head_dim], rotated; keys and values of the
        step's tokens in the cache."""
        from .lazy import PendingNorm

        tables = self.position.rotary() if self.position is not None else None
        writes = not view.read_only
        if isinstance(x, PendingNorm):
            if (self._plain and x.can_fuse(self.qkv.weight) and tables is not None and tables.rot_dim == self.head_dim
                    and self.head_dim % 32 == 0 and view.k_pages.dtype == torch.bfloat16):
                # residual sum, norm, the three projections, the rotation and the cache write in one kernel
                rope = dict(cos=tables.cos, sin=tables.sin, tok_slot=ctx.tok_slot, tok_pos=ctx.tok_pos,
                            tables=ctx.step_tables(rt, tables, view.block_table),
                            k_pages=view.k_pages if writes else None, v_pages=view.v_pages if writes else None,
                            block_table=view.block_table if writes else None, heads=self.heads,
                            kv_heads=self.kv_heads, head_dim=self.head_dim)
                return x.fused(self.qkv.weight, rt.empty(x.rows, self.heads * self.head_dim), rt.ops.EPILOGUE_ROPE, rope)
            x = x.materialize()
        tokens = x.shape[0]
        qkv = self.qkv(x, rt)
        q = rt.empty(tokens, self.heads * self.head_dim)
        rt.ops.rope_kv_write(
            qkv, q,
            tables.cos if tables else None, tables.sin if tables else None, tables.rot_dim if tables else 0,
            ctx.tok_slot, ctx.tok_pos,
            view.k_pages if writes else None, view.v_pages if writes else None, view.block_table if writes else None,
            self.heads, self.kv_heads, self.head_dim, self.value_dim, self.qkv_bias, values_from_keys=self.values_from_keys,
        )
        return q

    can_leave_bias = True  # ``forward(..., bias_later=True)`` leaves ``output_bias`` to a consumer that adds it in a kernel of its own

    def forward(self, x, ctx, view, rt, into=None, bias_later=False):
        gate = None
        if self.gate is not None:
            # (the gates read the mixer's input as the projections do; their logits stay 32-bit)
            if hasattr(x, "materialize"):
                x = x.materialize()
            gate = self.gate(x, rt, out_dtype=torch.float32)
            into = None  # the heads are gated before the output projection, which then takes plain rows
        q = self._project_rotate_store(x, ctx, view, rt)
        tokens = q.shape[0]
        attn = rt.empty(tokens, self.heads * self.value_dim)
        # a decode step over long sequences leaves its runs of keys to the output projection, if that takes them
        step = None
        fast = self._matrix_cores(rt) and view.k_pages.dtype == torch.bfloat16
        if ctx.decode and fast:
            step = ctx.step_tables(rt, self.position.rotary() if self.position is not None else None, view.block_table)
        plan = ctx.options.get("causal_attention")  # (a test or a sweep names the launch; else the sizes choose)
        if plan is None and fast:
            plan = (self.decode_plan(ctx.batch, ctx.planned_len, rt) if ctx.decode
                    else self.prompt_plan(ctx.batch, ctx.planned_rows, ctx.planned_len, rt))
        attn = rt.ops.attention(q, attn, view, ctx, self.heads, self.kv_heads, self.head_dim, self.scale, self.window or 0,
                                keep_runs=into is not None and self.output_bias is None, tables=step, plan=plan,
                                value_dim=self.value_dim, softcap=self.softcap, extras=self.extras)
        if isinstance(attn, rt.ops.KeyRuns) and not (into.can_take(attn, self.out.weight) and attn.fits(self.out.weight.shape[0])):
            attn = attn.combine()
        if gate is not None:
            rt.ops.head_scale(attn, gate, self.heads, logistic=True)
        if into is not None and self.output_bias is None and into.can_take(attn, self.out.weight):
            return into.take(attn, self.out.weight)  # the output projection adds to the stream itself
        y = self.out(attn, rt)
        if self.output_bias is not None and not bias_later:
            rt.ops.add_bias(y, self.output_bias)
        return y


register_part("mixer", "causal_attention", CausalSelfAttention)


class GatedWindowAttention(Mixer):
    """Grouped attention whose queries and keys are normed head by head, whose
    window may come with pooled blocks, and whose heads are gated:

        q = rot(R(Wq h, wq)),  k = rot(R(Wk h, wk)),  v = Wv h       R: RMS norm over a head's channels, one weight for
                                                                     all heads; rot: channel 2i turns with 2i + 1
        s(i, j) = cap * tanh(q_i . k_j * scale / cap)                0 <= i - j < window
        s(i, b) the same with the mean key of block b                b * pool + pool - 1 <= i - window
        p = exp(s) / (sum_j exp s(i, j) + sum_b exp s(i, b) + exp(sink_head))
        out = Wo (concat_heads(sum p v) * sigmoid(Wg h))

    A block's key and value are the means of its ``pool`` tokens' keys and
    values as the cache holds them; they live in pages of their own, one entry
    a block (``KVRequest.every``), written by the step that completes the
    block.  Tokens that have left the window and whose block is not complete
    before it are not seen.  Each of cap, window, pool and rotation is off when
    zero or None.  ``own_kv`` False: the layer has no keys and values; it reads
    those of the schedule entry that the model names (``reads_cache_of``) with
    its own queries and mask, and that entry's pooled blocks if their size
    (``source_pool``) is this layer's, else it keeps pooled blocks of its own
    beside them (``cache_request_beside``)."""

    graph_safe = True

    def __init__(self, width, heads, kv_heads, head_dim, value_dim, scale, eps, q, o, gate, q_norm, sink, k=None, v=None, k_norm=None,
                 position=None, positions=None, window=None, pool=None, softcap=None, own_kv=True, source_pool=None):
        if heads % kv_heads != 0:
            raise InvalidInput(f"{heads} query heads do not divide into {kv_heads} key/value heads")
        self.width, self.heads, self.kv_heads = int(width), int(heads), int(kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.scale, self.eps = float(scale), float(eps)
        if min(self.width, self.heads, self.head_dim, self.value_dim) <= 0 or not self.scale > 0.0:
            raise InvalidInput("attention needs positive sizes and a positive scale")
        self.softcap = 0.0 if not softcap else float(softcap)
        self.window = 0 if not window else int(window)
        self.pool = 0 if not pool else int(pool)
        if self.pool and not self.window:
            raise InvalidInput(f"pooled blocks of {self.pool} tokens stand beside a window only")
        self.own_kv = bool(own_kv)
        self.source_pool = 0 if not source_pool else int(source_pool)
        if self.own_kv and (k is None or v is None or k_norm is None):
            raise InvalidInput("a layer with keys and values of its own names their projections and the keys' norm")
        self.names = {"q": q, "k": k, "v": v, "o": o, "gate": gate, "q_norm": q_norm, "k_norm": k_norm, "sink": sink}
        self.position = None
        if position is not None:
            if positions is None or position not in positions:
                raise InvalidInput(f"attention names position encoding {position!r}, which the model does not define")
            self.position = positions[position]
            if getattr(self.position, "pairing", None) != "neighbours":
                raise InvalidInput("this attention turns neighbouring channels: the position encoding must say so")
        self.proj = self.out = self.q_norm = self.k_norm = self.extras = None

    def tensors(self):
        n, qw, ow = self.names, self.heads * self.head_dim, self.heads * self.value_dim
        out = [TensorSpec(n["q"], (qw, self.width)), TensorSpec(n["q_norm"], (self.head_dim,), init="gain"),
               TensorSpec(n["sink"], (self.heads,), init="small"), TensorSpec(n["gate"], (ow, self.width)),
               TensorSpec(n["o"], (self.width, ow))]
        if self.own_kv:
            out += [TensorSpec(n["k"], (self.kv_heads * self.head_dim, self.width)),
                    TensorSpec(n["v"], (self.kv_heads * self.value_dim, self.width)),
                    TensorSpec(n["k_norm"], (self.head_dim,), init="gain")]
        return out

    def bind(self, weights, rt):
        n = self.names
        # one projection for everything that reads the mixer's input: rows [q | k | v | gate] (or [q | gate])
        parts = [weights[n["q"]]] + ([weights[n["k"]], weights[n["v"]]] if self.own_kv else []) + [weights[n["gate"]]]
        self.proj = Projection(torch.cat(parts, dim=0), rt)
        self.out = Projection(weights[n["o"]], rt)
        self.q_norm = weights[n["q_norm"]].float().contiguous()
        self.k_norm = weights[n["k_norm"]].float().contiguous() if self.own_kv else None
        self.extras = rt.ops.ScoreExtras(0, None, weights[n["sink"]].float().contiguous())
        qw = self.heads * self.head_dim
        kw, vw = (self.kv_heads * self.head_dim, self.kv_heads * self.value_dim) if self.own_kv else (0, 0)
        self.columns = (0, qw, qw + kw)
        self.gate_column = qw + kw + vw

    def weight_bytes(self):
        return self.proj.weight_bytes() + self.out.weight_bytes()

    def _pooled_request(self):
        return KVRequest(self.kv_heads, self.head_dim, None, None if self.value_dim == self.head_dim else self.value_dim, every=self.pool)

    def cache_request(self):
        main = KVRequest(self.kv_heads, self.head_dim, None, None if self.value_dim == self.head_dim else self.value_dim)
        return (main, self._pooled_request() if self.pool else None)

    def cache_request_beside(self):
        """What this layer keeps while its keys and values are another entry's: pooled blocks, if it sees any and the
        other entry keeps none of this size."""
        if self.own_kv or not self.pool or self.pool == self.source_pool:
            return None
        return self._pooled_request()

    def check(self, rt):
        # (heads wider than the matrix-core kernels carry take the row kernel, at its pace)
        wide = max(self.head_dim, self.value_dim) > rt.ops.ATTENTION_MOST_CHANNELS
        rt.ops.attention_check(self.head_dim, self.value_dim, rt.ops.ATTENTION_ROWS_MOST_CHANNELS if wide else rt.ops.ATTENTION_MOST_CHANNELS)
        rot_dim = getattr(self.position, "rot_dim", 0)
        if rot_dim > self.head_dim:
            raise InvalidInput(f"a rotation of {rot_dim} channels does not fit heads of {self.head_dim}")

    def _matrix_cores(self, rt) -> bool:
        return rt.ops.attention_on_matrix_cores(rt.dtype, rt.dtype, self.head_dim, self.value_dim, self.softcap, self.extras)

    def decode_plan(self, batch, longest, rt):
        if not self._matrix_cores(rt):
            return None
        return rt.ops.decode_plan(batch, self.kv_heads, longest, width=self.heads * self.value_dim)

    def prompt_plan(self, batch, rows, longest, rt):
        if not self._matrix_cores(rt):
            return None
        return rt.ops.prefill_plan(longest, rows, self.heads, max(self.head_dim, self.value_dim), self.kv_heads)

    def held_buffers(self, rt):
        held = rt.ops.decode_scratch_held(rt.device)
        return [] if held is None else [held]

    def _views(self, view):
        """(keys and values, pooled blocks or None, whether this layer writes the pooled blocks)."""
        if isinstance(view[0], tuple):  # another entry's views, and pooled blocks of this layer's own beside them
            return view[0][0], view[1], True
        main, pooled = view
        if not self.pool:
            return main, None, False
        if pooled is None:
            raise InvalidInput("this layer sees pooled blocks, but its cache keeps none of its size")
        return main, pooled, not pooled.read_only

    def forward(self, x, ctx, view, rt):
        main, pooled_view, writes_pooled = self._views(view)
        if self.own_kv == main.read_only:
            raise InvalidInput("a layer with keys and values of its own writes them; one without reads another's")
        tokens = x.shape[0]
        rows = self.proj(x, rt)
        tables = self.position.rotary() if self.position is not None else None
        q = rt.ops.head_norm_write(
            rows, self.columns, rt.empty(tokens, self.heads * self.head_dim), self.q_norm, self.k_norm, self.eps,
            tables.cos if tables else None, tables.sin if tables else None, tables.rot_dim if tables else 0, True,
            ctx.tok_slot, ctx.tok_pos, main.k_pages if self.own_kv else None, main.v_pages if self.own_kv else None,
            main.block_table if self.own_kv else None, self.heads, self.kv_heads, self.head_dim, self.value_dim)
        pooled = None
        if pooled_view is not None:
            pooled = rt.ops.PooledBlocks(pooled_view.k_pages, pooled_view.v_pages, pooled_view.block_table, self.pool)
            if writes_pooled:
                rt.ops.pool_blocks(main.k_pages, main.v_pages, main.block_table, pooled, ctx, self.kv_heads, self.head_dim, self.value_dim)
        plan = None
        if self._matrix_cores(rt) and main.k_pages.dtype == torch.bfloat16:
            plan = (self.decode_plan(ctx.batch, ctx.planned_len, rt) if ctx.decode
                    else self.prompt_plan(ctx.batch, ctx.planned_rows, ctx.planned_len, rt))
        attn = rt.ops.attention(q, rt.empty(tokens, self.heads * self.value_dim), main, ctx, self.heads, self.kv_heads, self.head_dim,
                                self.scale, self.window, plan=plan, value_dim=self.value_dim, softcap=self.softcap,
                                extras=self.extras, pooled=pooled)
        gate = rows[:, self.gate_column:self.gate_column + self.heads * self.value_dim]
        rt.ops.sigmoid_gate(attn, gate)
        return self.out(attn, rt)


register_part("mixer", "gated_window_attention", GatedWindowAttention)
