"""Causal attention with grouped key/value heads over the paged cache.

Per layer, as in the reference (engine/model.py:281-315): q/k/v projections
(with bias if the spec says so), split into heads of `head_dim` (head j = output
features [j*hd, (j+1)*hd)), position encoding of q and k, new keys and values
stored at their cache slots, attention of every query over the sequence's keys
up to its own position (engine/attention.py:474-487), heads merged, output
projection.  The three projections are one product over concatenated weights;
row-wise dot products are unchanged by the concatenation.

The mixer owns its cache: it declares the pages it keeps (`paged_spec`), stores new
keys and values itself, and builds the work lists of its kernels from the step's shape
(`step_lists`).  The position encoding only encodes; when it is a rotation that hands
out its table, the rotation runs inside the mixer's fused kernels (projection +
rotation + store for up to 64 rows, rotation + store above).

A stop that borrows another stop's cache projects queries only and reads keys
and values written by the owner.

Beyond the reference's attention, each switched by the spec and absent when it says nothing:
values of a width of their own (`value_dim`), an RMS norm of the whole query projection and of the
whole key projection before the rotation (`qk_norm = "projection"`), scores capped by
softcap * tanh(score / softcap), and a learned sink per query head that joins the softmax's
denominator as exp(sink) without a key or a value (`sinks`), or one number that is every head's sink
(`fixed_sink`: with 0 the denominator is one larger than the sum of exponentials), or an RMS norm of
every query and key head by itself with one weight that the heads share (`qk_norm = "per_head"`).
A spec with any of them takes the
path `_forward_wide`: the projection, then one kernel that norms, rotates and stores, then the
attention kernel that knows caps, sinks and value widths.

And for designs that have them (`MixerSpec.convolved`, the path `_forward_convolved`): a short causal
convolution over time on every channel of q, k and v right after the projection, whose last
taps - 1 inputs are per-request state next to the pages; every query and key head divided by its own
root mean square (`qk_norm = "head"`, no weight); a bias by distance instead of a rotation,
score -= 2^(-b (h + 1) / H) * (i - j); a mask in chunks whose borders are multiples of the chunk length in the sequence
(`mask = "chunk"`); a gate sigmoid(W_g x) on the concatenated heads before W_o, whose projection is
part of the one product and which the attention kernel applies as it writes; and layers without
key/value tensors that read an earlier layer's pages (`own_kv = False`).  Pages of such a layer are
never handed back early: a reader with another mask may still want them.
"""

from __future__ import annotations

import torch

from ..cache.manager import StateSpec, attention_pages
from ..kernels import lib as K
from .base import POSITION_ENCODINGS, OwedRows, Part, ScaleShape, StepShape, build_part, plain_rows, register_mixer
from .delta import sequence_runs
from .linear import Linear, rows_a_graph_may_hold

WORK_LISTS = ("paged attention work lists", K.PREFILL_TILE)
CONV_LISTS = ("paged attention work lists and sequence runs", K.PREFILL_TILE)


def attention_work_lists(shape: StepShape):
    """What the matrix-core attention kernels walk: `decode_work`, one (flat row, position, table
    row, 0) for every sequence that brings one token (all a workgroup needs to know of its token in
    one 16-byte load), and `prefill_tiles`, runs of up to PREFILL_TILE consecutive tokens of the
    others as (table row, first flat token, count).  The runs with the most keys come first:
    workgroups start in list order, and the last to finish sets the kernel's time."""
    decode_work = [x for row, (start, n, past) in enumerate(zip(shape.q_starts, shape.q_lens, shape.past_lens))
                   if n == 1 for x in (start, past, row, 0)]
    runs = []
    for row, (start, n, past) in enumerate(zip(shape.q_starts, shape.q_lens, shape.past_lens)):
        if n > 1:
            for first in range(0, n, K.PREFILL_TILE):
                count = min(K.PREFILL_TILE, n - first)
                runs.append((past + first + count, (row, start + first, count)))
    runs.sort(key=lambda run: -run[0])
    return {"decode_work": (decode_work, 4), "prefill_tiles": ([x for _, tile in runs for x in tile], 3)}


def attend_paged(attn, q, k_cache, v_cache, positions, tok_seq, table, work, num_heads: int, num_kv_heads: int,
                 head_dim: int, value_dim: int, scale: float, window: int, softcap: float, sinks) -> None:
    """Attention of a step's queries over the paged cache into `attn`: with `work` (the device lists of
    `attention_work_lists`) on the matrix cores, single tokens by the decode kernel and runs of tokens by
    the prefill kernel; without, by the kernel that takes any shape and precision."""
    if work is not None:
        geometry = (num_heads, num_kv_heads, head_dim, scale, window, softcap, sinks)
        decode_work, prefill_tiles = work["decode_work"], work["prefill_tiles"]
        if decode_work.numel():
            K.attn_decode(attn, q, k_cache, v_cache, decode_work, table, *geometry)
        if prefill_tiles.numel():
            K.attn_prefill(attn, q, k_cache, v_cache, prefill_tiles, positions, table, *geometry)
    else:
        K.paged_attention_capped(attn, q, k_cache, v_cache, positions, tok_seq, table, num_heads, num_kv_heads,
                                 head_dim, value_dim, scale, window, softcap, sinks)


@register_mixer("attention")
class PagedAttention(Part):
    takes_owed_rows = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads over {spec.num_kv_heads} key/value heads")
        if not spec.plain and not (0 < spec.head_dim <= 1024 and 0 < spec.v_dim <= 256):
            raise ValueError(f"head_dim {spec.head_dim} / value_dim {spec.v_dim}: the attention kernel takes up to 1024 / 256")
        if spec.qk_norm not in (None, "projection", "head", "per_head"):
            raise ValueError(f"qk_norm '{spec.qk_norm}' is not known (known: projection, head, per_head)")
        if spec.sinks and spec.fixed_sink is not None:
            raise ValueError("an attention has learned sinks or one fixed sink, not both")
        if spec.mask not in ("window", "chunk"):
            raise ValueError(f"mask '{spec.mask}' is not known (known: window, chunk)")
        if spec.convolved:
            if (spec.position is not None or spec.qk_norm in ("projection", "per_head") or spec.sinks or spec.softcap
                    or spec.fixed_sink is not None):
                raise ValueError("an attention with convolutions, per-head norms, chunks, distance bias or a gate "
                                 "takes no rotation, projection norm, sinks or cap")
            if spec.conv_taps is not None and not 1 <= spec.conv_taps <= 64:
                raise ValueError(f"conv_taps {spec.conv_taps} is outside 1..64")
            if spec.mask == "chunk" and not spec.window:
                raise ValueError("a mask in chunks needs the chunk length (window)")
        elif not spec.own_kv:
            raise ValueError("only the convolution path knows layers without key/value tensors")
        if not spec.plain and not spec.convolved and spec.out_bias:
            raise ValueError("an attention with value widths, caps, sinks or query/key norms takes no bias on its output")
        self.position = (build_part(POSITION_ENCODINGS, "position encoding", spec.position, dtype, device)
                         if spec.position is not None else
                         POSITION_ENCODINGS["none"](None, dtype, device))

    @property
    def graph_safe(self) -> bool:
        return self.position.graph_safe

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.spec.hidden_size, self.spec.num_heads * self.spec.v_dim)

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        """One token a sequence, few rows: the fused projection, the decode attention and the output
        product are all this mixer launches (a rotation that hands out its table runs inside the first)."""
        s = self.spec
        group = s.num_heads // s.num_kv_heads
        return (s.plain and self.dtype == torch.bfloat16 and 0 < rows <= K.program_max_rows() and self._matrix_cores(block_size)
                and s.head_dim in (64, 128) and group * s.head_dim <= 1024 and not s.out_bias
                and hasattr(self.position, "rotary_table") and s.hidden_size % 8 == 0
                and getattr(s.position, "rotary_dim", 0) % 16 == 0
                and K.program_takes_product(rows, s.hidden_size, K.whole_sum_splits(
                    (s.num_heads + 2 * s.num_kv_heads) * s.head_dim, s.hidden_size, rows))
                and K.program_takes_product(rows, s.num_heads * s.head_dim, K.residual_splits(
                    s.hidden_size, s.num_heads * s.head_dim, rows)))

    state_when_borrowing = True  # the convolution on the queries has inputs to remember at every stop

    def paged_spec(self):
        s = self.spec
        return attention_pages(s.num_kv_heads, s.head_dim, None if s.convolved else s.window, s.value_dim)

    @property
    def conv_channels(self) -> int:
        s = self.spec
        return s.num_heads * s.head_dim + (s.num_kv_heads * (s.head_dim + s.v_dim) if s.own_kv else 0)

    def state_spec(self):
        taps = self.spec.conv_taps
        if not taps or taps < 2:
            return None
        return StateSpec((taps - 1, self.conv_channels), torch.float32, "conv_tail")

    def _matrix_cores(self, block_size: int) -> bool:
        s = self.spec
        return (s.v_dim == s.head_dim
                and K.mfma_attention_supported(self.dtype, s.num_heads, s.num_kv_heads, s.head_dim, block_size))

    def step_lists_key(self, block_size: int):
        if self.spec.convolved:
            return CONV_LISTS
        return WORK_LISTS if self._matrix_cores(block_size) else None

    def step_lists(self, shape: StepShape):
        if self.spec.convolved:
            return {**attention_work_lists(shape), **sequence_runs(shape)}
        return attention_work_lists(shape)

    def _projections(self):
        """(name, rows) of the projections that pass the convolution, in the order of the product's columns."""
        s = self.spec
        out = [(s.q_name, s.num_heads * s.head_dim)]
        if s.own_kv:
            out += [(s.k_name, s.num_kv_heads * s.head_dim), (s.v_name, s.num_kv_heads * s.v_dim)]
        return out

    def tensors(self, prefix):
        s = self.spec
        if s.convolved:
            out = {prefix + s.o_name + s.weight_suffix: (s.hidden_size, s.num_heads * s.v_dim)}
            for name, rows in self._projections():
                out[prefix + name + s.weight_suffix] = (rows, s.hidden_size)
                if s.qkv_bias:
                    out[prefix + name + s.bias_suffix] = (rows,)
                if s.conv_taps is not None:
                    out[prefix + name + s.conv_suffix] = (rows, s.conv_taps)
            if s.gate_name is not None:
                out[prefix + s.gate_name + s.weight_suffix] = (s.num_heads * s.v_dim, s.hidden_size)
            if s.out_bias:
                out[prefix + s.o_name + s.bias_suffix] = (s.hidden_size,)
            return out
        out = {prefix + s.q_name + s.weight_suffix: (s.num_heads * s.head_dim, s.hidden_size),
               prefix + s.k_name + s.weight_suffix: (s.num_kv_heads * s.head_dim, s.hidden_size),
               prefix + s.v_name + s.weight_suffix: (s.num_kv_heads * s.v_dim, s.hidden_size),
               prefix + s.o_name + s.weight_suffix: (s.hidden_size, s.num_heads * s.v_dim)}
        if s.qk_norm == "per_head":
            out[prefix + s.q_norm_name] = ScaleShape((s.head_dim,))
            out[prefix + s.k_norm_name] = ScaleShape((s.head_dim,))
        elif s.qk_norm:
            out[prefix + s.q_norm_name] = ScaleShape((s.num_heads * s.head_dim,))
            out[prefix + s.k_norm_name] = ScaleShape((s.num_kv_heads * s.head_dim,))
        if s.sinks:
            out[prefix + s.sink_name] = (s.num_heads,)
        if s.qkv_bias:
            out[prefix + s.q_name + s.bias_suffix] = (s.num_heads * s.head_dim,)
            out[prefix + s.k_name + s.bias_suffix] = (s.num_kv_heads * s.head_dim,)
            out[prefix + s.v_name + s.bias_suffix] = (s.num_kv_heads * s.v_dim,)
        if s.out_bias:
            out[prefix + s.o_name + s.bias_suffix] = (s.hidden_size,)
        return out

    def _bind_convolved(self, prefix, weights):
        s = self.spec
        f32 = dict(device=self.device, dtype=torch.float32)
        named = self._projections()
        parts = [weights[prefix + name + s.weight_suffix] for name, _ in named]
        bias = [weights[prefix + name + s.bias_suffix] for name, _ in named] if s.qkv_bias else None
        if s.gate_name is not None:  # the gate reads the same input: its rows ride in the same product, without a bias
            parts.append(weights[prefix + s.gate_name + s.weight_suffix])
            if bias is not None:
                bias.append(torch.zeros(s.num_heads * s.v_dim, dtype=bias[0].dtype, device=bias[0].device))
        self.qkv = Linear(self.matrix(torch.cat(parts, dim=0)), None if bias is None else self.vector(torch.cat(bias, dim=0)))
        if s.conv_taps is not None:
            self.conv = torch.cat([weights[prefix + name + s.conv_suffix] for name, _ in named], dim=0).to(**f32).contiguous()
        else:
            self.conv = torch.ones((self.conv_channels, 1), **f32)
        ob = weights[prefix + s.o_name + s.bias_suffix] if s.out_bias else None
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]), None if ob is None else self.vector(ob))
        self.slopes = None
        if s.distance_slope_base is not None:
            h = torch.arange(1, s.num_heads + 1, dtype=torch.float64)
            self.slopes = torch.pow(2.0, -float(s.distance_slope_base) * h / s.num_heads).to(**f32).contiguous()

    def bind(self, prefix, weights):
        s = self.spec
        if s.convolved:
            return self._bind_convolved(prefix, weights)
        names = (s.q_name, s.k_name, s.v_name)
        w = torch.cat([weights[prefix + n + s.weight_suffix] for n in names], dim=0)
        b = (torch.cat([weights[prefix + n + s.bias_suffix] for n in names], dim=0) if s.qkv_bias else None)
        self.qkv = Linear(self.matrix(w), None if b is None else self.vector(b))
        nq = s.num_heads * s.head_dim
        self.q_only = Linear(self.qkv.weight[:nq], None if b is None else self.qkv.bias[:nq])
        ob = weights[prefix + s.o_name + s.bias_suffix] if s.out_bias else None
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]), None if ob is None else self.vector(ob))
        self.q_norm = self.k_norm = self.sinks = None
        if s.qk_norm:
            self.q_norm = self.vector(weights[prefix + s.q_norm_name])
            self.k_norm = self.vector(weights[prefix + s.k_norm_name])
        if s.sinks:  # sinks enter the softmax, which is float32
            self.sinks = weights[prefix + s.sink_name].to(device=self.device, dtype=torch.float32).contiguous()
        elif s.fixed_sink is not None:
            self.sinks = torch.full((s.num_heads,), float(s.fixed_sink), dtype=torch.float32, device=self.device)

    def _project_encode_store(self, ctx, x, k_cache, v_cache, table):
        """Queries (and, at a stop that owns its cache, keys and values) of the step's tokens:
        projected, encoded by position, the new keys and values stored.  Returns rows whose first
        num_heads * head_dim features are the encoded queries."""
        s = self.spec
        bs = ctx.cache.block_size
        if ctx.writes_cache:
            linear, nkv = self.qkv, s.num_kv_heads
        else:
            linear, nkv, k_cache, v_cache, table = self.q_only, 0, None, None, None
        rotary = getattr(self.position, "rotary_table", None)
        owed = x if isinstance(x, OwedRows) else None
        if owed is not None:
            x = owed.rows
        if rotary is None:
            # any encoding: project, let it encode query and key heads in place, then store
            qkv = linear(owed if owed is not None else x)
            self.position.encode(ctx, qkv, s.num_heads + nkv, s.head_dim)
            if nkv:
                K.kv_store(qkv, s.num_heads, nkv, s.head_dim, ctx.positions, ctx.tok_seq, table, bs, k_cache, v_cache)
            return qkv
        rot, cos_sin = rotary(ctx)
        if x.dtype == torch.bfloat16 and K.skinny_rope_supported(x, linear.weight, s.head_dim, rot):
            # up to 64 rows: one kernel projects, rotates and stores
            q = torch.empty((x.shape[0], s.num_heads * s.head_dim), dtype=x.dtype, device=x.device)
            splits = K.whole_sum_splits(linear.out_features, linear.in_features, x.shape[0])
            K.gemm_skinny_rope(q, x, linear.weight, linear.bias, s.num_heads, nkv, s.head_dim, rot, cos_sin,
                               ctx.positions, ctx.tok_seq, table, bs, k_cache, v_cache, splits,
                               row_scale=owed.row_scale if owed is not None else None)
            return q
        # many rows: the library's plain product (its variant with a bias costs the host six times the
        # call), and the bias is added by the kernel that rotates and stores, which follows anyway
        qkv = linear.without_bias(x) if owed is None else None
        bias = linear.bias if qkv is not None else None
        if qkv is None:
            qkv = linear(owed if owed is not None else x)
        K.rope_kv_write(qkv, s.num_heads, nkv, s.head_dim, rot, cos_sin, ctx.positions, ctx.tok_seq, table, bs,
                        k_cache, v_cache, bias)
        return qkv

    def _forward_wide(self, ctx, x):
        """The path of a spec that is not `plain`: see the module's text."""
        s = self.spec
        pages = ctx.cache.pages_of(ctx.cache_entry)
        table = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)]
        if ctx.writes_cache:
            qkv, nkv, k_cache, v_cache = self.qkv(x), s.num_kv_heads, pages["k"], pages["v"]
        else:
            qkv, nkv, k_cache, v_cache = self.q_only(x), 0, None, None
        rotary = getattr(self.position, "rotary_table", None)
        if rotary is None and s.position is not None:
            raise ValueError("an attention with value widths, caps, sinks or query/key norms rotates by a table")
        rot, cos_sin = rotary(ctx) if rotary is not None else (0, None)
        K.qk_norm_rotate_store(qkv, s.num_heads, nkv, s.head_dim, s.v_dim, self.q_norm, self.k_norm if nkv else None,
                               s.qk_norm_eps, rot, bool(getattr(self.position, "interleaved", False)), cos_sin,
                               float(getattr(self.position, "magnitude", 1.0)), ctx.positions,
                               ctx.tok_seq if nkv else None, table if nkv else None, ctx.cache.block_size,
                               k_cache, v_cache, per_head=s.qk_norm == "per_head")
        attn = torch.empty((qkv.shape[0], s.num_heads * s.v_dim), dtype=qkv.dtype, device=qkv.device)
        work = ctx.memo.get(WORK_LISTS) if self._matrix_cores(ctx.cache.block_size) else None
        attend_paged(attn, qkv, pages["k"], pages["v"], ctx.positions, ctx.tok_seq, table, work, s.num_heads,
                     s.num_kv_heads, s.head_dim, s.v_dim, s.scale, s.window or 0, s.softcap or 0.0, self.sinks)
        return self.out.branch(attn, ctx.sink)

    def _forward_convolved(self, ctx, x):
        """The path of a spec that is `convolved`: one product [q | k | v | gate], one kernel that
        convolves, norms the heads and stores, and the attention kernel that knows chunks, the distance
        bias and the gate."""
        s = self.spec
        if s.own_kv != ctx.writes_cache:
            raise ValueError("a layer with key/value tensors writes its own pages, one without reads another stop's")
        pages = ctx.cache.pages_of(ctx.cache_entry)
        table = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)]
        proj = self.qkv(x)
        nkv = s.num_kv_heads if s.own_kv else 0
        taps = s.conv_taps or 1
        lists = ctx.memo[CONV_LISTS]
        q = torch.empty((proj.shape[0], s.num_heads * s.head_dim), dtype=proj.dtype, device=proj.device)
        K.conv_norm_store(proj, q, ctx.tok_seq, ctx.positions, lists["runs"], ctx.slots, self.conv,
                          ctx.cache.state_of(ctx.entry) if taps > 1 else None, taps, s.num_heads, nkv, s.head_dim, s.v_dim,
                          s.qk_norm == "head", s.qk_norm_eps, table if nkv else None, ctx.cache.block_size,
                          pages["k"] if nkv else None, pages["v"] if nkv else None)
        gate = None
        if s.gate_name is not None:
            first = self.conv_channels
            gate = proj[:, first:first + s.num_heads * s.v_dim]
        attn = torch.empty((proj.shape[0], s.num_heads * s.v_dim), dtype=proj.dtype, device=proj.device)
        chunked = s.mask == "chunk"
        if self._matrix_cores(ctx.cache.block_size) and s.scale > 0:
            # single tokens by the decode kernel, runs of tokens by the prefill kernel, both on the matrix cores
            geometry = (s.num_heads, s.num_kv_heads, s.head_dim, s.scale, s.window or 0, 0.0, None, chunked, self.slopes, gate)
            if lists["decode_work"].numel():
                K.attn_decode(attn, q, pages["k"], pages["v"], lists["decode_work"], table, *geometry)
            if lists["prefill_tiles"].numel():
                K.attn_prefill(attn, q, pages["k"], pages["v"], lists["prefill_tiles"], ctx.positions, table, *geometry)
        else:
            K.paged_attention_masked(attn, q, pages["k"], pages["v"], ctx.positions, ctx.tok_seq, table, s.num_heads,
                                     s.num_kv_heads, s.head_dim, s.v_dim, s.scale, s.window or 0, chunked, self.slopes, gate)
        return self.out.branch(attn, ctx.sink)

    def forward(self, ctx, x):
        """`x`: normalised activations, or `OwedRows` (the projection then pays their scale)."""
        s = self.spec
        if s.convolved:
            return self._forward_convolved(ctx, plain_rows(x))
        if not s.plain:
            return self._forward_wide(ctx, plain_rows(x))
        pages = ctx.cache.pages_of(ctx.cache_entry)  # as declared in `paged_spec`
        k_cache, v_cache = pages["k"], pages["v"]
        table = ctx.block_tables[ctx.cache.group_of(ctx.cache_entry)]
        qkv = self._project_encode_store(ctx, x, k_cache, v_cache, table)
        attn = torch.empty((x.shape[0], s.num_heads * s.head_dim), dtype=x.dtype, device=x.device)
        geometry = (s.num_heads, s.num_kv_heads, s.head_dim, s.scale, s.window or 0)
        work = ctx.memo.get(WORK_LISTS) if self._matrix_cores(ctx.cache.block_size) else None
        if work is not None:
            decode_work, prefill_tiles = work["decode_work"], work["prefill_tiles"]
            if decode_work.numel():
                K.attn_decode(attn, qkv, k_cache, v_cache, decode_work, table, *geometry)
            if prefill_tiles.numel():
                K.attn_prefill(attn, qkv, k_cache, v_cache, prefill_tiles, ctx.positions, table, *geometry)
        else:
            K.paged_attention_generic(attn, qkv, k_cache, v_cache, ctx.positions, ctx.tok_seq, table, *geometry)
        return self.out.branch(attn, ctx.sink)
