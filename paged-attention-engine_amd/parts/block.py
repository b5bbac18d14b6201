"""Arrangements of a layer's parts.

"prenorm" is the reference's block (engine/model.py:340-349):
h = h + mixer(norm1(h)); h = h + feed_forward(norm2(h)).  Each branch's output is
left pending on the stream and added by the next norm, in float32.
"""

from __future__ import annotations

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BranchSink, BranchTerms, Part, ResidualStream, ScaleShape,
                   StreamJoin, build_part, plain_rows, register_block)


@register_block("prenorm")
class PreNormBlock:
    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.mixer_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.feed_forward_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
        self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        """The fewest rows any part allows a recorded step to hold (None: no part sets a limit)."""
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def _named(self):
        s = self.spec
        return ((self.mixer_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix),
                (self.feed_forward_norm, s.prefix + s.feed_forward_norm_prefix),
                (self.feed_forward, s.prefix + s.feed_forward_prefix))

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        """Whether a step of `rows` single tokens runs this block through recordable kernels alone."""
        return all(part.decode_fusable(rows, block_size) for part, _ in self._named())

    def entry_fold(self, rows: int):
        """(norm, weight, eps) if whatever fills the stream before this block (the embedding) may
        prepare the first norm's rows for a step of `rows` rows; None if the norm runs its own kernel."""
        fold = getattr(self.mixer_norm, "folded_for", None) if self.mixer.takes_owed_rows else None
        got = fold(rows) if fold is not None else None
        return None if got is None else (self.mixer_norm, *got)

    def forward(self, ctx, stream: ResidualStream) -> None:
        """Each branch is offered a sink: its last product may add itself into the residual and
        prepare the rows of the norm that reads the stream next (this block's second norm, then
        `stream.next_norm`, the first norm of the block that follows), which then runs no kernel."""
        x = self.mixer_norm.forward(stream)
        ctx.sink = BranchSink(stream, self.feed_forward_norm)
        stream.pending = self.mixer.forward(ctx, x if self.mixer.takes_owed_rows else plain_rows(x))
        x = self.feed_forward_norm.forward(stream)
        ctx.sink = BranchSink(stream, stream.next_norm) if stream.next_norm is not None else None
        stream.pending = self.feed_forward.forward(ctx, x if self.feed_forward.takes_owed_rows else plain_rows(x))
        ctx.sink = None


@register_block("branchnorm")
class BranchNormBlock:
    """The norm on each branch's output, and the branches read the stream itself:
    x <- x + m * norm1(mixer(x)); x <- x + m * norm2(feed_forward(x)), m = `residual_scale`.
    A layer whose spec names no feed-forward has the first half only.  The stream is float32; a
    branch's product reads it rounded to the activation type, which the kernel that adds a branch
    writes on the way for the branch after it (`stream.rows`)."""

    reads_stream_rows = True

    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.dtype = dtype
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.mixer_out_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.feed_forward = self.feed_forward_out_norm = None
        if layer_spec.feed_forward is not None:
            self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)
            self.feed_forward_out_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
        for norm in (self.mixer_out_norm, self.feed_forward_out_norm):
            if norm is not None and not hasattr(norm, "add_scaled"):
                raise ValueError(f"the norm '{norm.spec.kind}' cannot stand on a branch's output (no add_scaled)")

    def _named(self):
        s = self.spec
        out = [(self.mixer_out_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix)]
        if self.feed_forward is not None:
            out += [(self.feed_forward_out_norm, s.prefix + s.feed_forward_norm_prefix),
                    (self.feed_forward, s.prefix + s.feed_forward_prefix)]
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def _rows(self, stream: ResidualStream):
        """The stream as a product's operand: what the branch before left, or a cast of the residual."""
        from ..kernels import lib as K
        rows = getattr(stream, "rows", None)
        stream.rows = None
        return rows if rows is not None else K.rows_from_residual(stream.residual, self.dtype)

    def _join(self, stream: ResidualStream, norm, y, more_follows: bool) -> None:
        import torch
        nxt = None
        if more_follows and self.dtype != torch.float32:
            nxt = torch.empty(stream.residual.shape, dtype=self.dtype, device=stream.residual.device)
        norm.add_scaled(stream.residual, y, self.spec.residual_scale, nxt)
        stream.rows = nxt

    def forward(self, ctx, stream: ResidualStream) -> None:
        if stream.pending is not None or stream.owed is not None:
            raise ValueError("a block with its norms on the branches' outputs follows one that left a branch pending")
        ctx.sink = None
        has_ff = self.feed_forward is not None
        y = self.mixer.forward(ctx, self._rows(stream))
        # the rows of the new stream are wanted by this block's feed-forward, or by a block of this
        # kind that follows (the model says whether one does)
        follows = bool(getattr(stream, "rows_wanted_next", False))
        self._join(stream, self.mixer_out_norm, y, has_ff or follows)
        if has_ff:
            y = self.feed_forward.forward(ctx, self._rows(stream))
            self._join(stream, self.feed_forward_out_norm, y, follows)


@register_block("hyper")
class HyperBlock:
    """Pre-norm branches on a stream that is kept in S copies x_1 .. x_S (hyper-connections), each
    branch's output scaled feature by feature before it joins (layer scale).  For sublayer q
    (mixer, then feed-forward) with its tensors in [S], out [S] and mix [S, S] (indexed [from, to]):

        u = sum_s in[s] x_s;   y = scale_q * sublayer(norm_q(u));   x_t <- sum_s mix[s, t] x_s + out[t] y

    for all t at once from the old copies.  Without connection tensors (`connection_prefixes` None)
    the copies are one and the join is x <- x + y; without `layer_scale_names` there is no scale; a
    layer whose spec names no feed-forward has the first half only.  The copies are float32.  A
    branch's output is left pending on the stream with the way it joins (`StreamJoin`), and the norm
    that reads the stream next does join, read and norm in one kernel."""

    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.dtype, self.device = dtype, device
        self.copies = int(layer_spec.streams)
        if layer_spec.connection_prefixes is None and self.copies != 1:
            raise ValueError(f"{self.copies} copies of the stream need connection tensors to join them")
        self.mixer_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.feed_forward = self.feed_forward_norm = None
        if layer_spec.feed_forward is not None:
            self.feed_forward_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
            self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and not hasattr(norm, "forward_copies"):
                raise ValueError(f"the norm '{norm.spec.kind}' cannot read a stream of several copies (no forward_copies)")
        self.reads = [None, None]   # float32 [S]: how each sublayer reads the copies
        self.joins = [None, None]   # StreamJoin: how each sublayer's output joins them

    def _named(self):
        s = self.spec
        out = [(self.mixer_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix)]
        if self.feed_forward is not None:
            out += [(self.feed_forward_norm, s.prefix + s.feed_forward_norm_prefix),
                    (self.feed_forward, s.prefix + s.feed_forward_prefix)]
        return out

    def _sublayers(self):
        return (0, 1) if self.feed_forward is not None else (0,)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def tensors(self):
        s, S = self.spec, self.copies
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        for q in self._sublayers():
            if s.connection_prefixes is not None:
                at = s.prefix + s.connection_prefixes[q]
                out[at + "in"] = (S,)
                out[at + "out"] = (S,)
                out[at + "mix"] = (S, S)
            if s.layer_scale_names is not None:
                out[s.prefix + s.layer_scale_names[q]] = ScaleShape((s.mixer_norm.size,))
        return out

    def bind(self, weights):
        import torch
        s, S = self.spec, self.copies
        for part, prefix in self._named():
            part.bind(prefix, weights)
        f32 = dict(device=self.device, dtype=torch.float32)
        for q in self._sublayers():
            if s.connection_prefixes is not None:
                at = s.prefix + s.connection_prefixes[q]
                read = weights[at + "in"].to(**f32).contiguous()
                mix, out = weights[at + "mix"].to(**f32).contiguous(), weights[at + "out"].to(**f32).contiguous()
            else:
                read, mix, out = (torch.ones(shape, **f32) for shape in ((1,), (1, 1), (1,)))
            scale = None
            if s.layer_scale_names is not None:  # the scale enters the residual sum, which is float32
                scale = weights[s.prefix + s.layer_scale_names[q]].to(**f32).contiguous()
            self.reads[q], self.joins[q] = read, StreamJoin(mix, out, scale)

    def forward(self, ctx, stream: ResidualStream) -> None:
        if stream.owed is not None or stream.copies != self.copies:
            raise ValueError("a block on a stream of several copies follows one that left the stream in another form")
        ctx.sink = None
        x = self.mixer_norm.forward_copies(stream, self.reads[0])
        stream.pending, stream.join = self.mixer.forward(ctx, x), self.joins[0]
        if self.feed_forward is not None:
            x = self.feed_forward_norm.forward_copies(stream, self.reads[1])
            stream.pending, stream.join = self.feed_forward.forward(ctx, x), self.joins[1]


@register_block("parallel")
class ParallelBlock:
    """Both branches read the same stream, each through a norm of its own:
    x <- x + mixer(norm1(x)) + feed_forward(norm2(x)).  A layer whose spec names no feed-forward has the
    mixer alone.  The branches' outputs stay pending on the stream as `BranchTerms`; the kernel that
    norms the stream for the next block (or the model's last norm) adds them into the float32 residual
    first, and forms both of this block's norms from one pass over the row."""

    def __init__(self, layer_spec, dtype, device):
        self.spec = layer_spec
        self.first_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.second_norm = self.feed_forward = None
        if layer_spec.feed_forward is not None:
            self.second_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
            self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)
        for norm in (self.first_norm, self.second_norm):
            if norm is not None and not hasattr(norm, "forward_pair"):
                raise ValueError(f"the norm '{norm.spec.kind}' cannot share a pass over the stream (no forward_pair)")

    def _named(self):
        s = self.spec
        out = [(self.first_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix)]
        if self.feed_forward is not None:
            out += [(self.second_norm, s.prefix + s.feed_forward_norm_prefix),
                    (self.feed_forward, s.prefix + s.feed_forward_prefix)]
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def forward(self, ctx, stream: ResidualStream) -> None:
        ctx.sink = None
        x1, x2 = self.first_norm.forward_pair(stream, self.second_norm)
        terms = BranchTerms()
        for y in (self.mixer.forward(ctx, x1), self.feed_forward.forward(ctx, x2) if self.feed_forward is not None else None):
            if isinstance(y, BranchTerms):
                terms.extend(y)
            elif y is not None:
                terms.append((y, 1.0))
        stream.pending = terms


@register_block("sandwich")
class SandwichBlock:
    """A norm before and a norm after each sublayer:
    x <- x + norm1b(mixer(norm1(x)));  x <- x + norm2b(feed_forward(norm2(x))), and, for a layer whose spec names a
    `token_side`, x <- x + norm_s(side(x, token)) (see parts/token_side.py).  A layer whose spec names no
    feed-forward has no second half.  A sublayer's output (a tensor, float32 partial sums, or the `BranchTerms` of
    mixers side by side) joins the float32 stream in one kernel that norms it, adds it, and writes what reads the
    stream next: the norm before the next sublayer, the stream itself for the token's input, or, after the layer's
    last sublayer, the first norm of the block that follows if that block takes it (`stream.prepared`)."""

    takes_prepared_norm = True

    def __init__(self, layer_spec, dtype, device):
        from .norm import RMSNorm
        from .token_side import TokenSide
        self.spec = layer_spec
        self.dtype = dtype
        if layer_spec.mixer_out_norm is None:
            raise ValueError("the arrangement 'sandwich' needs the norm after the mixer (mixer_out_norm)")
        self.mixer_norm = build_part(NORMS, "norm", layer_spec.mixer_norm, dtype, device)
        self.mixer = build_part(MIXERS, "mixer", layer_spec.mixer, dtype, device)
        self.mixer_out_norm = build_part(NORMS, "norm", layer_spec.mixer_out_norm, dtype, device)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_out_norm = None
        if layer_spec.feed_forward is not None:
            if layer_spec.feed_forward_norm is None or layer_spec.feed_forward_out_norm is None:
                raise ValueError("the arrangement 'sandwich' needs both norms around the feed-forward")
            self.feed_forward_norm = build_part(NORMS, "norm", layer_spec.feed_forward_norm, dtype, device)
            self.feed_forward = build_part(FEED_FORWARDS, "feed-forward", layer_spec.feed_forward, dtype, device)
            self.feed_forward_out_norm = build_part(NORMS, "norm", layer_spec.feed_forward_out_norm, dtype, device)
        for norm in (self.mixer_norm, self.mixer_out_norm, self.feed_forward_norm, self.feed_forward_out_norm):
            if norm is not None and (not isinstance(norm, RMSNorm) or norm.spec.weight_offset):
                raise ValueError(f"the norm '{norm.spec.kind}' cannot ride in the kernel that joins a sublayer's output "
                                 "(an RMS norm with a plain weight can)")
        self.side = None
        if layer_spec.token_side is not None:
            self.side = TokenSide(layer_spec.token_side, dtype, device, layer_spec.mixer_norm.size)

    def _named(self):
        s = self.spec
        out = [(self.mixer_norm, s.prefix + s.mixer_norm_prefix), (self.mixer, s.prefix + s.mixer_prefix),
               (self.mixer_out_norm, s.prefix + s.mixer_out_norm_prefix)]
        if self.feed_forward is not None:
            out += [(self.feed_forward_norm, s.prefix + s.feed_forward_norm_prefix),
                    (self.feed_forward, s.prefix + s.feed_forward_prefix),
                    (self.feed_forward_out_norm, s.prefix + s.feed_forward_out_norm_prefix)]
        if self.side is not None:
            out.append((self.side, s.prefix + s.token_side_prefix))
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for part, _ in self._named())

    @property
    def graph_max_rows(self):
        limits = [part.graph_max_rows for part, _ in self._named() if part.graph_max_rows is not None]
        return min(limits) if limits else None

    def parts(self):
        return [part for part, _ in self._named()]

    def tensors(self):
        out = {}
        for part, prefix in self._named():
            out.update(part.tensors(prefix))
        return out

    def bind(self, weights):
        for part, prefix in self._named():
            part.bind(prefix, weights)

    def _join(self, stream: ResidualStream, y, weight, eps: float, next_norm=None, want_rows: bool = False):
        """x <- x + norm(y) with the norm's `weight` and `eps`; returns (x normed by `next_norm`, x in the activation
        type), each None unless asked for."""
        import torch
        from ..kernels import lib as K
        terms = y if isinstance(y, BranchTerms) else BranchTerms([(y, 1.0)])
        new = lambda: torch.empty(stream.residual.shape, dtype=self.dtype, device=stream.residual.device)
        normed = new() if next_norm is not None else None
        rows = new() if want_rows else None
        K.norm_join(stream.residual, terms, weight, eps, next_norm.weight if next_norm is not None else None,
                    next_norm.spec.eps if next_norm is not None else 0.0, normed, rows)
        return normed, rows

    def _next_first_norm(self, stream: ResidualStream):
        """The first norm of the block that follows, if that block takes its rows prepared (the model says so) and
        the norm is one the joining kernel can form (an RMS norm with a plain weight); else None."""
        norm = stream.next_norm if stream.prepared_wanted_next else None
        if norm is None or not isinstance(norm, type(self.mixer_norm)) or norm.spec.weight_offset:
            return None
        return norm

    def forward(self, ctx, stream: ResidualStream) -> None:
        if stream.pending is not None or stream.owed is not None or stream.copies != 1:
            raise ValueError("a block with norms around its sublayers follows one that left the stream in another form")
        ctx.sink = None
        prepared, stream.prepared = stream.prepared, None
        x = prepared[1] if prepared is not None and prepared[0] is self.mixer_norm else self.mixer_norm.forward(stream)
        follows = self._next_first_norm(stream)
        has_ff, has_side = self.feed_forward is not None, self.side is not None
        y = self.mixer.forward(ctx, x)
        out = self.mixer_out_norm
        x, rows = self._join(stream, y, out.weight, out.spec.eps,
                             self.feed_forward_norm if has_ff else (None if has_side else follows),
                             want_rows=has_side and not has_ff)
        if has_ff:
            y = self.feed_forward.forward(ctx, x)
            out = self.feed_forward_out_norm
            x, rows = self._join(stream, y, out.weight, out.spec.eps, None if has_side else follows, want_rows=has_side)
        if has_side:
            y = self.side.forward(ctx, rows)
            x, _ = self._join(stream, y, self.side.weight, self.side.eps, follows)
        if follows is not None:
            stream.prepared = (follows, x)


def build_block(layer_spec, dtype, device):
    if layer_spec.arrangement not in BLOCKS:
        raise KeyError(f"no block arrangement '{layer_spec.arrangement}'; known: {', '.join(sorted(BLOCKS))}")
    return BLOCKS[layer_spec.arrangement](layer_spec, dtype, device)
