"""RMS normalisation fused with the pending residual add.

Formula of the reference (engine/model.py:117-123): variance and scaling in
float32, the result cast to the activation type and then multiplied by the
weight.  The residual sum itself stays float32 here (the reference adds in the
activation type, engine/model.py:343,349).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import lib as K
from .base import BranchTerms, OwedRows, Part, ResidualStream, ScaleShape, register_norm


@register_norm("rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    def tensors(self, prefix):
        # a weight that is stored minus an offset lies around zero like any other tensor
        shape = (self.spec.size,)
        return {prefix + self.spec.weight_name: shape if self.spec.weight_offset else ScaleShape(shape)}

    def bind(self, prefix, weights):
        stored = weights[prefix + self.spec.weight_name]
        if self.spec.weight_offset:
            # offset + w is formed in float32 and stays so: rounded to the storage type it would lose w's last bits
            self.weight = (stored.to(device=self.device, dtype=torch.float32) + float(self.spec.weight_offset)).contiguous()
        else:
            self.weight = self.vector(stored)

    def folded_for(self, rows: int):
        """(weight, eps) if, in a step of `rows` rows, whatever writes the residual before this norm
        may prepare its rows instead (see `OwedRows`: the consumer's product then pays the scale and
        no norm kernel runs); None if this norm wants to run its own kernel.  The limits are those of
        the products that pay (bfloat16, few rows, rows of 16-byte multiples) and of where it pays
        (`kernels.lib.folds`)."""
        if self.dtype != torch.bfloat16 or not K.folds(rows, self.spec.size) or self.spec.size % 8:
            return None
        return self.weight, self.spec.eps

    def decode_fusable(self, rows: int, block_size: int) -> bool:
        return self.folded_for(rows) is not None  # then `forward` hands prepared rows on and launches nothing

    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None):
        """Add the pending branch output into the residual and return the normalised
        rows.  With `rows` (int32 indices) only those rows are produced and the
        stream is left untouched.  When the branch before has added itself into the residual
        and prepared this norm's rows, they are returned as they are (`OwedRows`): no kernel runs."""
        if stream.copies > 1 or stream.join is not None:
            return self.forward_copies(stream, stream.sum_weights, rows)
        if isinstance(stream.pending, BranchTerms):
            return self.forward_pair(stream, None, rows)[0]
        if stream.owed is not None:
            owed, mine = stream.owed, stream.owed_to is self
            if rows is None:
                stream.owed = stream.owed_to = None
                if mine:
                    return owed
            # prepared for another norm, or only some rows are wanted: the residual is complete
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=stream.residual.device)
        K.add_rmsnorm(stream.residual, stream.pending, self.weight, self.spec.eps, out, rows)
        if rows is None:
            stream.pending = None
        return out

    def forward_pair(self, stream: ResidualStream, other: Optional["RMSNorm"], rows: Optional[torch.Tensor] = None):
        """For blocks whose branches read the same stream: the pending branches (a tensor, or `BranchTerms`)
        join the residual, and the new residual is normed by this norm and by `other` (None: by this one
        alone) in one kernel.  Returns both results.  With `rows` only those rows, and the stream stays as it is."""
        if stream.owed is not None or stream.copies > 1:
            raise ValueError("a norm for two branches reads a plain stream with nothing prepared for another norm")
        pending = stream.pending
        terms = pending if isinstance(pending, BranchTerms) else BranchTerms([] if pending is None else [(pending, 1.0)])
        n = stream.residual.shape[0] if rows is None else rows.numel()
        new = lambda: torch.empty((n, self.spec.size), dtype=self.dtype, device=stream.residual.device)
        out1, out2 = new(), (new() if other is not None else None)
        if other is not None and other.spec.eps != self.spec.eps:
            raise ValueError("two norms of one stream in one kernel share their eps")
        K.sum_norm2(stream.residual, terms, self.weight, other.weight if other is not None else None, self.spec.eps,
                    out1, out2, rows)
        if rows is None:
            stream.pending = None
        return out1, out2

    def forward_copies(self, stream: ResidualStream, read_weights: torch.Tensor,
                       rows: Optional[torch.Tensor] = None):
        """The norm on a stream kept in several copies: the pending branch joins them as `stream.join`
        says, then the row sum_s read_weights[s] x_s is normed.  Sum and norm are float32 and the
        result is rounded once.  With `rows` only those rows are produced and the stream stays as it is."""
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=stream.residual.device)
        join = stream.join if stream.pending is not None else None
        if stream.pending is not None and join is None:
            raise ValueError("a branch is pending on a stream of several copies without the way it joins them")
        K.hyper_norm(stream.residual, stream.copies, stream.pending if join else None, join.scale if join else None,
                     join.mix if join else None, join.out if join else None, read_weights, self.weight, self.spec.eps,
                     out, rows)
        if rows is None:
            stream.pending = stream.join = None
        return out

    def add_scaled(self, residual: torch.Tensor, y: torch.Tensor, scale: float,
                   next_rows: Optional[torch.Tensor] = None) -> None:
        """The norm on a branch's output: residual += scale * norm(y), in float32 (`y` in the activation
        type, or float32 partial sums [P, T, H]); `next_rows` receives the new residual in the
        activation type, for the product that reads the stream next."""
        K.norm_scale_add(residual, y, self.weight, self.spec.eps, scale, next_rows)
