"""A layer's own input from the token: a few columns of a second token table gate a narrow product of the stream.

With x the stream as the layer's feed-forward has left it and e = table[token][first_column : first_column + dim],
the layer's share of a table [vocab, table_width] that all layers declare under one name:

    g = act(W_gate x) * e;    y = W_proj g;    x <- x + y / sqrt(mean(y^2) + eps) * w

The part computes y; the block adds it through the norm (`weight`, `eps`) like any sublayer's output.  The
activation and the product with e are float32 and rounded once.  At bind time the layer's columns are cut out of
the table and, like the two narrow matrices, padded with zeros to a multiple of eight (the few-row products want
rows of 16-byte multiples; a column of zeros adds nothing).
"""

from __future__ import annotations

import torch

from ..kernels import lib as K
from .base import Part, ScaleShape
from .linear import Linear, rows_a_graph_may_hold


class TokenSide(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device, hidden_size: int):
        super().__init__(spec, dtype, device)
        self.hidden_size = hidden_size
        if spec.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}' is not one of {', '.join(K.ACTIVATIONS)}")
        if spec.dim <= 0 or spec.first_column < 0 or spec.first_column + spec.dim > spec.table_width:
            raise ValueError(f"columns {spec.first_column} .. {spec.first_column + spec.dim} of a table of {spec.table_width}")
        self.padded = -(-spec.dim // 8) * 8
        self.eps = spec.eps

    @property
    def graph_max_rows(self):
        return rows_a_graph_may_hold(self.dtype, self.hidden_size, self.padded)

    def tensors(self, prefix):
        s = self.spec
        return {s.table_name: (s.vocab_size, s.table_width),
                prefix + s.gate_name + s.weight_suffix: (s.dim, self.hidden_size),
                prefix + s.proj_name + s.weight_suffix: (self.hidden_size, s.dim),
                prefix + s.norm_name: ScaleShape((self.hidden_size,))}

    def bind(self, prefix, weights):
        s = self.spec
        pad = self.padded - s.dim

        def widened(t: torch.Tensor, axis: int) -> torch.Tensor:
            if not pad:
                return t
            shape = list(t.shape)
            shape[axis] = pad
            return torch.cat([t, torch.zeros(shape, dtype=t.dtype, device=t.device)], dim=axis)

        table = weights[s.table_name]
        self.columns = self.matrix(widened(table[:, s.first_column:s.first_column + s.dim], 1))
        self.gate = Linear(self.matrix(widened(weights[prefix + s.gate_name + s.weight_suffix], 0)))
        self.proj = Linear(self.matrix(widened(weights[prefix + s.proj_name + s.weight_suffix], 1)))
        self.weight = self.vector(weights[prefix + s.norm_name])

    def forward(self, ctx, rows: torch.Tensor):
        """`rows`: the stream in the activation type.  Returns y, as a branch's last product returns it."""
        if ctx.token_ids is None:
            raise ValueError("a layer that reads a second token table needs the step's token ids")
        g = K.token_gate(self.gate(rows), self.columns, ctx.token_ids, self.spec.activation)
        return self.proj.branch(g, None)
