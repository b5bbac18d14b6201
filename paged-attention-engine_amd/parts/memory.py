"""A matrix memory with exponential gates (the mLSTM cell): a recurrent mixer that keeps, per request and
head, a matrix C [D, V], the sum n [D] of its gated keys and a running maximum m of the gates' logarithms.

Per token, with h the mixer's input:  q = W_q h * D^-1/2, k = W_k h (H heads of D), v = W_v h (H heads of V);
with the cap c, the input gate's logarithm is i = c tanh((W_i h + b_i) / c) and the forget gate's
f = logsigmoid(c tanh((W_f h + b_f) / c)).  Then, with m starting at 0 like C and n:

    m_t = max(f + m_(t-1), i)
    C <- exp(f + m_(t-1) - m_t) C + exp(i - m_t) k v^T;    n likewise with k alone
    o = C^T q / (max(|n . q|, exp(-m_t)) + floor)

Each head's o is divided by its root mean square over V, multiplied by a weight (one per head and feature)
and by sigmoid(W_g h), and projected out by W_o.

q, k, v and the output gate are one product over concatenated weights; the two gates' sums are formed in
float32 by a product of their own (their logarithms add up over a sequence, so they do not pass the
activation type).  The state lives in the cache manager's per-request slots as two named float32 tensors,
"memory" [H, V + 1, D] (column V holds n: it is the memory's column for a value that is always 1) and
"memory_max" [H]; a slot is zeroed when a request takes it, which is the design's start state.  Everything
after the projections is float32 inside `kernels.lib.matrix_memory_step`.  Nothing is kept per token.
"""

from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..kernels import lib as K
from .base import Part, ScaleShape, StepShape, plain_rows, register_mixer
from .delta import SEQ_RUNS, sequence_runs
from .linear import Linear, rows_a_graph_may_hold


@register_mixer("matrix_memory")
class MatrixMemory(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if min(spec.num_heads, spec.key_dim, spec.value_dim) <= 0:
            raise ValueError("matrix memory: heads, key_dim and value_dim must be positive")
        if spec.key_dim > 1024 or spec.value_dim > 1023:
            raise ValueError(f"matrix memory: key_dim {spec.key_dim} / value_dim {spec.value_dim}: the kernels take up to 1024 / 1023")
        if not spec.gate_cap > 0:
            raise ValueError(f"matrix memory: gate_cap must be positive, got {spec.gate_cap}")

    @property
    def graph_max_rows(self):
        s = self.spec
        return rows_a_graph_may_hold(self.dtype, s.hidden_size, s.num_heads * s.value_dim)

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.num_heads, s.value_dim + 1, s.key_dim), torch.float32, "memory"),
                StateSpec((s.num_heads,), torch.float32, "memory_max"))

    def step_lists_key(self, block_size: int):
        return SEQ_RUNS

    def step_lists(self, shape: StepShape):
        return sequence_runs(shape)

    def _projections(self):
        """(name, rows) of the projections that share one product, in the order of its columns."""
        s = self.spec
        hd, hv = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        return ((s.q_name, hd), (s.k_name, hd), (s.v_name, hv), (s.gate_name, hv))

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + name + s.weight_suffix: (rows, s.hidden_size) for name, rows in self._projections()}
        for name in (s.input_gate_name, s.forget_gate_name):
            out[prefix + name + s.weight_suffix] = (s.num_heads, s.hidden_size)
            out[prefix + name + s.bias_suffix] = (s.num_heads,)
        out[prefix + s.norm_name] = ScaleShape((s.num_heads * s.value_dim,))
        out[prefix + s.o_name + s.weight_suffix] = (s.hidden_size, s.num_heads * s.value_dim)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        self.proj = Linear(self.matrix(torch.cat([weights[prefix + name + s.weight_suffix]
                                                  for name, _ in self._projections()], dim=0)))
        gates = (s.input_gate_name, s.forget_gate_name)
        self.gate_weight = self.matrix(torch.cat([weights[prefix + name + s.weight_suffix] for name in gates], dim=0))
        # what enters the recurrence is float32 whatever it is stored in
        self.gate_bias = torch.cat([weights[prefix + name + s.bias_suffix] for name in gates], dim=0).to(
            device=self.device, dtype=torch.float32).contiguous()
        self.norm = self.vector(weights[prefix + s.norm_name])
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]))

    def forward(self, ctx, x):
        s = self.spec
        if not ctx.writes_cache:
            raise ValueError("a recurrent mixer cannot borrow another stop's state")
        x = plain_rows(x)
        H, D, V = s.num_heads, s.key_dim, s.value_dim
        proj = self.proj(x)
        gate_logits = K.project_f32(x, self.gate_weight, self.gate_bias)
        state = ctx.cache.state_of(ctx.cache_entry)
        out = torch.empty((x.shape[0], H * V), dtype=x.dtype, device=x.device)
        K.matrix_memory_step(proj, proj[:, 2 * H * D + H * V:], gate_logits, out, ctx.memo[SEQ_RUNS]["runs"], ctx.slots,
                             state["memory"], state["memory_max"], self.norm, H, D, V, s.gate_cap, s.norm_eps,
                             s.readout_floor)
        return self.out.branch(out, ctx.sink)
