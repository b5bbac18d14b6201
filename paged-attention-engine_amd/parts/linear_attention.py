"""Gated linear attention: a recurrent mixer that keeps, per request, one matrix per head that decays by a
learned factor per key channel, instead of keys and values per token.

Per token, with h the mixer's input:  q = W_q h * D^-1/2 and k = W_k h (H heads of D), v = W_v h (H heads of V);
the decay of head j's key channel d is  a = sigmoid(z)^(1 / tau)  with  z = W_a2 (W_a1 h) + b  laid out [H, D].
Head j then moves its state S [D, V] on:

    S <- diag(a) S + k v^T;   o = S^T q

(the decay multiplies the rows of S, which belong to key channels), and o is divided by its root mean square
over V, multiplied by a weight [V] that the heads share and by silu(W_g h) (or sigmoid, by the spec), and
projected out by W_o.

The projections that read h (q, k, v, the gate, the decay's first narrow product) are one product over
concatenated weights.  The state lives in the cache manager's per-request slots as a float32 tensor "matrices"
[H, V, D]; a slot is zeroed when a request takes it, which is the design's start state.  Everything after the
projections runs in float32 inside `kernels.lib.linear_attention_step`: the decay's bias, its logarithm and
exponential, the state, the read-out, the norm and the gate.  The mixer keeps nothing per token.
"""

from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..kernels import lib as K
from .base import Part, ScaleShape, StepShape, plain_rows, register_mixer
from .delta import SEQ_RUNS, sequence_runs
from .linear import Linear, rows_a_graph_may_hold


@register_mixer("gated_linear_attention")
class GatedLinearAttention(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if min(spec.num_heads, spec.key_dim, spec.value_dim, spec.decay_rank) <= 0:
            raise ValueError("gated linear attention: heads, key_dim, value_dim and decay_rank must be positive")
        if spec.key_dim > 1024 or spec.value_dim > 1024:
            raise ValueError(f"gated linear attention: key_dim {spec.key_dim} / value_dim {spec.value_dim}: "
                             "the kernels take up to 1024")
        if not spec.decay_temperature > 0:
            raise ValueError(f"gated linear attention: decay_temperature must be positive, got {spec.decay_temperature}")
        if spec.gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"gate_activation '{spec.gate_activation}' is not known (known: silu, sigmoid)")

    @property
    def graph_max_rows(self):
        s = self.spec
        return rows_a_graph_may_hold(self.dtype, s.hidden_size, s.num_heads * s.value_dim, s.decay_rank)

    def state_spec(self):
        s = self.spec
        return StateSpec((s.num_heads, s.value_dim, s.key_dim), torch.float32, "matrices")

    def step_lists_key(self, block_size: int):
        return SEQ_RUNS

    def step_lists(self, shape: StepShape):
        return sequence_runs(shape)

    def _projections(self):
        """(name, rows) of the projections of h in the order of the one product's columns."""
        s = self.spec
        hd, hv = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        return ((s.q_name, hd), (s.k_name, hd), (s.v_name, hv), (s.gate_name, hv), (s.decay_name + "1", s.decay_rank))

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + name + s.weight_suffix: (rows, s.hidden_size) for name, rows in self._projections()}
        out[prefix + s.decay_name + "2" + s.weight_suffix] = (s.num_heads * s.key_dim, s.decay_rank)
        out[prefix + s.decay_name + "2" + s.bias_suffix] = (s.num_heads * s.key_dim,)
        out[prefix + s.norm_name] = ScaleShape((s.value_dim,))
        out[prefix + s.o_name + s.weight_suffix] = (s.hidden_size, s.num_heads * s.value_dim)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        stacked = [weights[prefix + name + s.weight_suffix] for name, _ in self._projections()]
        # rows of zeros before the narrow product's weights and behind them: the product's columns that the second
        # narrow product reads then start, and its rows end, on 16-byte boundaries, which the few-row kernels want
        before = sum(w.shape[0] for w in stacked[:-1])
        self.narrow_at = -(-before // 8) * 8
        self.narrow_width = -(-s.decay_rank // 8) * 8
        zeros = lambda rows: torch.zeros((rows, s.hidden_size), dtype=stacked[0].dtype, device=stacked[0].device)
        pieces = stacked[:-1] + [zeros(self.narrow_at - before), stacked[-1], zeros(self.narrow_width - s.decay_rank)]
        self.proj = Linear(self.matrix(torch.cat([p for p in pieces if p.shape[0]], dim=0)))
        second = weights[prefix + s.decay_name + "2" + s.weight_suffix]
        if self.narrow_width != s.decay_rank:  # columns of zeros meet the rows of zeros above
            second = torch.cat([second, torch.zeros((second.shape[0], self.narrow_width - s.decay_rank), dtype=second.dtype,
                                                    device=second.device)], dim=1)
        self.decay_up = Linear(self.matrix(second))
        # what enters the recurrence is float32 whatever it is stored in
        self.decay_bias = weights[prefix + s.decay_name + "2" + s.bias_suffix].to(device=self.device, dtype=torch.float32).contiguous()
        self.norm = self.vector(weights[prefix + s.norm_name])
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]))

    def forward(self, ctx, x):
        s = self.spec
        if not ctx.writes_cache:
            raise ValueError("a recurrent mixer cannot borrow another stop's state")
        x = plain_rows(x)
        H, D, V = s.num_heads, s.key_dim, s.value_dim
        proj = self.proj(x)
        gate = proj[:, 2 * H * D + H * V:2 * H * D + 2 * H * V]
        decay_in = self.decay_up(proj[:, self.narrow_at:self.narrow_at + self.narrow_width])
        state = ctx.cache.state_of(ctx.cache_entry)
        if isinstance(state, dict):  # beside another mixer that keeps state, the tensors are found by name
            state = state["matrices"]
        out = torch.empty((x.shape[0], H * V), dtype=x.dtype, device=x.device)
        K.linear_attention_step(proj, decay_in, self.decay_bias, s.decay_temperature, gate, out, ctx.memo[SEQ_RUNS]["runs"],
                                ctx.slots, state, self.norm, H, D, V, s.norm_eps, s.gate_activation)
        return self.out.branch(out, ctx.sink)
