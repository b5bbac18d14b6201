"""The gated delta rule: a recurrent mixer that keeps, per request, one matrix per head and the
last inputs of its short convolutions, instead of keys and values per token.

Per token, with h the mixer's input:  q = W_q h and k = W_k h (G heads of D), v = W_v h (H heads
of V); each passes a causal convolution over time (one filter per channel) and SiLU; q and k
become unit vectors per head (q also times D^-1/2); beta = sigmoid(W_b h) and
decay = exp(-exp(A_log) * softplus(W_a h + dt_bias)), one of each per head.  Head j, which reads
q/k head j // (H / G), then moves its state S [D, V] on:

    S <- decay S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

and o is divided by its root mean square over V, multiplied by a weight shared by the heads and by
silu(W_g h), and projected out by W_o.

For designs that have them (`DeltaMixerSpec.decay`, `decay_rank`, `gate_rank`, `gate_activation`): one decay
per head and key channel, acting on the rows of S (A_log stays one per head, dt_bias is [H, D]); the decay's
input and the gate's through two narrow products each, W_a2 (W_a1 h) and W_g2 (W_g1 h); sigmoid instead of
SiLU on the gate.

The projections that read h are one product over concatenated weights.  The state (the matrices, and the
last taps - 1 inputs of the convolutions) lives in the cache manager's per-request slots as two
named float32 tensors; a request's slot is zeroed when it is taken, which is the design's start
state.  Everything after the projections runs in float32 inside `kernels.lib.delta_rule_step`.
The mixer keeps nothing per token, so a model made of such mixers alone needs no pages.
"""

from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..kernels import lib as K
from .base import Part, ScaleShape, StepShape, plain_rows, register_mixer
from .linear import Linear, rows_a_graph_may_hold

SEQ_RUNS = "runs of the step's sequences"


def sequence_runs(shape: StepShape):
    """For every sequence of the step (first flat row, rows, tokens held before the step, 0)."""
    return {"runs": ([x for start, n, past in zip(shape.q_starts, shape.q_lens, shape.past_lens)
                      for x in (start, n, past, 0)], 4)}


@register_mixer("gated_delta")
class GatedDeltaMixer(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} value heads over {spec.num_kv_heads} query/key heads")
        if not 0 < spec.key_dim <= 1024:
            raise ValueError(f"key_dim {spec.key_dim}: the recurrence kernel takes up to 1024")
        if not 1 <= spec.conv_taps <= 64:
            raise ValueError(f"conv_taps {spec.conv_taps} is outside 1..64")
        if not 0 < spec.value_dim <= 1024:
            raise ValueError(f"value_dim {spec.value_dim}: the kernels take up to 1024")
        if spec.decay not in ("head", "channel"):
            raise ValueError(f"decay '{spec.decay}' is not known (known: head, channel)")
        if spec.gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"gate_activation '{spec.gate_activation}' is not known (known: silu, sigmoid)")

    @property
    def channels(self) -> int:
        s = self.spec
        return 2 * s.num_kv_heads * s.key_dim + s.num_heads * s.value_dim

    @property
    def graph_max_rows(self):
        s = self.spec
        return rows_a_graph_may_hold(self.dtype, s.hidden_size, s.num_heads * s.value_dim)

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.num_heads, s.value_dim, s.key_dim), torch.float32, "matrices"),
                StateSpec((s.conv_taps - 1, self.channels), torch.float32, "conv_tail"))

    def step_lists_key(self, block_size: int):
        return SEQ_RUNS

    def step_lists(self, shape: StepShape):
        return sequence_runs(shape)

    @property
    def decay_width(self) -> int:
        s = self.spec
        return s.num_heads * (s.key_dim if s.decay == "channel" else 1)

    def _projections(self):
        """(name, rows) of the projections of h in the order of the one product's columns: q, k, v first (they
        pass the convolutions), then the gate (or its narrow first product), the decay's input (likewise), beta."""
        s = self.spec
        qk, hv = s.num_kv_heads * s.key_dim, s.num_heads * s.value_dim
        one, _ = s.low_rank_suffixes
        gate = (s.gate_name, hv) if s.gate_rank is None else (s.gate_name + one, s.gate_rank)
        decay = (s.decay_name, self.decay_width) if s.decay_rank is None else (s.decay_name + one, s.decay_rank)
        return ((s.q_name, qk), (s.k_name, qk), (s.v_name, hv), gate, decay, (s.beta_name, s.num_heads))

    def tensors(self, prefix):
        s = self.spec
        _, two = s.low_rank_suffixes
        out = {prefix + name + s.weight_suffix: (rows, s.hidden_size) for name, rows in self._projections()}
        for name, rows in self._projections()[:3]:
            out[prefix + name + s.conv_suffix] = (rows, s.conv_taps)
        if s.gate_rank is not None:
            out[prefix + s.gate_name + two + s.weight_suffix] = (s.num_heads * s.value_dim, s.gate_rank)
        if s.decay_rank is not None:
            out[prefix + s.decay_name + two + s.weight_suffix] = (self.decay_width, s.decay_rank)
        out[prefix + s.a_log_name] = (s.num_heads,)
        out[prefix + s.dt_bias_name] = (self.decay_width,)
        out[prefix + s.norm_name] = ScaleShape((s.value_dim,))
        out[prefix + s.o_name + s.weight_suffix] = (s.hidden_size, s.num_heads * s.value_dim)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        _, two = s.low_rank_suffixes
        stacked = [weights[prefix + name + s.weight_suffix] for name, _ in self._projections()]
        rows = sum(w.shape[0] for w in stacked)
        if rows % 8:
            # rows of zeros behind the last projection: the product's rows then start on 16-byte boundaries, which
            # the few-row kernels want of the views that the narrow products read
            stacked.append(torch.zeros((8 - rows % 8, s.hidden_size), dtype=stacked[0].dtype, device=stacked[0].device))
        self.proj = Linear(self.matrix(torch.cat(stacked, dim=0)))
        self.gate_up = self.decay_up = None
        if s.gate_rank is not None:
            self.gate_up = Linear(self.matrix(weights[prefix + s.gate_name + two + s.weight_suffix]))
        if s.decay_rank is not None:
            self.decay_up = Linear(self.matrix(weights[prefix + s.decay_name + two + s.weight_suffix]))
        f32 = dict(device=self.device, dtype=torch.float32)
        # what enters the recurrence is float32 whatever it is stored in
        self.conv = torch.cat([weights[prefix + name + s.conv_suffix] for name, _ in self._projections()[:3]],
                              dim=0).to(**f32).contiguous()
        self.a_log = weights[prefix + s.a_log_name].to(**f32).contiguous()
        self.dt_bias = weights[prefix + s.dt_bias_name].to(**f32).contiguous()
        self.norm = self.vector(weights[prefix + s.norm_name])
        self.out = Linear(self.matrix(weights[prefix + s.o_name + s.weight_suffix]))

    def forward(self, ctx, x):
        s = self.spec
        if not ctx.writes_cache:
            raise ValueError("a recurrent mixer cannot borrow another stop's state")
        x = plain_rows(x)
        proj = self.proj(x)
        # the product's columns behind q, k, v: [gate | decay input | beta], each as wide as `_projections` says
        at, views = self.channels, []
        for _, rows in self._projections()[3:]:
            views.append(proj[:, at:at + rows])
            at += rows
        gate, decay_in, beta = views
        if self.gate_up is not None:
            gate = self.gate_up(gate)
        if self.decay_up is not None:
            decay_in = self.decay_up(decay_in)
        state = ctx.cache.state_of(ctx.cache_entry)
        runs = ctx.memo[SEQ_RUNS]["runs"]
        out = torch.empty((x.shape[0], s.num_heads * s.value_dim), dtype=x.dtype, device=x.device)
        K.delta_rule_step(proj, out, ctx.tok_seq, ctx.positions, runs, ctx.slots, self.conv, state["conv_tail"],
                          state["matrices"], self.a_log, self.dt_bias, self.norm, s.num_kv_heads, s.num_heads,
                          s.key_dim, s.value_dim, s.conv_taps, s.unit_eps, s.norm_eps, gate=gate, beta=beta,
                          decay_in=decay_in, channel_decay=s.decay == "channel", gate_activation=s.gate_activation)
        return self.out.branch(out, ctx.sink)
