"""A feed-forward of many small gated experts, of which every token uses a few.

Per token, with h the feed-forward's input:  router logits z = W_router h, summed in float32; scores
s = softmax(z) over all experts.  The experts form `groups` equal groups of neighbours; a group's score is the
largest score in it, and only experts of the `groups_kept` best groups can be chosen.  The `top` largest scores
among those are chosen, and the output is

    sum over the chosen e of  (route_scale * s_e) * W_down_e (act(W_gate_e h) * (W_up_e h))

with the weights not renormalised.  Experts have no biases.  A design may add a stored tensor [E] to the scores
where experts (and groups) are compared (`choice_bias_name`); the weights stay the scores themselves.

The experts' matrices are bound stacked, [E, F, H], [E, F, H] and [E, H, F], so that a kernel finds an
expert's weights by its index.  Routing is a function of the token alone, and every (token, expert) pair is
computed by itself, so a token's result does not depend on the batch.  The weighted sum is float32 and is
returned so, for the norm that next reads the stream to add.
"""

from __future__ import annotations

import torch

from ..kernels import lib as K
from .base import Part, plain_rows, register_feed_forward


@register_feed_forward("experts")
class Experts(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}' is not one of {', '.join(K.ACTIVATIONS)}")
        if spec.num_experts <= 0 or spec.groups <= 0 or spec.num_experts % spec.groups:
            raise ValueError(f"{spec.num_experts} experts do not form {spec.groups} equal groups")
        if not 0 < spec.groups_kept <= spec.groups:
            raise ValueError(f"{spec.groups_kept} groups kept of {spec.groups}")
        if not 0 < spec.top <= spec.groups_kept * (spec.num_experts // spec.groups):
            raise ValueError(f"{spec.top} experts chosen, but only "
                             f"{spec.groups_kept * (spec.num_experts // spec.groups)} can be")
        if spec.num_experts > 1024:
            raise ValueError(f"{spec.num_experts} experts: the routing kernel takes up to 1024")
        # for comparing a model with another implementation: called after every routing with (chosen, weights);
        # a step with a tap that reads them on the host cannot be recorded as a graph
        self.routing_tap = None

    def _expert(self, prefix: str, index: int, name: str) -> str:
        s = self.spec
        return f"{prefix}{s.expert_prefix}{index}.{name}{s.weight_suffix}"

    def tensors(self, prefix):
        s = self.spec
        out = {prefix + s.router_name + s.weight_suffix: (s.num_experts, s.hidden_size)}
        if s.choice_bias_name is not None:
            out[prefix + s.choice_bias_name] = (s.num_experts,)
        for e in range(s.num_experts):
            out[self._expert(prefix, e, s.gate_name)] = (s.intermediate_size, s.hidden_size)
            out[self._expert(prefix, e, s.up_name)] = (s.intermediate_size, s.hidden_size)
            out[self._expert(prefix, e, s.down_name)] = (s.hidden_size, s.intermediate_size)
        return out

    def bind(self, prefix, weights):
        s = self.spec
        self.router = self.matrix(weights[prefix + s.router_name + s.weight_suffix])
        self.choice_bias = None
        if s.choice_bias_name is not None:  # it meets the float32 scores
            self.choice_bias = weights[prefix + s.choice_bias_name].to(device=self.device, dtype=torch.float32).contiguous()

        def stacked(name: str, shape) -> torch.Tensor:
            out = torch.empty((s.num_experts, *shape), dtype=self.dtype, device=self.device)
            for e in range(s.num_experts):
                out[e].copy_(weights[self._expert(prefix, e, name)])
            return out

        self.gate = stacked(s.gate_name, (s.intermediate_size, s.hidden_size))
        self.up = stacked(s.up_name, (s.intermediate_size, s.hidden_size))
        self.down = stacked(s.down_name, (s.hidden_size, s.intermediate_size))

    def forward(self, ctx, x):
        s = self.spec
        x = plain_rows(x)
        logits = K.project_f32(x, self.router)
        chosen, weights = K.moe_route(logits, s.groups, s.groups_kept, s.top, s.route_scale, self.choice_bias)
        if self.routing_tap is not None:
            self.routing_tap(chosen, weights)
        return K.moe_experts(x, self.gate, self.up, self.down, chosen, weights, s.activation)
