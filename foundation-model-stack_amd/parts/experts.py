"""Feed-forwards beside the gated linear unit: a plain two-layer one, and a mixture of small experts.

``MLP``: down(act(up(x))).

``ExpertsFeedForward``: a router gives every token float32 logits over the experts; the `top` largest are its
experts, weighted by the softmax over those logits alone (`score` "softmax"), by each one's sigmoid ("sigmoid") or by
the sigmoids divided by their sum ("sigmoid_normed").  The weight multiplies the expert's output, or, with
`weight_on` "input", its input (the experts are not linear, so the two differ).  An expert is down(a(gate(x), up(x))) with the clamped
gated activation a(g, u) = g' sigmoid(alpha g') (u' + shift), g' = min(g, limit), u' = clamp(u, -limit, limit).
A shared expert of the same form (sizes and limit of its own) may run for every token, times sigmoid of one
learned logit per token.  Routing, grouping by expert and the experts' products all run on the device: a step never
waits for the host, and a token's result does not depend on what else is in the batch.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import BranchOutput, FeedForward, register_part
from .linear import Linear


class MLP(FeedForward):
    def __init__(self, width: int, hidden_dim: int, activation: str = "gelu", use_bias: bool = False):
        super().__init__()
        activation = str(activation).lower()
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.width, self.hidden_dim, self.activation = width, int(hidden_dim), activation
        self.up = self.add_child("up", Linear(width, self.hidden_dim, use_bias))
        self.down = self.add_child("down", Linear(self.hidden_dim, width, use_bias))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward_branch(x).value()

    def forward_branch(self, x) -> BranchOutput:
        return BranchOutput(ops.activation(self.up.forward(x), self.activation), self.down)


class ExpertsFeedForward(FeedForward):
    def __init__(self, width: int, experts: int, top: int, hidden_dim: int, limit: Optional[float], alpha: float = 1.702,
                 shift: float = 1.0, shared_hidden_dim: int = 0, shared_limit: Optional[float] = None, shared_gate: bool = True,
                 score: str = "softmax", weight_on: str = "output"):
        """limit None: no clamp (with alpha 1 and shift 0 the activation is silu(gate) * up)."""
        super().__init__()
        if score not in ops.ROUTE_SCORES:
            raise ValueError(f"score {score!r} is not one of {sorted(ops.ROUTE_SCORES)}")
        if weight_on not in ("output", "input"):
            raise ValueError(f"weight_on {weight_on!r} is not 'output' or 'input'")
        self.score, self.weight_on = score, weight_on
        limit = float("inf") if limit is None else limit
        if not 0 < top <= experts:
            raise ValueError(f"every token uses {top} of {experts} experts: that must be at least one and at most all")
        self.width, self.experts, self.top, self.hidden_dim = width, int(experts), int(top), int(hidden_dim)
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        self.shared_hidden_dim = int(shared_hidden_dim)
        self.shared_limit = float(shared_limit if shared_limit is not None else limit)
        self.has_shared_gate = bool(shared_gate) and self.shared_hidden_dim > 0
        # the router's rows, and behind them the row of the shared expert's gate: one product, float32 logits
        self.router = self.add_child("router", Linear(width, self.experts + (1 if self.has_shared_gate else 0)))
        self.declare("experts.gate", (self.experts, self.hidden_dim, width))
        self.declare("experts.up", (self.experts, self.hidden_dim, width))
        self.declare("experts.down", (self.experts, width, self.hidden_dim))
        if self.shared_hidden_dim:
            self.shared_gate_up = self.add_child("shared.gate_up", Linear(width, 2 * self.shared_hidden_dim))
            self.shared_down = self.add_child("shared.down", Linear(self.shared_hidden_dim, width))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = self.router.forward(x, out_dtype=torch.float32)
        ids, weights = ops.moe_route(logits, self.experts, self.top, self.score)
        on_input = self.weight_on == "input"
        y = ops.moe_experts(x, ids, self.w["experts.gate"], self.w["experts.up"], self.w["experts.down"], self.limit, self.alpha,
                            self.shift, in_scale=weights if on_input else None)
        shared = gate = None
        if self.shared_hidden_dim:
            hidden = ops.clamped_gated_act(self.shared_gate_up.forward(x), self.shared_limit, self.alpha, self.shift)
            shared = self.shared_down.forward(hidden)
            if self.has_shared_gate:
                gate = logits[:, self.experts]
        return ops.moe_combine(y, None if on_input else weights, shared, gate, x.dtype, top=self.top)


register_part("feed_forward", "mlp", MLP)
register_part("feed_forward", "experts", ExpertsFeedForward)
