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
    POLYNORM = "polynorm"

    def __init__(self, width: int, hidden_dim: int, activation: str = "gelu", use_bias: bool = False, eps: float = 1e-6):
        """activation "polynorm": a N(z) + b N(z^2) + c N(z^3) + e with four learned numbers (the parameter `act`), powers
        taken element by element, N dividing a token's hidden values by their root mean square (`eps` inside the root)."""
        super().__init__()
        activation = str(activation).lower()
        if activation != self.POLYNORM and activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS) + [self.POLYNORM]}")
        self.width, self.hidden_dim, self.activation, self.eps = width, int(hidden_dim), activation, float(eps)
        self.up = self.add_child("up", Linear(width, self.hidden_dim, use_bias))
        self.down = self.add_child("down", Linear(self.hidden_dim, width, use_bias))
        self._coefficients = None
        if activation == self.POLYNORM:
            self.declare("act", (4,), init="ones", kind="scale")

    def finalize(self, device, dtype) -> None:
        if self.activation == self.POLYNORM:
            self._coefficients = tuple(float(v) for v in self.w["act"].to(torch.float32).tolist())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward_branch(x).value()

    def forward_branch(self, x) -> BranchOutput:
        if self.activation == self.POLYNORM:
            # the three norms are formed from the float32 sums of the product
            hidden = ops.poly_norm(self.up.forward(x, out_dtype=torch.float32), self._coefficients, self.eps, x.dtype)
            return BranchOutput(hidden, self.down)
        return BranchOutput(ops.activation(self.up.forward(x), self.activation), self.down)


class ExpertsFeedForward(FeedForward):
    def __init__(self, width: int, experts: int, top: int, hidden_dim: int, limit: Optional[float], alpha: float = 1.702,
                 shift: float = 1.0, shared_hidden_dim: int = 0, shared_limit: Optional[float] = None, shared_gate: bool = True,
                 score: str = "softmax", weight_on: str = "output", expert_gate: bool = True, activation: str = "gelu",
                 identity: int = 0, correction: bool = False, groups: int = 1, keep: int = 1, route_scale: float = 1.0):
        """limit None: no clamp (with alpha 1 and shift 0 the activation is silu(gate) * up).
        expert_gate False: the experts (and the shared one) have no gate, down(activation(up(x))).
        score "softmax_all": the softmax over all router outputs; the chosen ones' scores divided by their sum, times
        `route_scale`, are the weights.  With it: `correction` (a learned number per output, added to the scores for
        the choice only), `groups` and `keep` (the outputs form equal groups of neighbours, and only those of the `keep`
        groups with the largest best choice score can be chosen), and `identity`: the router's last `identity`
        outputs are experts without tensors, whose output is their input."""
        super().__init__()
        if score not in ops.ROUTE_SCORES and score != "softmax_all":
            raise ValueError(f"score {score!r} is not one of {sorted(ops.ROUTE_SCORES) + ['softmax_all']}")
        if weight_on not in ("output", "input"):
            raise ValueError(f"weight_on {weight_on!r} is not 'output' or 'input'")
        self.score, self.weight_on = score, weight_on
        limit = float("inf") if limit is None else limit
        self.identity = int(identity)
        self.outputs = int(experts) + self.identity  # what the router chooses from
        if not 0 < top <= self.outputs:
            raise ValueError(f"every token uses {top} of {self.outputs} experts: that must be at least one and at most all")
        if score != "softmax_all" and (self.identity or correction or groups != 1 or keep != 1 or route_scale != 1.0):
            raise ValueError("identity experts, a correction, groups and a scale go with the score 'softmax_all'")
        if self.identity and weight_on != "output":
            raise ValueError("identity experts are weighted on their output")
        if groups < 1 or self.outputs % groups or not 1 <= keep <= groups or keep * (self.outputs // groups) < top:
            raise ValueError(f"{groups} groups over {self.outputs} router outputs with {keep} kept cannot give {top} choices")
        activation = str(activation).lower()
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.width, self.experts, self.top, self.hidden_dim = width, int(experts), int(top), int(hidden_dim)
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        self.expert_gate, self.activation = bool(expert_gate), activation
        self.groups, self.keep, self.route_scale, self.has_correction = int(groups), int(keep), float(route_scale), bool(correction)
        self.shared_hidden_dim = int(shared_hidden_dim)
        self.shared_limit = float(shared_limit if shared_limit is not None else limit)
        self.has_shared_gate = bool(shared_gate) and self.shared_hidden_dim > 0
        # the router's rows, and behind them the row of the shared expert's gate: one product, float32 logits
        self.router = self.add_child("router", Linear(width, self.outputs + (1 if self.has_shared_gate else 0)))
        if self.has_correction:
            self.declare("correction", (self.outputs,), init="zeros", kind="scale")
        if self.experts:
            if self.expert_gate:
                self.declare("experts.gate", (self.experts, self.hidden_dim, width))
            self.declare("experts.up", (self.experts, self.hidden_dim, width))
            self.declare("experts.down", (self.experts, width, self.hidden_dim))
        if self.shared_hidden_dim:
            if self.expert_gate:
                self.shared_gate_up = self.add_child("shared.gate_up", Linear(width, 2 * self.shared_hidden_dim))
            else:
                self.shared_up = self.add_child("shared.up", Linear(width, self.shared_hidden_dim))
            self.shared_down = self.add_child("shared.down", Linear(self.shared_hidden_dim, width))
        self._correction = None

    def finalize(self, device, dtype) -> None:
        if self.has_correction:
            self._correction = self.w["correction"].to(torch.float32).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = self.router.forward(x, out_dtype=torch.float32)
        if self.score == "softmax_all":
            ids, weights = ops.moe_route_grouped(logits, self.outputs, self.top, self._correction, self.groups, self.keep, self.route_scale)
        else:
            ids, weights = ops.moe_route(logits, self.experts, self.top, self.score)
        on_input = self.weight_on == "input"
        if self.experts:
            y = ops.moe_experts(x, ids, self.w["experts.gate"] if self.expert_gate else None, self.w["experts.up"], self.w["experts.down"],
                                self.limit, self.alpha, self.shift, in_scale=weights if on_input else None, activation=self.activation)
        else:  # identity experts only: no row of y is ever read
            y = torch.empty(x.shape[0] * self.top, self.width, dtype=torch.float32, device=x.device)
        shared = gate = None
        if self.shared_hidden_dim:
            if self.expert_gate:
                hidden = ops.clamped_gated_act(self.shared_gate_up.forward(x), self.shared_limit, self.alpha, self.shift)
            else:
                hidden = ops.activation(self.shared_up.forward(x), self.activation)
            shared = self.shared_down.forward(hidden)
            if self.has_shared_gate:
                gate = logits[:, self.outputs]
        if self.identity:
            return ops.moe_combine(y, weights, shared, gate, x.dtype, top=self.top, ids=ids, n_experts=self.experts,
                                   x_in=x if x.is_contiguous() else x.contiguous())
        return ops.moe_combine(y, None if on_input else weights, shared, gate, x.dtype, top=self.top)


register_part("feed_forward", "mlp", MLP)
register_part("feed_forward", "experts", ExpertsFeedForward)
