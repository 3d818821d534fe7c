"""Feed-forward of experts that a router chooses.

Scores s = sigmoid(W_r h), computed in float32; a token runs the ``top`` experts with the largest scores, each a gated
feed-forward y_e(x) = Wd_e (silu(Wg_e x) * (Wu_e x)) without biases. Options: ``scores`` "softmax" (over all experts);
``groups`` / ``keep_groups``: the experts form equal groups of neighbours, a group's score is its best expert's, and
only experts of the best ``keep_groups`` groups can be chosen; ``gated`` False: experts of one matrix in,
y_e(x) = Wd_e relu(Wu_e x)^2; ``weight_on`` "output": a weight multiplies what its expert returns. The weights are the chosen scores (divided by
their sum with ``renormalize``). A weight multiplies what its expert is given, not what it returns: the layer's
result is sum_e y_e(s_e h). An expert that every token runs (``shared``) is added, multiplied by sigmoid(w_sg . h), one
number a token, where ``shared_gate`` names that vector.

The router's product (with the shared expert's gate as one more row) is one float32 product; the choice is made on
the device (csrc/moe.hip: lmsf_moe_route), so that a step needs nothing from the host and replays from a graph; the
experts run in the kernels that also serve experts assigned by a table (parts/table_moe.py), the router's choice
standing for the table's rows. The reference has dense feed-forwards only
(core/src/model_executor/models/llama/llama.rs:223-274).
"""
from typing import Callable, Dict, Optional

import torch

from .base import FeedForward, PartSpec, Runtime, TensorDecl, build_part, register_part
from .linear import FusedLinear


@register_part("feed_forward", "routed_moe")
class RoutedMoE(FeedForward):
    graph_safe = True
    recordable = False

    def __init__(self, prefix: str, rt: Runtime, hidden_size: int, expert_size: int, num_experts: int, top: int,
                 shared: Optional[PartSpec] = None, shared_gate: Optional[str] = None,
                 renormalize: bool = False, router_name: str = "router", expert_prefix: str = "e",
                 gate_name: str = "gate", up_name: str = "up", down_name: str = "down", gated: bool = True,
                 scores: str = "sigmoid", groups: int = 1, keep_groups: int = 1, weight_on: str = "input"):
        super().__init__(prefix, rt)
        self.gated, self.scores, self.weight_on = bool(gated), str(scores), str(weight_on)
        self.groups, self.keep_groups = int(groups), int(keep_groups)
        if self.scores not in ("sigmoid", "softmax") or self.weight_on not in ("input", "output"):
            raise ValueError("%s: scores %r (sigmoid, softmax), weight_on %r (input, output)" % (prefix, scores, weight_on))
        if not (0 < self.keep_groups <= self.groups <= 256) or int(num_experts) % self.groups \
                or self.keep_groups * (int(num_experts) // self.groups) < int(top):
            raise ValueError("%s: %d of %d groups of %d experts cannot hold %d choices"
                             % (prefix, keep_groups, groups, num_experts, top))
        # (the router that knows groups and the softmax has no column for a shared expert's gate)
        self.plain_route = self.scores == "sigmoid" and self.groups == 1
        if not self.plain_route and shared_gate is not None:
            raise ValueError("%s: a gated shared expert goes with sigmoid scores and one group" % prefix)
        self.W, self.F, self.E, self.top = int(hidden_size), int(expert_size), int(num_experts), int(top)
        if not (0 < self.top <= self.E) or self.top > 64:
            raise ValueError("%s: %d of %d experts (at most 64 a token)" % (prefix, self.top, self.E))
        self.renormalize = bool(renormalize)
        self.names = [("%s.%s%d" % (prefix, expert_prefix, e), gate_name, up_name, down_name) for e in range(self.E)]
        self.shared = build_part("feed_forward", shared, "%s.%s" % (prefix, shared.params.get("prefix", "shared")), rt) \
            if shared is not None else None
        if shared_gate is not None and self.shared is None:
            raise ValueError("%s: a gate without a shared expert" % prefix)
        sources = [(router_name, self.E)] + ([(shared_gate, 1)] if shared_gate is not None else [])
        self.has_shared_gate = shared_gate is not None
        # the router (and the shared expert's gate) as one product with a float32 result; rows of zeros make them a
        # multiple of eight, which the many-rows form of that product asks for
        self.router = FusedLinear(prefix, rt, self.W, sources, bare_names=True, pad_rows_to=8)
        self.w_gate_up: Optional[torch.Tensor] = None     # [E, 2F, W]
        self.w_down: Optional[torch.Tensor] = None        # [E, W, F]

    def children(self):
        return [self.router] + ([self.shared] if self.shared is not None else [])

    def tensors(self):
        return [t for t in (self.w_gate_up, self.w_down) if t is not None]

    def checkpoint_tensors(self) -> Dict[str, TensorDecl]:
        out = {}
        for p, g, u, d in self.names:
            if self.gated:
                out["%s.%s" % (p, g)] = TensorDecl((self.F, self.W))
            out["%s.%s" % (p, u)] = TensorDecl((self.F, self.W))
            out["%s.%s" % (p, d)] = TensorDecl((self.W, self.F))
        return out

    def load_weights(self, fetch: Callable[[str], torch.Tensor]) -> None:
        gu = torch.empty((self.E, (2 if self.gated else 1) * self.F, self.W), dtype=self.rt.dtype, device=self.rt.device)
        dn = torch.empty((self.E, self.W, self.F), dtype=self.rt.dtype, device=self.rt.device)
        for e, (p, g, u, d) in enumerate(self.names):
            if self.gated:
                gu[e, :self.F].copy_(fetch("%s.%s" % (p, g)))
            gu[e, self.F if self.gated else 0:].copy_(fetch("%s.%s" % (p, u)))
            dn[e].copy_(fetch("%s.%s" % (p, d)))
        self.w_gate_up, self.w_down = gu, dn

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ops = self.rt.ops
        logits = ops.linear_wide(h, self.router.weight, None)                       # float32 [N, >= E (+ 1)]
        if self.plain_route:
            choice, weight, gate = ops.moe_route(logits, self.E, self.top, renorm=self.renormalize,
                                                 extra=self.E if self.has_shared_gate else -1)
        else:
            choice, weight = ops.moe_route_groups(logits, self.E, self.top, softmax=self.scores == "softmax",
                                                  groups=self.groups, keep=self.keep_groups, renorm=self.renormalize)
            gate = None
        base = self.shared.forward(h) if self.shared is not None else None
        if self.gated and self.weight_on == "input":
            return ops.table_moe(h, self.w_gate_up, self.w_down, None, choice, 1.0, base=base, pair_scale=weight,
                                 base_scale=gate)
        on_input = self.weight_on == "input"
        return ops.table_moe(h, self.w_gate_up, self.w_down, None, choice, 1.0, base=base,
                             pair_scale=weight if on_input else None, base_scale=gate,
                             out_scale=None if on_input else weight, gated=self.gated)
