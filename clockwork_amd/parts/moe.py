"""A routed feed-forward: every token through ``top_k`` of ``num_experts`` small gated
feed-forwards (``RoutedExpertsSpec``).

Steps, all on the device, so a step replays as a captured graph: the router's product in float32
with the choice of the top_k experts (one kernel); the (token, choice) pairs sorted by expert
into rows, every expert's rows in tiles of their own (one kernel); the experts' gate and up
products with the activation over those tiles; their down products, scattered back to the pairs
(bfloat16 on the matrix cores: tiles of 16 rows that stream an expert's matrix for steps of few
tokens, tiles of 128 rows through LDS for portions; float32 in plain arithmetic);
the sum over a token's pairs in float32 (not needed when top_k is 1). The experts' matrices are
stacked: gate_up [experts, 2 * ff, hidden] (an expert's gate rows, then its up rows) and down
[experts, hidden, ff]. Cache manager and scheduler are not involved.

Options of the spec: a correction per expert that joins the scores for the choice only; experts
in runs of which only the best can be chosen (both inside the router's kernel); a shared expert
that every token uses (the dense gated products) whose output, times a logistic gate of the same
input (one more row of the router's product), joins in the kernel that sums a token's pairs.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import RoutedExpertsSpec


class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, spec: RoutedExpertsSpec) -> None:
        self.spec = spec

    def param_specs(self):
        s = self.spec
        specs = {
            # the router's rows, then (with a gated shared expert) the row of that gate
            "router_weight": ParamSpec((s.num_experts + (1 if s.shared_gate else 0), s.hidden_size), init=("normal", 0.5)),
            "gate_up_weight": ParamSpec((s.num_experts * 2 * s.intermediate_size, s.hidden_size)),
            "down_weight": ParamSpec((s.num_experts * s.hidden_size, s.intermediate_size)),
        }
        if s.choice_correction:
            specs["correction"] = ParamSpec((s.num_experts,), precision="float32", init=("normal", 0.1))
        if s.shared_intermediate is not None:
            specs["shared_gate_up_weight"] = ParamSpec((2 * s.shared_intermediate, s.hidden_size))
            specs["shared_down_weight"] = ParamSpec((s.hidden_size, s.shared_intermediate))
        return specs

    def kernel_libraries(self) -> list:
        s = self.spec
        # long portions of experts wide enough run through the dense products' wide-tile kernel
        grouped = ops.moe_grouped_ok(s.hidden_size, s.intermediate_size)
        return [("moe", None)] + ([("gemm_tile", None)] if grouped else [])

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        self.router = params["router_weight"]
        self.gate_up = params["gate_up_weight"].view(s.num_experts, 2 * s.intermediate_size, s.hidden_size)
        self.down = params["down_weight"].view(s.num_experts, s.hidden_size, s.intermediate_size)
        self.correction = params.get("correction")
        self.shared_gate_up, self.shared_down = params.get("shared_gate_up_weight"), params.get("shared_down_weight")
        self.kernel = None   # a kernel's name: that one for every step (tests); None: chosen by the step's shape

    def route(self, x: torch.Tensor):
        """(choice int32 [T, top_k], score float32 [T, top_k]), and with a gated shared expert
        its gate, float32 [T, 1], as a third."""
        s = self.spec
        return ops.moe_route(x, self.router, s.top_k, s.router, s.renormalize, correction=self.correction, groups=s.groups,
                             extra=1 if s.shared_gate else 0, renorm_eps=s.renorm_eps)

    def forward(self, x, ctx) -> torch.Tensor:
        s = self.spec
        T = x.shape[0]
        choice, score, *gate = self.route(x)
        if s.shared_intermediate is not None:
            policy = getattr(ctx, "products", None)
            shared = ops.linear(ops.linear_swiglu(x, self.shared_gate_up, policy=policy), self.shared_down, policy=policy)
            return self._routed(x, choice, score, shared, gate[0] if gate else None)
        return self._routed(x, choice, score, None, None)

    def _routed(self, x, choice, score, shared, shared_gate) -> torch.Tensor:
        s = self.spec
        T = x.shape[0]
        kernel = self.kernel or ops.moe_kernel_for(x.dtype, T * s.top_k, s.num_experts, s.hidden_size, s.intermediate_size)
        plan = ops.moe_plan(choice, s.num_experts, kernel)
        inner = ops.moe_gate_up(x, self.gate_up, plan, score, s.top_k, scale_input=s.weight_on == "input")
        out = torch.empty((T, s.hidden_size), dtype=x.dtype, device=x.device)
        if s.top_k == 1 and shared is None:
            return ops.moe_down(inner, self.down, plan, score, 1, s.weight_on == "output", out)
        y = torch.empty((T * s.top_k, s.hidden_size), dtype=x.dtype, device=x.device)
        ops.moe_down(inner, self.down, plan, score, s.top_k, s.weight_on == "output", y)
        return ops.moe_combine(y, s.top_k, out, always=shared, always_gate=shared_gate)
