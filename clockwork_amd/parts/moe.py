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
        return {
            "router_weight": ParamSpec((s.num_experts, s.hidden_size), init=("normal", 0.5)),
            "gate_up_weight": ParamSpec((s.num_experts * 2 * s.intermediate_size, s.hidden_size)),
            "down_weight": ParamSpec((s.num_experts * s.hidden_size, s.intermediate_size)),
        }

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
        self.kernel = None   # a kernel's name: that one for every step (tests); None: chosen by the step's shape

    def route(self, x: torch.Tensor):
        """(choice int32 [T, top_k], score float32 [T, top_k])."""
        s = self.spec
        return ops.moe_route(x, self.router, s.top_k, s.router, s.renormalize)

    def forward(self, x, ctx) -> torch.Tensor:
        s = self.spec
        T = x.shape[0]
        choice, score = self.route(x)
        kernel = self.kernel or ops.moe_kernel_for(x.dtype, T * s.top_k, s.num_experts, s.hidden_size, s.intermediate_size)
        plan = ops.moe_plan(choice, s.num_experts, kernel)
        inner = ops.moe_gate_up(x, self.gate_up, plan, score, s.top_k, scale_input=s.weight_on == "input")
        out = torch.empty((T, s.hidden_size), dtype=x.dtype, device=x.device)
        if s.top_k == 1:
            return ops.moe_down(inner, self.down, plan, score, 1, s.weight_on == "output", out)
        y = torch.empty((T * s.top_k, s.hidden_size), dtype=x.dtype, device=x.device)
        ops.moe_down(inner, self.down, plan, score, s.top_k, s.weight_on == "output", y)
        return ops.moe_combine(y, s.top_k, out)
