"""Dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)) (clockwork/engine/model.py:52-63).

gate and up are one product over a fused [2 I, H] weight; the gate multiply is one kernel.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import SwiGLUSpec


class SwiGLU(Part):
    graph_safe = True
    def __init__(self, spec: SwiGLUSpec) -> None:
        self.spec = spec

    def param_specs(self):
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return {"gate_up_weight": ParamSpec((2 * I, H)), "down_weight": ParamSpec((H, I))}

    def bind(self, params, device, dtype) -> None:
        self.gate_up = params["gate_up_weight"]
        self.down = params["down_weight"]

    def fuses_input_norm(self, n_tokens: int, dtype, delta) -> bool:
        """True if ``forward`` can take an ``ops.LazyAddNorm`` of that many rows and make the
        norm inside the gate/up product (decode: few rows)."""
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return ops.swiglu_norm_fusable(n_tokens, 2 * I, H, dtype, self.gate_up, delta)

    def forward(self, x, ctx) -> torch.Tensor:
        policy = getattr(ctx, "products", None)
        return ops.linear(ops.linear_swiglu(x, self.gate_up, policy=policy), self.down, partial_ok=True, policy=policy)


class GatedMLP(Part):
    """down(act(gate(x)) * up(x)) with the activation the spec names. "silu" takes the fused
    kernels of :class:`SwiGLU`; "gelu_tanh" runs the gate/up product, one kernel for
    gelu_tanh(gate) * up in float32, and the down product."""

    graph_safe = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return {"gate_up_weight": ParamSpec((2 * I, H)), "down_weight": ParamSpec((H, I))}

    def kernel_libraries(self) -> list:
        return [("rowwise", None)] if self.spec.activation != "silu" else []

    def bind(self, params, device, dtype) -> None:
        self.gate_up = params["gate_up_weight"]
        self.down = params["down_weight"]

    def forward(self, x, ctx) -> torch.Tensor:
        policy = getattr(ctx, "products", None)
        if self.spec.activation == "silu":
            return ops.linear(ops.linear_swiglu(x, self.gate_up, policy=policy), self.down, policy=policy)
        gate_up = ops.linear(x, self.gate_up, policy=policy)
        inner = torch.empty((x.shape[0], self.spec.intermediate_size), dtype=x.dtype, device=x.device)
        return ops.linear(ops.gelu_tanh_mul(gate_up, inner), self.down, policy=policy)


class DenseMLP(Part):
    """down(act(up(x))) (``DenseMLPSpec``). "gelu": the up product with the erf GELU (float32
    inside) in its epilogue for few rows, as a kernel of its own behind the product otherwise;
    "relu2": max(z, 0)^2 on the float32 sums in the epilogue of the up product for few rows
    (the weight-streaming kernel) and for long portions (the wide-tile kernel), in place behind
    the product otherwise; the down product."""

    graph_safe = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return {"up_weight": ParamSpec((I, H)), "down_weight": ParamSpec((H, I))}

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.up = params["up_weight"]
        self.down = params["down_weight"]

    def forward(self, x, ctx) -> torch.Tensor:
        policy = getattr(ctx, "products", None)
        if self.spec.activation == "relu2":
            return ops.linear(ops.linear_relu_squared(x, self.up, policy=policy), self.down, policy=policy)
        return ops.linear(ops.linear_gelu(x, self.up, policy=policy), self.down, policy=policy)
