"""RMSNorm fused with the residual add (clockwork/engine/model.py:38-49, 147-152)."""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import RMSNormSpec


class RMSNorm(Part):
    graph_safe = True
    # takes a delta that is an ops.PendingPair (two branch outputs not yet added to the residual)
    accepts_pending = True
    def __init__(self, spec: RMSNormSpec) -> None:
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.size,), precision="stored", init=("one_plus_uniform", 0.1))}

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.dtype = dtype

    def forward(self, resid: torch.Tensor, delta, rows=None) -> torch.Tensor:
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=resid.device)
        return ops.add_rmsnorm(resid, delta, self.weight, self.spec.eps, out, rows)

    def forward_pair(self, resid: torch.Tensor, delta, other: "RMSNorm"):
        """(this norm, ``other``'s norm) of resid + delta in one kernel: two norms of the same rows
        share the statistics when their eps agree; else two kernels."""
        if other.spec.eps != self.spec.eps or other.spec.size != self.spec.size or other.weight.dtype != self.weight.dtype:
            return self.forward(resid, delta), other.forward(resid, None)
        shape = (resid.shape[0], self.spec.size)
        out = torch.empty(shape, dtype=self.dtype, device=resid.device)
        out2 = torch.empty(shape, dtype=self.dtype, device=resid.device)
        ops.add_rmsnorm(resid, delta, self.weight, self.spec.eps, out, weight2=other.weight, out2=out2)
        return out, out2

    def lazy(self, resid: torch.Tensor, delta) -> "ops.LazyAddNorm":
        """The norm of resid + delta for a consumer that computes it inside its own kernel; the
        residual is not updated, so ``delta`` has to reach the next norm as well."""
        return ops.LazyAddNorm(resid, delta, self.weight, self.spec.eps, self.dtype)


class LayerNorm(Part):
    """LayerNorm with weight and bias, fused with the residual add. The statistics are float32:
    the mean first, then the mean of the squared deviations. What it can add before norming is a
    block's gated branches (``ops.GatedBranches``): the gates' sigmoids are made inside the kernel."""

    graph_safe = True
    accepts_gated = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        specs = {"weight": ParamSpec((self.spec.size,), precision="stored", init=("one_plus_uniform", 0.1))}
        if self.spec.bias:
            specs["bias"] = ParamSpec((self.spec.size,), precision="stored", init=("normal", 0.02))
        return specs

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.bias = params.get("bias")
        if self.bias is not None and self.bias.dtype != self.weight.dtype:
            self.bias = self.bias.to(self.weight.dtype)
        self.dtype = dtype

    def forward(self, resid: torch.Tensor, delta, rows=None) -> torch.Tensor:
        if delta is not None and not isinstance(delta, ops.GatedBranches):
            delta = ops.GatedBranches(None, None, delta if not isinstance(delta, ops.PartialSums) else delta.sum(self.dtype))
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=resid.device)
        return ops.add_layernorm(resid, delta, self.weight, self.bias, self.spec.eps, out, rows)


class DynamicTanh(Part):
    """tanh(alpha * x) * weight + bias (``DynamicTanhSpec``), fused with the residual add: the
    pending branch output joins the float32 stream multiplied by the spec's ``delta_scale``, and
    after it a second float32 stream when the model hands one on (``ops.WithStreamInput``)."""

    graph_safe = True
    accepts_stream_input = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        specs = {"weight": ParamSpec((self.spec.size,), precision="stored", init=("one_plus_uniform", 0.1)),
                 "alpha": ParamSpec((1,), precision="float32", init=("uniform", 0.3, 1.0))}
        if self.spec.bias:
            specs["bias"] = ParamSpec((self.spec.size,), precision="stored", init=("normal", 0.02))
        return specs

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.bias = params.get("bias")
        if self.bias is not None and self.bias.dtype != self.weight.dtype:
            self.bias = self.bias.to(self.weight.dtype)
        self.alpha = params["alpha"].reshape(1)
        self.dtype = dtype

    def forward(self, resid: torch.Tensor, delta, rows=None) -> torch.Tensor:
        extra = None
        if isinstance(delta, ops.WithStreamInput):
            delta, extra = delta.delta, delta.extra
        if isinstance(delta, ops.PartialSums):
            delta = delta.sum(self.dtype)
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=resid.device)
        return ops.add_dynamic_tanh(resid, delta, self.spec.delta_scale, extra, self.weight, self.bias, self.alpha, out, rows)


class BranchRMSNorm(Part):
    """RMS norm with a weight kept as a distance from a constant (``BranchRMSNormSpec``), float32
    throughout. ``join(resid, branch, image)`` norms a sublayer's output, adds it to the stream
    multiplied by the spec's ``branch_scale`` and leaves the stream's image in the activation type,
    all in one kernel; ``forward(resid, delta, rows)`` is the norm of the stream itself (a final
    norm): nothing may be pending then but an ``ops.StreamImage``, which says so."""

    graph_safe = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.size,), precision="stored", init=("normal", 0.1))}

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.dtype = dtype

    def image(self, resid: torch.Tensor) -> torch.Tensor:
        """The stream in the activation type (the stream itself where that is float32)."""
        if self.dtype == torch.float32:
            return resid
        return ops.branch_norm_add(resid, None, None, 0.0, self.spec.eps, 0.0, torch.empty(tuple(resid.shape), dtype=self.dtype, device=resid.device))

    def join(self, resid: torch.Tensor, branch) -> torch.Tensor:
        """resid += branch_scale * N(branch); returns the stream's image in the activation type."""
        s = self.spec
        if isinstance(branch, ops.PartialSums):
            branch = branch.sum(self.dtype)
        image = None if self.dtype == torch.float32 else torch.empty(tuple(resid.shape), dtype=self.dtype, device=resid.device)
        ops.branch_norm_add(resid, branch, self.weight, s.weight_offset, s.eps, s.branch_scale, image)
        return resid if image is None else image

    def forward(self, resid: torch.Tensor, delta, rows=None) -> torch.Tensor:
        if delta is not None and not isinstance(delta, ops.StreamImage):
            raise TypeError("this norm reads the stream as it stands: a pending branch output must have joined it before")
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=resid.device)
        return ops.stream_norm(resid, self.weight, self.spec.weight_offset, self.spec.eps, out, rows)
