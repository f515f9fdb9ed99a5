"""Python face of the HIP libraries: shape and type checks on the host, then one C call.

Every function takes torch tensors that live on the GPU, checks what the kernel
and its grid assume (so a wrong shape is an exception here, never an
out-of-bounds access there) and launches on torch's current stream. There is no
other implementation behind these functions: if a library cannot be built or
loaded the call raises.
"""

from __future__ import annotations

import contextlib
import ctypes
import gc
import hashlib
import json
import os
import tempfile
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from clockwork_amd.csrc import build

F32, BF16 = 0, 1
_ERRORS = {
    -1: "an argument the kernel does not take",
    -2: "an element type the kernel is not built for",
    -3: "the HIP runtime refused the launch",
    -4: "a size beyond the kernel's stated maximum",
}


class KernelError(RuntimeError):
    pass


def _check(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what}: {_ERRORS.get(code, f'error {code}')}")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"the kernels take float32 and bfloat16 tensors, not {dtype}")


_libs: dict = {}


def _load(name: str, head_dim: int | None = None) -> ctypes.CDLL:
    key = (name, head_dim)
    lib = _libs.get(key)
    if lib is None:
        path = build.ensure_built(name, head_dim)
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelError(f"cannot load the HIP library {path}: {e}") from e
        _declare(name, lib)
        _libs[key] = lib
    return lib


def preload(libraries=(), tiled_products: bool = False, sampling: bool = False) -> None:
    """Build (side by side, if several are missing) and load what a model runs: the common
    kernels, the products and the ``libraries`` its parts name, as (name, head size or None)
    pairs, e.g. ("attention", 128); the tiled products (a bfloat16 model's gate/up product of a
    long portion, and every large product with ``hip_products``) and the sampling kernels only for
    a caller that uses them."""
    jobs = [("core", None), ("gemm", None)]
    if tiled_products:
        jobs.append(("gemm_tile", None))
    if sampling:
        jobs.append(("sampling", None))
    for name, head_dim in libraries:
        job = (str(name), None if head_dim is None else int(head_dim))
        if job not in jobs:
            jobs.append(job)
    build.ensure_many(jobs)
    for name, hd in jobs:
        _load(name, hd)


def loaded_libraries() -> list[str]:
    return sorted(str(lib._name) for lib in _libs.values())


def _declare(name: str, lib: ctypes.CDLL) -> None:
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sigs = {
        "core": {
            "cw_embedding": [P, I, P, P, I, I, I, P],
            "cw_add_rmsnorm": [P, P, P, I, I, P, I, F, P, I, P, I, I, P, P, P],
            "cw_rope_kv_write": [P, I, P, I, P, P, P, I, I, I, I, I, P, P, L, P],
            "cw_silu_mul": [P, P, I, I, I, P],
            "cw_copy_pages": [P, I, L, L, P, I, P],
            "cw_fresh_state_rows": [P, I, I, I, I, L, P, P, I, P],
            "cw_bf16_to_f32": [P, P, L, P],
        },
        "gemm": {
            "cw_gemm_f32": [P, L, P, P, P, L, I, I, I, P, L, P],
            "cw_gemm_f32_workspace_floats": [I, I, I],
            "cw_gemm_bf16_skinny": [I, P, L, P, P, L, I, I, I, I, P],
            "cw_gemm_bf16_skinny_ksplits": [I, I, I],
            "cw_gemm_bf16_skinny_fast": [I, I, I, I],
            "cw_gemm_bf16_swiglu_normed_ok": [I, I, I],
            "cw_gemm_bf16_swiglu_normed": [P, P, P, I, F, P, P, L, I, I, I, P],
            "cw_gemm_qkv_rope_bf16": [P, L, P, P, I, P, P, P, P, P, P, L, I, I, I, I, I, P],
        },
        "gemm_tile": {
            "cw_gemm_bf16_tiled": [I, P, L, P, P, I, P, L, I, I, I, P],
            "cw_gemm_bf16_wide_tiles": [I, I, I, I, L],
            "cw_gemm_bf16_wide": [I, P, L, P, P, I, P, L, I, I, I, I, P],
            "cw_gemm_bf16_wide_partial_ok": [I, I, I, L, I],
            "cw_gemm_bf16_wide_partial": [P, L, P, P, L, I, I, I, I, I, P],
            "cw_gemm_bf16_wide_grouped": [I, P, L, P, L, P, L, I, I, P, P, I, P, P, I, P],
        },
        "rowwise": {
            "cw_embedding_pos": [P, I, P, P, P, F, P, I, I, I, I, P],
            "cw_add_layernorm": [P, P, P, I, P, P, I, P, P, I, F, P, I, P, I, I, P],
            "cw_gated_residual_add": [P, P, P, I, P, P, I, I, I, I, P],
            "cw_gelu_tanh_mul": [P, P, I, I, I, P],
            "cw_softcap": [P, L, F, P],
            "cw_rms_mean2": [P, P, P, P, I, F, P, I, I, I, P],
            "cw_qk_rownorm_store": [P, I, L, I, I, I, I, I, I, P, P, I, F, P, P, P, L, I, P],
            "cw_add_dyt": [P, P, I, F, P, P, P, I, P, P, I, P, I, I, P],
            "cw_gelu_erf": [P, I, L, P],
            "cw_sigmoid_mul": [P, P, I, L, I, I, I, I, P],
            "cw_bias_store": [P, I, L, I, I, I, I, I, I, P, I, P, P, P, L, I, P],
            "cw_latent_store": [P, I, L, I, I, I, I, I, I, P, P, I, F, P, P, P, P, P, L, I, P],
            "cw_rotate_part": [P, I, L, L, I, P, L, L, I, I, I, I, P, P, I, P],
            "cw_branch_norm_add": [P, P, P, I, F, F, F, P, I, I, I, P],
            "cw_stream_norm": [P, P, I, F, F, P, I, P, I, I, P],
            "cw_headnorm_rope_store": [P, I, L, I, I, I, I, I, I, I, P, I, P, P, I, F, P, P, I, P, P, P, I, L, I, I, I, F, I, P],
            "cw_tanh": [P, I, L, P],
            "cw_shift_mix": [P, I, P, I, I, P, L, L, I, P, P, P, I, P, L, I, P],
            "cw_stream_beside_input": [P, P, P, P, P, I, I, I, I, I, P],
            "cw_relu_squared": [P, I, L, P],
            "cw_scale": [P, L, F, P],
        },
        "moe": {
            "cw_moe_tile_rows": [I],
            "cw_moe_max_tiles": [I, I, I],
            "cw_moe_route": [P, P, I, I, I, I, I, I, I, P, P, P, I, I, I, I, P, F, P],
            "cw_moe_plan": [P, I, I, I, P, I, P, I, P, P],
            "cw_moe_expert_product": [I, I, P, P, P, I, P, P, P, I, P, I, I, I, I, P],
            "cw_moe_gather": [P, P, I, P, P, I, I, P, I, I, I, P],
            "cw_moe_combine": [P, P, I, I, I, I, P, P, I, P],
        },
        "rows_attention": {
            "cw_rows_attention_key_chunk": [I, I, I, I],
            "cw_rows_attention_heads_per_group": [I, I, I],
            "cw_rows_attention_tokens_per_item": [I, I, I],
            "cw_rows_mfma_supported": [I, I, I, I],
            "cw_rows_mfma_grid_y": [I, I, I, I, I, I],
            "cw_rows_mfma_workspace_floats": [I, I, I, I, I, I, I, I],
            "cw_rows_attention_mfma": [P, L, L, P, L, L, P, P, I, I, L, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, I, F, I, F, F,
                                       I, P, L, I, F, P, L, I, P],
            "cw_rows_attention": [I, P, L, L, P, L, L, P, P, I, I, L, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, I, F, I, F, F,
                                  I, F, P, L, I, P],
        },
        "sink_attention": {
            "cw_sink_attention_max_bq": [I, I, I, I],
            "cw_sink_attention": [I, P, L, P, P, P, L, P, I, P, P, P, I, I, P, P, P, P, I, I, I, I, I, I, F, P],
            "cw_sink_decode_workspace_floats": [I, I, I, I, I],
            "cw_sink_prefill_mfma_supported": [I, I, I, I],
            "cw_sink_prefill_mfma": [P, L, P, P, P, L, P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, I, F, I, P],
            "cw_sink_decode_supported": [I, I, I, I],
            "cw_sink_decode": [I, P, L, P, P, P, L, P, I, P, P, I, I, I, P, P, P, P, P, I, I, I, I, I, I, F, P],
        },
        "linear_recurrence": {
            "cw_linear_recurrence_supported": [I, I],
            "cw_linear_recurrence": [I, P, L, I, I, I, I, I, P, P, P, P, I, P, P, P, I, I, I, I, I, F, F, F, I, P, I, P, L, L, P],
            "cw_linear_recurrence_segments_supported": [I, I],
            "cw_linear_recurrence_segments_workspace_floats": [I, I, I, I, I],
            "cw_linear_recurrence_segments": [I, P, L, I, I, I, I, I, P, P, P, P, I, P, P, P, I, I, P, P, P, I, I, I, I, I, I,
                                              F, F, F, I, P, I, P, L, L, P],
        },
        "sampling": {
            "cw_argmax_chunks": [I],
            "cw_argmax": [P, L, I, I, P, P, L, P],
            "cw_argmax_static_init": [],
            "cw_argmax_static": [P, L, I, I, P, P],
            "cw_sample": [P, L, I, I, P, P, P, P, P, P, P, L, I, P],
            "cw_sample_workspace_bytes": [I, I],
        },
        "attention": {
            "cw_attention_head_dim": [],
            "cw_attention_workspace_floats": [I, I, I, I, I],
            "cw_attention": [I, I, P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, P, L, P],
            "cw_attention_prefill_supported": [],
            "cw_attention_prefill_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, P, I, I, P, L, F, P],
            "cw_attention_prefill_workspace_floats": [I, I, I, I],
            "cw_attention_prefill_row_blocks_ok": [I],
            "cw_attention_decode_supported": [],
            "cw_attention_decode_gh": [I],
            "cw_attention_decode_max_splits": [],
            "cw_attention_decode_workspace_floats": [I, I, I, I],
            "cw_attention_decode_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, F, P, L, P, I, I, I, F, P],
        },
    }[name]
    for fn, argtypes in sigs.items():
        f = getattr(lib, fn)
        f.argtypes = argtypes
        f.restype = c_int64 if fn.endswith(("workspace_floats", "workspace_bytes")) else c_int


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (also the capture stream inside a graph capture). Asked
    for at every launch, so through torch's raw accessor where there is one: a tenth of the cost
    of building a Stream object."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise KernelError("kernel arguments must live on the GPU and be contiguous")


def _i32(t, n: int | None, what: str) -> None:
    if not (t.dtype == torch.int32 and t.dim() == 1):
        raise KernelError(f"{what} must be a 1-d int32 tensor")
    if n is not None:
        if not (t.numel() >= n):
            raise KernelError(f"{what} holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------------------------
def embedding(table: torch.Tensor, ids: torch.Tensor, out_resid: torch.Tensor) -> torch.Tensor:
    """out_resid[t] = float32(table[ids[t]]); out_resid is [T, H] float32."""
    _gpu(table, ids, out_resid)
    T = ids.numel()
    V, H = table.shape
    _i32(ids, T, "ids")
    if not (out_resid.dtype == torch.float32 and tuple(out_resid.shape) == (T, H)):
        raise KernelError("residual must be [T, H] float32")
    _check(
        _load("core").cw_embedding(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out_resid), T, H, V, _stream()),
        "embedding",
    )
    return out_resid


class PartialSums:
    """A product whose K loop was split over workgroups: ``parts`` is float32 [splits, M, N] and the
    value is their sum, taken in order by whoever reads it next (``add_rmsnorm`` does)."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor) -> None:
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def sum(self, dtype=None) -> torch.Tensor:
        total = self.parts[0].clone()
        for i in range(1, self.parts.shape[0]):
            total += self.parts[i]
        return total if dtype is None else total.to(dtype)


_row_indices: dict = {}


def _all_rows(n: int, device) -> torch.Tensor:
    """int32 [0, n) on ``device`` (kept: a HIP graph may hold its address)."""
    t = _row_indices.get((n, device))
    if t is None:
        t = _row_indices[(n, device)] = torch.arange(n, dtype=torch.int32, device=device)
    return t


class PendingPair:
    """Two branch outputs that are both still to be added to the residual stream, ``first``
    before ``second``: what a block hands on when its second norm ran inside the feed-forward's
    product kernel (which writes no residual). ``first`` is a tensor in the activation type,
    ``second`` a tensor or :class:`PartialSums`."""

    __slots__ = ("first", "second")

    def __init__(self, first, second) -> None:
        self.first = first
        self.second = second


class LazyAddNorm:
    """rmsnorm(resid + delta) * weight, not computed yet: a consumer that can make it inside its
    own kernel takes the pieces, any other calls :meth:`value`. The residual is not updated
    either way: ``delta`` stays pending."""

    __slots__ = ("resid", "delta", "weight", "eps", "dtype")

    def __init__(self, resid, delta, weight, eps: float, dtype) -> None:
        self.resid, self.delta, self.weight, self.eps, self.dtype = resid, delta, weight, eps, dtype

    @property
    def shape(self):
        return self.resid.shape

    def value(self) -> torch.Tensor:
        out = torch.empty(tuple(self.resid.shape), dtype=self.dtype, device=self.resid.device)
        return add_rmsnorm(self.resid, self.delta, self.weight, self.eps, out, write_back=False)


def add_rmsnorm(resid, delta, weight, eps: float, out, rows=None, write_back: bool = True, weight2=None, out2=None) -> torch.Tensor:
    """resid += delta (when given), out = rmsnorm(resid) * weight; with ``rows`` only those rows
    are normed into out[i] and resid is left alone, as it is with ``write_back`` off. resid
    float32 [T, H]; delta/out in the activation type, or delta a :class:`PartialSums` of that
    shape, or a :class:`PendingPair` (both are added, ``first`` first). ``weight2`` / ``out2``: a
    second norm of the same rows with weights of its own (the same eps, so the same statistics),
    written beside the first by the same kernel."""
    delta0 = None
    if isinstance(delta, PendingPair):
        delta0, delta = delta.first, delta.second
    if not write_back and rows is None:
        rows = _all_rows(resid.shape[0], resid.device)
    parts = 0
    if isinstance(delta, PartialSums):
        parts = delta.parts.shape[0]
        delta = delta.parts
    _gpu(resid, delta, delta0, weight, out, rows)
    T, H = resid.shape
    if not (resid.dtype == torch.float32):
        raise KernelError("the residual stream is float32")
    if delta0 is not None:
        if not (tuple(delta0.shape) == (T, H) and delta0.dtype == out.dtype):
            raise KernelError("the first pending delta must be [T, H] in the activation type")
    n = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "rows")
    if not (tuple(out.shape) == (n, H)):
        raise KernelError(f"out must be [{n}, {H}]")
    if not (weight.numel() == H):
        raise KernelError("norm weight has the wrong size")
    if (weight2 is None) != (out2 is None):
        raise KernelError("a second norm needs its weights and its output")
    if weight2 is not None:
        _gpu(weight2, out2)
        if not (weight2.numel() == H and weight2.dtype == weight.dtype and tuple(out2.shape) == (n, H) and out2.dtype == out.dtype):
            raise KernelError("the second norm's weights and output must match the first's")
    if parts:
        if not (tuple(delta.shape) == (parts, T, H) and delta.dtype == torch.float32):
            raise KernelError("partial sums must be float32 [parts, T, H]")
    elif delta is not None:
        if not (tuple(delta.shape) == (T, H) and delta.dtype == out.dtype):
            raise KernelError("delta must be [T, H] in the activation type")
    _check(
        _load("core").cw_add_rmsnorm(
            _ptr(resid), _ptr(delta0), _ptr(delta), parts, T, _ptr(weight), dtype_code(weight.dtype), float(eps), _ptr(out),
            dtype_code(out.dtype), _ptr(rows), n, H, _ptr(weight2), _ptr(out2), _stream()),
        "add_rmsnorm",
    )
    return out


def rope_kv_write(qkv, bias, positions, slots, inv_freq, rotary_dim: int, nh: int, nkv: int, hd: int,
                  k_cache, v_cache) -> None:
    """Add the bias, rotate q (in place) and k, write k and v rows to the cache at ``slots``.

    qkv [T, (nh + 2 nkv) hd]; k_cache/v_cache [rows, nkv, hd] flat over pages; slots int32 [T]
    (None: nothing is cached, for a mixer that reads another's cache: then nkv must be 0)."""
    _gpu(qkv, bias, positions, slots, inv_freq, k_cache, v_cache)
    T = qkv.shape[0]
    width = (nh + 2 * nkv) * hd
    if not (qkv.dim() == 2 and qkv.shape[1] == width):
        raise KernelError(f"qkv must be [T, {width}]")
    _i32(positions, T, "positions")
    cache_rows = 0
    if slots is not None:
        _i32(slots, T, "slots")
        if not (k_cache is not None and v_cache is not None):
            raise KernelError("slots without a cache")
        if not (k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype):
            raise KernelError("cache and activations differ in type")
        if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
            raise KernelError("cache must be [..., nkv, hd]")
        cache_rows = k_cache.numel() // (nkv * hd)
    else:
        if not (nkv == 0):
            raise KernelError("keys and values need slots to be written to")
    if bias is not None:
        if not (bias.numel() == width):
            raise KernelError("qkv bias has the wrong size")
    if inv_freq is not None:
        if not (inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2):
            raise KernelError("inv_freq must be float32 [rotary_dim / 2]")
    else:
        rotary_dim = 0
    _check(
        _load("core").cw_rope_kv_write(
            _ptr(qkv), dtype_code(qkv.dtype), _ptr(bias), dtype_code(bias.dtype) if bias is not None else 0,
            _ptr(positions), _ptr(slots), _ptr(inv_freq), int(rotary_dim), T, nh, nkv, hd,
            _ptr(k_cache), _ptr(v_cache), cache_rows, _stream()),
        "rope_kv_write",
    )


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _gpu(gate_up, out)
    T, two_i = gate_up.shape
    if not (two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and out.dtype == gate_up.dtype):
        raise KernelError("silu_mul shapes")
    _check(_load("core").cw_silu_mul(_ptr(gate_up), _ptr(out), dtype_code(out.dtype), T, two_i // 2, _stream()), "silu_mul")
    return out


def copy_pages(pool: torch.Tensor, pairs: torch.Tensor) -> None:
    """pool [planes, num_blocks, ...]: for each (src, dst) row of ``pairs`` copy page src to dst in every plane."""
    _gpu(pool, pairs)
    planes, num_blocks = pool.shape[0], pool.shape[1]
    block_bytes = pool[0, 0].numel() * pool.element_size()
    if not (pairs.dtype == torch.int32 and pairs.dim() == 2 and pairs.shape[1] == 2):
        raise KernelError("pairs must be int32 [n, 2]")
    _check(_load("core").cw_copy_pages(_ptr(pool), planes, num_blocks, block_bytes, _ptr(pairs), pairs.shape[0], _stream()), "copy_pages")


def fresh_state_rows(pool: torch.Tensor, slots: torch.Tensor, starts: torch.Tensor, n: int) -> None:
    """pool [entries, slots, ...], its last slot the template of a fresh state: for each of the
    first ``n`` requests of a step that starts at position 0 (``starts[r] == 0``), set row
    ``slots[r]`` to the template in every entry; a slot outside [0, slots - 1) writes nothing. A
    kernel, so a captured step may hold it."""
    _gpu(pool, slots, starts)
    _i32(slots, n, "slots")
    _i32(starts, n, "starts")
    if pool.dim() < 2 or pool.shape[1] < 2:
        raise KernelError("a state pool is [entries, slots, ...] with the template as its last slot")
    row_bytes = (pool[0, 0].numel() if pool.dim() > 2 else 1) * pool.element_size()
    pool_slots = pool.shape[1]
    _check(_load("core").cw_fresh_state_rows(_ptr(pool), pool.shape[0], pool_slots, pool_slots - 1, pool_slots - 1,
                                             row_bytes, _ptr(slots), _ptr(starts), int(n), _stream()), "fresh_state_rows")


def linear(x: torch.Tensor, weight: torch.Tensor, bias=None, out_dtype=None, partial_ok: bool = False,
           policy: "ProductPolicy | None" = None):
    """y = x @ weight.T (+ bias). float32: the true-float32 HIP product. bfloat16: few rows go
    through the weight-streaming kernel, many through the library product (as the reference's
    engine uses one) or, where ``policy`` (the calling engine's :class:`ProductPolicy`) says so,
    through this package's tiled kernels; float32 accumulation either way. With ``partial_ok``
    the result may come back as :class:`PartialSums` (a narrow output with a long K, few rows):
    only for a result that goes straight into ``add_rmsnorm``."""
    policy = policy if policy is not None else DEFAULT_POLICY
    _gpu(x, weight, bias)
    M, K = x.shape
    N = weight.shape[0]
    if not (weight.shape[1] == K):
        raise KernelError(f"weight is {tuple(weight.shape)}, input has {K} columns")
    if x.dtype == torch.float32:
        if not (weight.dtype == torch.float32):
            raise KernelError("a float32 product needs float32 weights")
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
        if bias is not None:
            if not (bias.dtype == torch.float32 and bias.numel() == N):
                raise KernelError("bias must be float32 [N]")
        lib = _load("gemm")
        # a narrow output with a long K is summed in parts over K (the same parts whatever M is)
        need = lib.cw_gemm_f32_workspace_floats(M, N, K)
        parts = torch.empty(need, dtype=torch.float32, device=x.device) if need else None
        _check(lib.cw_gemm_f32(_ptr(x), K, _ptr(weight), _ptr(bias), _ptr(out), N, M, N, K, _ptr(parts), need, _stream()),
               "gemm_f32")
        return out
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        raise KernelError("a bfloat16 product needs bfloat16 operands")
    if M <= STREAM_MAX_ROWS and K % 8 == 0 and bias is None:
        lib = _load("gemm")
        if partial_ok and out_dtype is None:
            splits = lib.cw_gemm_bf16_skinny_ksplits(M, N, K)
            chosen = 0
            if splits > 1 and M <= SKINNY_MAX_ROWS:
                # a tuning start-up has timed the split counts for this shape, or does so now
                if policy.tuning and (N, K) not in policy.k_split_choices and policy.recall("k_split_choices", (N, K)) is None:
                    policy.k_split_choices[(N, K)] = _measure_k_splits(x, weight, splits)
                chosen = policy.k_split_choices.get((N, K), 0)
                splits = chosen or splits
            if splits > 1:
                parts = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
                _check(lib.cw_gemm_bf16_skinny(3, _ptr(x), K, _ptr(weight), _ptr(parts), N, M, N, K, chosen, _stream()),
                       "gemm_bf16_skinny(partial)")
                return PartialSums(parts)
        want_f32 = out_dtype == torch.float32
        if lib.cw_gemm_bf16_skinny_fast(1 if want_f32 else 0, M, N, K):
            out = torch.empty((M, N), dtype=torch.float32 if want_f32 else torch.bfloat16, device=x.device)
            _check(lib.cw_gemm_bf16_skinny(1 if want_f32 else 0, _ptr(x), K, _ptr(weight), _ptr(out), N, M, N, K, 0, _stream()),
                   "gemm_bf16_skinny")
            return out
    if partial_ok and out_dtype is None and bias is None and M >= WIDE_PRODUCT_MIN_ROWS and x.is_contiguous():
        splits = _wide_partial_chosen(x, weight, policy)
        if splits:
            return linear_wide_partial(x, weight, splits)
    if policy.hip_products and K % 8 == 0 and x.is_contiguous():
        y = linear_tiled(x, weight, bias)
    elif _wide_product_chosen(x, weight, bias, policy):
        y = linear_tiled(x, weight, bias, wide=True)
    else:
        y = _library_product(x, weight, bias)
    if out_dtype == torch.float32:
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
        _check(_load("core").cw_bf16_to_f32(_ptr(y), _ptr(out), M * N, _stream()), "bf16_to_f32")
        return out
    return y


class ProductPolicy:
    """How one engine runs its products of many bfloat16 rows. Every runner has one of its own and
    hands it to the parts through the step context, so two engines in a process (other options,
    other weights) never see each other's choices.

    ``hip_products``: such products go through this package's own LDS-tiled kernels instead of the
    library (about half as fast on an MI355X; for a run that must not depend on the library).
    ``swiglu_choices`` / ``product_choices``: for a weight shape that a tuning start-up has timed
    both ways, whether the wide-tile kernel was the faster one ((rows of [gate; up], K) and
    (N, K, with bias)); shapes never timed follow the fixed rules. ``k_split_choices``: for an
    (N, K) whose product of few rows is summed in parts over K (a narrow output with a long K),
    the number of parts that start-up found the fastest, the same for every step of up to 16 rows.
    ``wide_partial_choices``: for an (N, K) of a long portion's product with a narrow output and a
    long K, into how many runs of K the wide-tile kernel sums it (0: the library's product stays).
    ``tuning``: such a start-up is under way (``library_tuning``)."""

    __slots__ = ("hip_products", "swiglu_choices", "product_choices", "k_split_choices", "wide_partial_choices", "tuning",
                 "_remembered")

    TABLES = ("swiglu_choices", "product_choices", "k_split_choices", "wide_partial_choices")

    def __init__(self, hip_products: bool = False) -> None:
        self.hip_products = bool(hip_products)
        self.swiglu_choices: dict = {}
        self.product_choices: dict = {}
        self.k_split_choices: dict = {}
        self.wide_partial_choices: dict = {}
        self.tuning = False
        self._remembered: dict = {name: {} for name in self.TABLES}

    def read_choices(self, path: str) -> int:
        """Remember what earlier start-ups on this card and kernel build measured and left in
        ``path``: a shape's entry comes into use when this engine's own start-up asks for that
        shape (``recall``), in place of measuring it again; other models' shapes stay aside. A file
        that is missing, unreadable or from another card or build is passed over. Returns the number
        of entries remembered."""
        try:
            with open(path) as f:
                record = json.load(f)
            if record.get("made_for") != _choices_made_for():
                return 0
            taken = 0
            for name in self.TABLES:
                for key, value in record.get(name, []):
                    self._remembered[name][tuple(key)] = value
                    taken += 1
            return taken
        except (OSError, ValueError, TypeError, AttributeError):
            return 0

    def recall(self, table: str, key):
        """What an earlier start-up measured for ``key`` of ``table``, put into use; None if
        nothing is remembered (or this policy holds a choice of its own already)."""
        active = getattr(self, table)
        if key in active or key not in self._remembered[table]:
            return None
        active[key] = self._remembered[table][key]
        return active[key]

    def write_choices(self, path: str) -> None:
        """Leave what is remembered and this policy's own choices (which win) in ``path``, written
        beside it and moved over it, so a reader never sees half a file; where the folder cannot be
        written nothing is kept."""
        record = {"made_for": _choices_made_for()}
        for name in self.TABLES:
            merged = {**self._remembered[name], **getattr(self, name)}
            record[name] = [[list(key), value] for key, value in merged.items()]
        try:
            fd, tmp = tempfile.mkstemp(dir=os.path.dirname(path) or ".", prefix=".choices-")
            with os.fdopen(fd, "w") as f:
                json.dump(record, f)
            os.replace(tmp, path)
        except OSError:
            pass


def choices_file() -> str:
    """Where a tuning start-up keeps what it measured for this package's own kernels: a file in
    the temporary folder, one per user and per card and kernel build (so that what one kind of
    card measured is never handed to, or overwritten by, another), or where
    CLOCKWORK_AMD_CHOICES_FILE points."""
    named = os.environ.get("CLOCKWORK_AMD_CHOICES_FILE")
    if named:
        return named
    mark = hashlib.sha256(json.dumps(_choices_made_for()).encode()).hexdigest()[:10]
    return os.path.join(tempfile.gettempdir(), f"clockwork_amd_choices_{os.getuid()}_{mark}.json")


def _choices_made_for() -> list:
    """What measured choices hold for: the card (its architecture, compute units and memory: the
    marketing name is empty under a profiler) and the builds of the kernels that were timed."""
    card = ["none"]
    if torch.cuda.is_available():
        props = torch.cuda.get_device_properties(torch.cuda.current_device())
        card = [str(getattr(props, "gcnArchName", props.name)), int(props.multi_processor_count), int(props.total_memory)]
    return card + [torch.__version__] + [build.library_path(n).name for n in ("gemm", "gemm_tile", "core")]


# what a call without an engine behind it runs by: the library for large products, nothing timed
DEFAULT_POLICY = ProductPolicy()


# up to this many rows every product goes through the weight-streaming kernels
SKINNY_MAX_ROWS = 16
# up to this many rows the shapes that the persistent streaming kernel takes do (the library
# product is faster for the others, measured)
STREAM_MAX_ROWS = 64
# the fused q/k/v kernel takes more than SKINNY_MAX_ROWS rows for weight matrices up to this many elements
FUSED_QKV_MAX_WEIGHTS = 8 << 20


def linear_tiled(x: torch.Tensor, weight: torch.Tensor, bias=None, swiglu: bool = False, wide=None) -> torch.Tensor:
    """y = x @ weight.T (+ bias), or with ``swiglu`` silu(x @ gate.T) * (x @ up.T) for weight =
    [gate; up], through the LDS-tiled matrix-core kernels for many bfloat16 rows (csrc/gemm_tile.hip):
    the one with 256 x 192 tiles where it takes the shape and has tiles enough to fill the GPU, the
    one with 128 x 128 tiles otherwise (``wide``: True or False to say which). The rows of x may
    have a stride (a slice of a wider buffer)."""
    _gpu(weight, bias)
    if not (x.is_cuda and x.dim() == 2):
        raise KernelError("x must be a 2-d tensor on the GPU")
    M, K = x.shape
    N = weight.shape[0]
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        raise KernelError("the tiled product is bfloat16")
    if not (weight.shape[1] == K and K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0):
        raise KernelError("rows of 16-byte multiples")
    if not (not swiglu or (N % 2 == 0 and bias is None)):
        raise KernelError("gate_up weight must be [2 I, K], without bias")
    if bias is not None:
        if not (bias.numel() == N and bias.dtype in (torch.bfloat16, torch.float32)):
            raise KernelError("bias must be [N] bfloat16 or float32")
    out = torch.empty((M, N // 2 if swiglu else N), dtype=torch.bfloat16, device=x.device)
    lib = _load("gemm_tile")
    mode = 2 if swiglu else 0
    bias_f32 = int(bias is not None and bias.dtype == torch.float32)
    if wide is None:
        wide = lib.cw_gemm_bf16_wide_tiles(mode, M, N, K, x.stride(0)) >= WIDE_MIN_TILES
    if wide:
        _check(lib.cw_gemm_bf16_wide(mode, _ptr(x), x.stride(0), _ptr(weight), _ptr(bias), bias_f32, _ptr(out), out.shape[1],
                                     M, N, K, _compute_units(x.device), _stream()), "gemm_bf16_wide")
    else:
        _check(lib.cw_gemm_bf16_tiled(mode, _ptr(x), x.stride(0), _ptr(weight), _ptr(bias), bias_f32, _ptr(out), out.shape[1],
                                      M, N, K, _stream()), "gemm_bf16_tiled")
    return out


# the wide-tile kernel runs one workgroup per compute unit: with fewer tiles than this the
# 128 x 128 kernel, whose tiles are a quarter of the size, fills the GPU better
WIDE_MIN_TILES = 64
# The engine takes the wide-tile kernel for the gate/up product by itself (no ``hip_products``)
# where it beats the library product followed by the gate kernel. Measured on an MI355X over the
# Qwen2.5 layer shapes from 0.5B to 72B with 256 to 4096 rows: with 180 tiles or more (seven tenths
# of the compute units busy in the last round) and 1024 rows or more it is 5 to 25 % faster; with
# fewer rows the product is bound by reading W once, which the library does better for the large
# shapes (and 512 rows win only for the small ones). Against the library's TUNED choice it wins for
# the 0.5B, 1.5B, 3B, 14B and 32B shapes (the 1.5B shape's whole prefill step: 8.9 -> 7.9 ms) and
# loses 3 % of the step for the 7B and 72B shapes, so a start-up that tunes (``library_tuning``)
# times both ways on the model's own weights and keeps the faster (``ProductPolicy.swiglu_choices``).
WIDE_SWIGLU_MIN_TILES = 180
WIDE_SWIGLU_MIN_ROWS = 1024
WIDE_SWIGLU_SMALL_WEIGHTS = 64 << 20    # elements of [gate; up] up to which 512 rows are enough

_cu_counts: dict = {}


def _compute_units(device) -> int:
    n = _cu_counts.get(device)
    if n is None:
        n = _cu_counts[device] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return n


def wide_swiglu_pays(M: int, two_i: int, K: int, ldx: int) -> bool:
    """Is the gate/up product of M rows faster through the wide-tile kernel (with the gate in its
    epilogue) than through the library and the gate kernel?"""
    if M < WIDE_SWIGLU_MIN_ROWS and not (M >= WIDE_SWIGLU_MIN_ROWS // 2 and two_i * K <= WIDE_SWIGLU_SMALL_WEIGHTS):
        return False
    return _load("gemm_tile").cw_gemm_bf16_wide_tiles(2, M, two_i, K, ldx) >= WIDE_SWIGLU_MIN_TILES


@contextlib.contextmanager
def library_tuning(policy: "ProductPolicy | None" = None):
    """While active, a library product of a shape not seen before is timed over the library's
    candidate kernels and the fastest is remembered; afterwards the remembered choices stay in
    use and unseen shapes take the library's own default again. The library keeps its choices in a
    file in the temporary folder (or where PYTORCH_TUNABLEOP_FILENAME points), which later
    processes of the same user read. ``policy``: the engine whose own kernels are timed against the
    library's meanwhile; what it measures is kept in a file beside the library's
    (``choices_file``), so that a later process on the same card and build, a profiled run among
    them, takes the same kernels without timing them again. Not to be left active during
    HIP-graph capture."""
    import torch.cuda.tunable as tunable

    policy = policy if policy is not None else DEFAULT_POLICY
    if not os.environ.get("PYTORCH_TUNABLEOP_FILENAME"):
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"clockwork_amd_products_{os.getuid()}.csv"), True)
    tunable.enable(True)
    tunable.tuning_enable(True)
    policy.tuning = True
    policy.read_choices(choices_file())
    try:
        yield
    finally:
        policy.tuning = False
        tunable.tuning_enable(False)
        policy.write_choices(choices_file())


# a plain product is timed against the library's only with this many rows and tiles (half the
# compute units busy): below that the library has always been the faster one
WIDE_PRODUCT_MIN_ROWS = 1024
WIDE_PRODUCT_MIN_TILES = 128


def _library_product(x, weight, bias):
    return torch.mm(x, weight.t()) if bias is None else torch.addmm(bias, x, weight.t())


def _wide_product_chosen(x: torch.Tensor, weight: torch.Tensor, bias, policy: ProductPolicy) -> bool:
    """Does a plain product of many bfloat16 rows go through the wide-tile kernel? Only where a
    tuning start-up has timed it against the library's tuned kernel on these very shapes and
    found it faster (measured: the 7B shape's down product, 279 against 351 us)."""
    M, K = x.shape
    if M < WIDE_PRODUCT_MIN_ROWS or not policy.product_choices and not policy.tuning:
        return False
    key = (weight.shape[0], K, bias is not None)
    choice = policy.product_choices.get(key)
    if choice is None and policy.tuning:
        choice = policy.recall("product_choices", key)
    if choice is None and policy.tuning and x.is_contiguous():
        if _load("gemm_tile").cw_gemm_bf16_wide_tiles(0, M, key[0], K, K) >= WIDE_PRODUCT_MIN_TILES:
            library = _timed_us(lambda: _library_product(x, weight, bias))
            own = _timed_us(lambda: linear_tiled(x, weight, bias, wide=True))
            choice = own <= library
        else:
            choice = False
        policy.product_choices[key] = choice
    return bool(choice) and x.is_contiguous()


def _timed_us(fn, repeats: int = 5) -> float:
    """The median time of ``fn`` with its operands out of the caches, as a layer finds its weights
    in a model larger than the last-level cache: 512 MB are written between the runs. (Timed
    back to back, a product whose weights fit that cache looks faster than it is in a step.)"""
    fn()
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    times = []
    for _ in range(repeats):
        flush.zero_()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        fn()
        end.record()
        end.synchronize()
        times.append(begin.elapsed_time(end) * 1e3)
    return sorted(times)[len(times) // 2]


def _replayed_us(candidates: dict, rounds: int, flush: bool, replays: int = 3) -> dict:
    """The time of each of ``candidates`` (name -> a function of the round's number that launches
    this package's own kernels only) as the kernels take it inside a captured graph of ``rounds``
    rounds, replayed a few times. The operands have to come from memory as they do in a step:
    either the candidate takes other copies of them from round to round, more than the caches
    hold, or (``flush``) 512 MB are written before every round and what a graph of the writes
    alone takes is subtracted. For kernels of a few microseconds, whose differences a timing of
    eager launches blurs (the launches' own time lies on top and overlaps the kernels differently
    from one candidate to the next: two counts of parts over K that differ by 5 us in the decode
    step differed by 2 us timed that way)."""
    wash = torch.empty(512 << 20, dtype=torch.uint8, device="cuda") if flush else None

    def median_replay(fn) -> float:
        def body():
            for i in range(rounds):
                if wash is not None:
                    wash.zero_()
                if fn is not None:
                    fn(i)

        body()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        was_enabled = gc.isenabled()
        gc.disable()  # a collection must not destroy another graph while this capture is open
        try:
            with torch.cuda.graph(graph):
                body()
        finally:
            if was_enabled:
                gc.enable()
        graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(replays):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            graph.replay()
            end.record()
            end.synchronize()
            times.append(begin.elapsed_time(end) * 1e3)
        del graph
        return sorted(times)[len(times) // 2]

    writes = median_replay(None) if flush else 0.0
    return {name: (median_replay(fn) - writes) / rounds for name, fn in candidates.items()}


# copies of a weight matrix that a timing walks through so that each comes from memory again:
# together more than the memory-side cache holds
_COLD_COPIES_BYTES = 320 << 20


def _cold_copies(weight: torch.Tensor) -> list:
    """``weight`` and as many copies of it as together exceed the caches (16 at most); the matrix
    alone where the memory for them is not there."""
    n = min(16, max(2, -(-_COLD_COPIES_BYTES // (weight.numel() * weight.element_size())) + 1))
    try:
        return [weight] + [weight.clone() for _ in range(n - 1)]
    except torch.OutOfMemoryError:
        return [weight]


def linear_wide_partial(x: torch.Tensor, weight: torch.Tensor, k_splits: int) -> PartialSums:
    """x @ weight.T as ``k_splits`` float32 planes of partial sums over runs of K, through the
    wide-tile kernel (csrc/gemm_tile.hip): for a long portion's product whose output is too narrow
    to fill the card with whole tiles (the down product: 64 tiles of 256 x 192 for 2048 rows of the
    1.5B shape), and whose result goes straight into ``add_rmsnorm``."""
    _gpu(x, weight)
    M, K = x.shape
    N = weight.shape[0]
    lib = _load("gemm_tile")
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.shape[1] == K
            and lib.cw_gemm_bf16_wide_partial_ok(M, N, K, x.stride(0), int(k_splits))):
        raise KernelError("the wide-tile kernel does not sum this product in parts")
    parts = torch.empty((int(k_splits), M, N), dtype=torch.float32, device=x.device)
    _check(lib.cw_gemm_bf16_wide_partial(_ptr(x), x.stride(0), _ptr(weight), _ptr(parts), N, M, N, K, int(k_splits),
                                         _compute_units(x.device), _stream()), "gemm_bf16_wide_partial")
    return PartialSums(parts)


# a long portion's product is a candidate for the wide-tile kernel's partial sums when whole tiles
# would leave most compute units idle and K is long enough to cut
WIDE_PARTIAL_MAX_TILES = 128
WIDE_PARTIAL_MIN_K = 1024


def _wide_partial_chosen(x: torch.Tensor, weight: torch.Tensor, policy: ProductPolicy) -> int:
    """Into how many runs of K does the wide-tile kernel sum this product of many rows (0: it
    does not, the library's product runs)? Only what a tuning start-up has measured on these very
    shapes: the kernel's partial sums and the norm that adds them against the library's product and
    the norm of its bfloat16 result."""
    M, K = x.shape
    N = weight.shape[0]
    key = (N, K)
    choice = policy.wide_partial_choices.get(key)
    if choice is None and policy.tuning:
        choice = policy.recall("wide_partial_choices", key)
    if choice is None and policy.tuning:
        lib = _load("gemm_tile")
        tiles = lib.cw_gemm_bf16_wide_tiles(0, M, N, K, K)
        choice = 0
        if 0 < tiles <= WIDE_PARTIAL_MAX_TILES and K >= WIDE_PARTIAL_MIN_K:
            resid = torch.zeros((M, N), dtype=torch.float32, device=x.device)
            norm_weight = torch.ones(N, dtype=torch.bfloat16, device=x.device)
            out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            best = _timed_us(lambda: add_rmsnorm(resid, _library_product(x, weight, None), norm_weight, 1e-6, out, write_back=False))
            for splits in (2, 3, 4, 5, 6, 7, 8):
                if not lib.cw_gemm_bf16_wide_partial_ok(M, N, K, K, splits):
                    continue
                t = _timed_us(lambda: add_rmsnorm(resid, linear_wide_partial(x, weight, splits), norm_weight, 1e-6, out, write_back=False))
                if t < 0.97 * best:
                    best, choice = t, splits
        policy.wide_partial_choices[key] = choice
    return int(choice or 0)


def _measure_k_splits(x: torch.Tensor, weight: torch.Tensor, default: int) -> int:
    """Into how many parts over K is the product of these few rows with ``weight`` [N, K] summed
    the fastest, together with the norm kernel that adds the parts up? Which count lets the
    streaming kernel in, fills the card evenly and leaves whole chunks to a wave differs from shape
    to shape (the 7B shape's down product with the norm: 38.4 us with 5 parts, 32.4 with 7; the 32B
    shape's: 64.8 with 7, 59.2 with 6), so the candidates are timed on the model's own weights,
    inside captured graphs that walk through copies of the matrix (each comes from memory again)."""
    M, K = x.shape
    N = weight.shape[0]
    lib = _load("gemm")
    resid = torch.zeros((M, N), dtype=torch.float32, device=x.device)
    norm_weight = torch.ones(N, dtype=torch.bfloat16, device=x.device)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)

    weights = _cold_copies(weight)

    def run(splits: int, round_no: int):
        w = weights[round_no % len(weights)]
        parts = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        _check(lib.cw_gemm_bf16_skinny(3, _ptr(x), K, _ptr(w), _ptr(parts), N, M, N, K, splits, _stream()),
               "gemm_bf16_skinny(partial)")
        add_rmsnorm(resid, PartialSums(parts), norm_weight, 1e-6, out, write_back=False)

    candidates = sorted({default, *(s for s in (2, 3, 4, 5, 6, 7, 8, 10, 12) if K // s >= 256)})
    rounds = len(weights) * -(-12 // len(weights)) if len(weights) > 1 else 6
    times = _replayed_us({splits: (lambda i, splits=splits: run(splits, i)) for splits in candidates},
                         rounds=rounds, flush=len(weights) == 1)
    best = min(times, key=times.get)
    # the fixed rule stays unless something is clearly faster: no flapping between equals
    return best if times[best] < 0.97 * times[default] else default


def _measure_swiglu(x: torch.Tensor, gate_up_weight: torch.Tensor, out: torch.Tensor) -> bool:
    """Time the two ways of a long portion's gate/up product on these operands (the library has
    just chosen its kernel for the shape): is this package's kernel at least as fast as the
    library's product followed by the gate kernel?"""
    library = _timed_us(lambda: silu_mul(_library_product(x, gate_up_weight, None), out))
    own = _timed_us(lambda: linear_tiled(x, gate_up_weight, swiglu=True, wide=True))
    return own <= library


def qkv_rope_fused_supported(x: torch.Tensor, weight: torch.Tensor, rotary_dim: int, hd: int) -> bool:
    """The fused q/k/v product + rotary + cache write takes few bfloat16 rows and a full rotary
    dimension. Beyond 16 rows it serves small weight matrices only: a large one is faster as a
    product and a rotation kernel (measured: 33 MB at 24 rows and more)."""
    rows = x.shape[0]
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and (rows <= SKINNY_MAX_ROWS or (rows <= STREAM_MAX_ROWS and weight.numel() <= FUSED_QKV_MAX_WEIGHTS))
            and x.shape[1] % 8 == 0 and rotary_dim == hd and hd % 16 == 0)


def qkv_rope_fused(x, weight, bias, positions, slots, inv_freq, nh: int, nkv: int, hd: int, k_cache, v_cache) -> torch.Tensor:
    """q = rope(x @ Wq.T + bq) returned as [M, nh * hd]; rope(x @ Wk.T + bk) and x @ Wv.T + bv written
    to the cache rows ``slots``: one kernel for few bfloat16 rows (see csrc/gemm.hip)."""
    _gpu(x, weight, bias, positions, slots, inv_freq, k_cache, v_cache)
    M, K = x.shape
    if not (qkv_rope_fused_supported(x, weight, hd, hd)):
        raise KernelError("the fused q/k/v kernel does not take these operands")
    if not (tuple(weight.shape) == ((nh + 2 * nkv) * hd, K)):
        raise KernelError("qkv weight must be [(nh + 2 nkv) hd, K]")
    _i32(positions, M, "positions")
    _i32(slots, M, "slots")
    if not (inv_freq.dtype == torch.float32 and inv_freq.numel() == hd // 2):
        raise KernelError("inv_freq must be float32 [hd / 2]")
    _need(k_cache.dtype == torch.bfloat16 and tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape,
          "cache must be bfloat16 [..., nkv, hd]")
    if bias is not None:
        if not (bias.numel() == weight.shape[0] and bias.dtype in (torch.bfloat16, torch.float32)):
            raise KernelError("qkv bias")
    q = torch.empty((M, nh * hd), dtype=torch.bfloat16, device=x.device)
    _check(
        _load("gemm").cw_gemm_qkv_rope_bf16(
            _ptr(x), K, _ptr(weight), _ptr(bias), int(bias is not None and bias.dtype == torch.float32), _ptr(positions),
            _ptr(slots), _ptr(inv_freq), _ptr(q), _ptr(k_cache), _ptr(v_cache), k_cache.numel() // (nkv * hd),
            M, K, nh, nkv, hd, _stream()),
        "gemm_qkv_rope_bf16",
    )
    return q


def swiglu_norm_fusable(M: int, two_i: int, K: int, dtype, gate_up_weight, delta) -> bool:
    """Can the gate/up product make its own input rmsnorm(resid + delta)? Few bfloat16 rows of a
    shape the streaming kernel takes, the pending delta a plain bfloat16 tensor."""
    return (dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and gate_up_weight.shape[1] == K
            and isinstance(delta, torch.Tensor) and delta.dtype == torch.bfloat16 and delta.is_contiguous()
            and bool(_load("gemm").cw_gemm_bf16_swiglu_normed_ok(M, two_i, K)))


def linear_swiglu(x, gate_up_weight: torch.Tensor, policy: "ProductPolicy | None" = None) -> torch.Tensor:
    """silu(x @ gate.T) * (x @ up.T) for gate_up_weight = [gate; up] stacked along dim 0.

    Few bfloat16 rows: one kernel that streams the weights once and applies the gate in its
    epilogue. Otherwise the product followed by the gate kernel, or (``policy``, see ``linear``)
    a tiled kernel with the gate in its epilogue."""
    policy = policy if policy is not None else DEFAULT_POLICY
    if isinstance(x, LazyAddNorm):
        M, K = x.shape
        two_i = gate_up_weight.shape[0]
        if swiglu_norm_fusable(M, two_i, K, x.dtype, gate_up_weight, x.delta):
            _gpu(x.resid, x.delta, x.weight, gate_up_weight)
            out = torch.empty((M, two_i // 2), dtype=x.dtype, device=x.resid.device)
            _check(
                _load("gemm").cw_gemm_bf16_swiglu_normed(
                    _ptr(x.resid), _ptr(x.delta), _ptr(x.weight), int(x.weight.dtype == torch.float32), float(x.eps),
                    _ptr(gate_up_weight), _ptr(out), two_i // 2, M, two_i, K, _stream()),
                "gemm_bf16_swiglu_normed",
            )
            return out
        x = x.value()
    _gpu(x, gate_up_weight)
    M, K = x.shape
    two_i = gate_up_weight.shape[0]
    if not (gate_up_weight.shape[1] == K and two_i % 2 == 0):
        raise KernelError("gate_up weight must be [2 I, K]")
    out = torch.empty((M, two_i // 2), dtype=x.dtype, device=x.device)
    if (x.dtype == torch.bfloat16 and M <= STREAM_MAX_ROWS and K % 8 == 0
            and _load("gemm").cw_gemm_bf16_skinny_fast(2, M, two_i, K)):
        if not (gate_up_weight.dtype == torch.bfloat16):
            raise KernelError("a bfloat16 product needs bfloat16 operands")
        _check(_load("gemm").cw_gemm_bf16_skinny(2, _ptr(x), K, _ptr(gate_up_weight), _ptr(out), two_i // 2, M, two_i, K, 0, _stream()),
               "gemm_bf16_skinny(swiglu)")
        return out
    if x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and K % 8 == 0 and x.is_contiguous():
        if policy.hip_products:
            return linear_tiled(x, gate_up_weight, swiglu=True)
        if wide_swiglu_pays(M, two_i, K, K):
            # with enough rows the shape of the weights decides, and a start-up that tunes the
            # library's products has measured it for this model's
            measured = M >= WIDE_SWIGLU_MIN_ROWS
            if (measured and policy.tuning and (two_i, K) not in policy.swiglu_choices
                    and policy.recall("swiglu_choices", (two_i, K)) is None):
                policy.swiglu_choices[(two_i, K)] = _measure_swiglu(x, gate_up_weight, out)
            if not measured or policy.swiglu_choices.get((two_i, K), True):
                return linear_tiled(x, gate_up_weight, swiglu=True, wide=True)
    return silu_mul(linear(x, gate_up_weight, policy=policy), out)


_zero_rows: dict = {}


def _zero_row(device) -> int:
    """Address of 1 KiB of zeros on ``device``: what the attention kernels read masked rows from."""
    t = _zero_rows.get(device)
    if t is None:
        t = _zero_rows[device] = torch.zeros(512, dtype=torch.bfloat16, device=device)
    return t.data_ptr()


def prefill_attention_supported(hd: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and bool(_load("attention", hd).cw_attention_prefill_supported())


def attention_prefill(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
                      nh: int, nkv: int, hd: int, block_size: int, window: int, scale: float,
                      n_tokens: int, n_requests: int, row_blocks: int = 4, workspace=None, softcap: float = 0.0) -> None:
    """Portions of prompts through the bfloat16 matrix-core kernel (``softcap`` c > 0: scores are
    squashed, c * tanh(scale * q . k / c), before the softmax); an item holds at most
    ``prefill_tokens_per_item(nh // nkv, row_blocks)`` tokens. ``row_blocks`` 2 instead of 4: smaller
    workgroups for launches with few items (head sizes up to 128). Other arguments as for ``attention``.
    An item's fourth field is ``part | parts << 8``: with parts > 1 the item stands that many times
    in the list, one after the other, and each takes a share of its keys; such a list needs a
    float32 ``workspace`` of ``prefill_attention_workspace_floats`` elements (without one every item
    computes all of its keys)."""
    if not (prefill_row_blocks_ok(hd, row_blocks)):
        raise KernelError(f"the kernel for head size {hd} does not take {row_blocks} row blocks")
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    ws_floats = 0
    if workspace is not None:
        need = prefill_attention_workspace_floats(hd, n_items, nh, nkv, row_blocks)
        _need(workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"attention over parts of key ranges needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("the kernel is bfloat16")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    _check(
        _load("attention", hd).cw_attention_prefill_bf16(
            q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
            block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv, block_size,
            window, float(scale), _zero_row(out.device), int(row_blocks), int(workspace is not None), _ptr(workspace),
            ws_floats, float(softcap), _stream()),
        "attention_prefill_bf16",
    )


def prefill_attention_workspace_floats(hd: int, n_items: int, nh: int, nkv: int, row_blocks: int) -> int:
    return int(_load("attention", hd).cw_attention_prefill_workspace_floats(n_items, nh, nkv, int(row_blocks)))


def prefill_row_blocks_ok(hd: int, row_blocks: int) -> bool:
    return bool(_load("attention", hd).cw_attention_prefill_row_blocks_ok(int(row_blocks)))


def prefill_tokens_per_item(group: int, row_blocks: int = 4) -> int:
    """Tokens one work item of ``attention_prefill`` may hold: a row block is 32 rows, a row a
    (token, head of the group) pair."""
    return row_blocks * (32 // min(group, 32))


def decode_attention_supported(hd: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and bool(_load("attention", hd).cw_attention_decode_supported())


# the most splits the bfloat16 decode kernel takes (DEC_MAX_SPLITS in csrc/attention.hip)
DECODE_MAX_SPLITS = 256


def decode_attention_workspace_floats(hd: int, n_items: int, nh: int, nkv: int, n_splits: int) -> int:
    return int(_load("attention", hd).cw_attention_decode_workspace_floats(n_items, nh, nkv, n_splits))


def attention_decode(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
                     nh: int, nkv: int, hd: int, block_size: int, n_splits: int, window: int, scale: float,
                     n_tokens: int, n_requests: int, workspace=None, identity: bool = False,
                     split_keys: int = 0, max_ctx: int = 0, softcap: float = 0.0) -> None:
    """Single-token items through the bfloat16 decode kernel; arguments as for ``attention``
    (``softcap`` as for ``attention_prefill``).
    With more than one split it needs a float32 ``workspace``. ``identity``: item i is request i
    with its token in row i (no other items). ``split_keys`` > 0: every split takes that many
    keys at a fixed place; no context may then be longer than ``max_ctx`` <= n_splits * split_keys."""
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("the decode kernel is bfloat16")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    if identity:
        if not (n_items == n_requests == n_tokens):
            raise KernelError("identity items: one single-token item per request, nothing else")
    if split_keys:
        if not (split_keys % 32 == 0 and split_keys * n_splits >= max_ctx > 0):
            raise KernelError("fixed key ranges do not cover the longest context")
    lib = _load("attention", hd)
    need = lib.cw_attention_decode_workspace_floats(n_items, nh, nkv, n_splits)
    ws_floats = 0
    if need > 0:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"decode attention needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    _check(
        lib.cw_attention_decode_bf16(
            q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
            block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv, block_size, n_splits,
            window, float(scale), _ptr(workspace), ws_floats, _zero_row(out.device), int(bool(identity)),
            int(split_keys), int(max_ctx), float(softcap), _stream()),
        "attention_decode_bf16",
    )


def attention(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
              rows: int, nh: int, nkv: int, hd: int, block_size: int, gh: int, n_splits: int, window: int,
              scale: float, n_tokens: int, n_requests: int, workspace=None) -> None:
    """Paged causal attention for ``n_items`` work items (see csrc/attention.hip).

    q: any tensor whose token rows are ``q_stride`` elements apart with head h at column h * hd;
    out [n_tokens, nh * hd]; caches [num_blocks * block_size, nkv, hd]; block_tables int32
    [n_requests, max_blocks]; items int32 [n_items, 4] = (request, first token, tokens, 0)."""
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention operands differ in type or device")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    lib = _load("attention", hd)
    group = nh // nkv
    n_chunks = -(-group // gh)
    need = lib.cw_attention_workspace_floats(rows, n_items, nkv, n_chunks, n_splits)
    ws_floats = 0
    if need > 0:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"attention needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    _check(
        lib.cw_attention(
            rows, dtype_code(out.dtype), q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache),
            _ptr(block_tables), block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv,
            block_size, gh, n_splits, window, float(scale), _ptr(workspace), ws_floats, _stream()),
        "attention",
    )


def attention_workspace_floats(hd: int, rows: int, n_items: int, nkv: int, n_chunks: int, n_splits: int) -> int:
    return int(_load("attention", hd).cw_attention_workspace_floats(rows, n_items, nkv, n_chunks, n_splits))


def argmax(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """First index of the maximum of every row of float32 ``logits`` [n, V] -> int32 [n]."""
    _gpu(logits, out)
    if not (logits.dtype == torch.float32 and logits.dim() == 2):
        raise KernelError("logits must be float32 [n, V]")
    n, V = logits.shape
    lib = _load("sampling")
    chunks = lib.cw_argmax_chunks(V)
    ws = torch.empty(max(1, n * chunks * 2), dtype=torch.int32, device=logits.device)
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
    _i32(out, n, "out")
    _check(lib.cw_argmax(_ptr(logits), V, n, V, _ptr(out), _ptr(ws), ws.numel() * 4, _stream()), "argmax")
    return out


def sample(logits, temperature, top_k, top_p, seeds, draws, out=None, any_top_k: bool = True,
           any_top_p: bool = True) -> torch.Tensor:
    """One token per row: rows with temperature 0 take the arg-max, the others are drawn.
    ``any_top_k`` / ``any_top_p`` off: the caller knows that no row has that option, and its
    kernels are not launched."""
    _gpu(logits, temperature, top_k, top_p, seeds, draws, out)
    if not (logits.dtype == torch.float32 and logits.dim() == 2):
        raise KernelError("logits must be float32 [n, V]")
    n, V = logits.shape
    if not (temperature.dtype == torch.float32 and temperature.numel() == n):
        raise KernelError("temperature must be float32 [n]")
    if not (top_p.dtype == torch.float32 and top_p.numel() == n):
        raise KernelError("top_p must be float32 [n]")
    _i32(top_k, n, "top_k")
    if not (seeds.dtype == torch.int64 and seeds.numel() == n):
        raise KernelError("seeds must be int64 [n]")
    if not (draws.dtype == torch.int64 and draws.numel() == n):
        raise KernelError("draws must be int64 [n]")
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
    _i32(out, n, "out")
    lib = _load("sampling")
    ws = torch.empty(int(lib.cw_sample_workspace_bytes(n, V)), dtype=torch.uint8, device=logits.device)
    _check(
        lib.cw_sample(_ptr(logits), V, n, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds), _ptr(draws),
                      _ptr(out), _ptr(ws), ws.numel(), int(bool(any_top_k)) | (int(bool(any_top_p)) << 1), _stream()),
        "sample",
    )
    return out


# ---------------------------------------------------------------------------------------------
# Row-wise kernels of blocks with a LayerNorm, gated branches, a position table, a capped head
def embedding_positions(table: torch.Tensor, ids: torch.Tensor, positions, pos_table, scale: float,
                        out_resid: torch.Tensor) -> torch.Tensor:
    """out_resid[t] = scale * table[ids[t]] + pos_table[positions[t]] in float32 ([T, H]);
    ``pos_table`` None: no position is added."""
    _gpu(table, ids, positions, pos_table, out_resid)
    T = ids.numel()
    V, H = table.shape
    _i32(ids, T, "ids")
    P = 0
    if pos_table is not None:
        _i32(positions, T, "positions")
        _need(pos_table.dim() == 2 and pos_table.shape[1] == H and pos_table.dtype == table.dtype,
              "the position table must be [positions, H] in the embedding table's type")
        P = pos_table.shape[0]
    _need(out_resid.dtype == torch.float32 and tuple(out_resid.shape) == (T, H), "residual must be [T, H] float32")
    _check(_load("rowwise").cw_embedding_pos(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(positions),
                                             _ptr(pos_table), float(scale), _ptr(out_resid), T, H, V, P, _stream()),
           "embedding_positions")
    return out_resid


class GatedBranches:
    """What a block with gated branches still has to add to the residual stream:
    sigmoid(z[:, :H] + zb[:H]) * a + sigmoid(z[:, H:] + zb[H:]) * b. ``z`` [T, H or 2H] are the
    gates' products, ``zb`` their biases (or None); without ``z`` the branches count as they are;
    ``b`` may be None. A norm that ``accepts_gated`` adds it inside its own kernel."""

    __slots__ = ("z", "zb", "a", "b")

    def __init__(self, z, zb, a, b=None) -> None:
        self.z, self.zb, self.a, self.b = z, zb, a, b

    @property
    def shape(self):
        return self.a.shape

    def check(self, T: int, H: int, dtype) -> None:
        _gpu(self.z, self.zb, self.a, self.b)
        _need(tuple(self.a.shape) == (T, H) and self.a.dtype == dtype, "a gated branch must be [T, H] in the activation type")
        if self.b is not None:
            _need(tuple(self.b.shape) == (T, H) and self.b.dtype == dtype, "a gated branch must be [T, H] in the activation type")
        if self.z is not None:
            cols = 2 * H if self.b is not None else H
            _need(self.z.dim() == 2 and self.z.shape[0] == T and self.z.shape[1] in (cols, 2 * H) and self.z.dtype == dtype,
                  f"the gates' products must be [T, {cols}] in the activation type")
            if self.zb is not None:
                _need(self.zb.numel() == self.z.shape[1], "the gates' biases must match their products")
        else:
            _need(self.zb is None, "gate biases without gates")

    def args(self):
        return (_ptr(self.z), _ptr(self.zb), dtype_code(self.zb.dtype) if self.zb is not None else 0, _ptr(self.a),
                _ptr(self.b), int(self.z.shape[1]) if self.z is not None else 0)


def gated_residual_add(resid: torch.Tensor, pending: GatedBranches) -> torch.Tensor:
    """resid += the gated branches' value (float32)."""
    _gpu(resid)
    T, H = resid.shape
    _need(resid.dtype == torch.float32, "the residual stream is float32")
    pending.check(T, H, pending.a.dtype)
    _check(_load("rowwise").cw_gated_residual_add(_ptr(resid), *pending.args(), dtype_code(pending.a.dtype), T, H, _stream()),
           "gated_residual_add")
    return resid


def add_layernorm(resid, pending, weight, bias, eps: float, out, rows=None) -> torch.Tensor:
    """resid += pending (a :class:`GatedBranches` or None), out = LayerNorm(resid) * weight + bias
    with float32 statistics (the mean, then the mean of the squared deviations); with ``rows``
    only those rows are normed into out[i] and resid is left alone."""
    _gpu(resid, weight, bias, out, rows)
    T, H = resid.shape
    _need(resid.dtype == torch.float32, "the residual stream is float32")
    n = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "rows")
    _need(tuple(out.shape) == (n, H), f"out must be [{n}, {H}]")
    _need(weight.numel() == H and (bias is None or (bias.numel() == H and bias.dtype == weight.dtype)),
          "norm weight and bias must have the row's size and one type")
    if pending is not None:
        pending.check(T, H, out.dtype)
        args = pending.args()
    else:
        args = (None, None, 0, None, None, 0)
    _check(_load("rowwise").cw_add_layernorm(_ptr(resid), *args, _ptr(weight), _ptr(bias), dtype_code(weight.dtype),
                                             float(eps), _ptr(out), dtype_code(out.dtype), _ptr(rows), n, H, _stream()),
           "add_layernorm")
    return out


def gelu_tanh_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = gelu_tanh(gate_up[t, i]) * gate_up[t, I + i]."""
    _gpu(gate_up, out)
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and out.dtype == gate_up.dtype, "gelu_tanh_mul shapes")
    _check(_load("rowwise").cw_gelu_tanh_mul(_ptr(gate_up), _ptr(out), dtype_code(out.dtype), T, two_i // 2, _stream()),
           "gelu_tanh_mul")
    return out


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _gpu(logits)
    _need(logits.dtype == torch.float32 and cap > 0, "the cap takes float32 logits and a positive cap")
    _check(_load("rowwise").cw_softcap(_ptr(logits), logits.numel(), float(cap), _stream()), "softcap")
    return logits


def rms_mean2(a: torch.Tensor, b, wa: torch.Tensor, wb, eps: float) -> torch.Tensor:
    """(rms(a) * wa + rms(b) * wb) / 2 row by row, rms(x) = x / sqrt(mean(x^2) + eps) in float32;
    ``b`` None: rms(a) * wa."""
    _gpu(a, b, wa, wb)
    T, H = a.shape
    _need(wa.numel() == H, "norm weight has the wrong size")
    if b is not None:
        _need(b.shape == a.shape and b.dtype == a.dtype and wb is not None and wb.numel() == H and wb.dtype == wa.dtype,
              "the second row and its weight must match the first")
    out = torch.empty_like(a)
    _check(_load("rowwise").cw_rms_mean2(_ptr(a), _ptr(b), _ptr(wa), _ptr(wb), dtype_code(wa.dtype), float(eps), _ptr(out),
                                         dtype_code(a.dtype), T, H, _stream()), "rms_mean2")
    return out


def qk_rownorm_store(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, nq: int, nk: int, nv: int, q_weight, k_weight,
                     eps: float, slots, k_cache, v_cache) -> None:
    """Rows of ``proj`` [T, width] hold a token's query, key and value projections at the given
    columns: the query projection is RMS-normed as one vector (all heads at once) with
    ``q_weight`` and rewritten in place, the key projection likewise into the cache row
    ``k_cache[slots[t]]``, the values are copied to ``v_cache[slots[t]]``. Caches are flat
    [rows, nk] and [rows, nv] (any trailing shape of that many elements); a negative slot writes
    nothing; ``slots`` None: queries only."""
    _gpu(proj, q_weight, k_weight, slots, k_cache, v_cache)
    T, width = proj.shape
    cache_rows = 0
    if slots is not None:
        _i32(slots, T, "slots")
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == proj.dtype and v_cache.dtype == proj.dtype,
              "the cache must be there and of the activations' type")
        _need(k_cache.numel() % nk == 0 and v_cache.numel() % nv == 0 and k_cache.numel() // nk == v_cache.numel() // nv,
              "key and value planes must hold the same number of rows")
        cache_rows = k_cache.numel() // nk
    for w, n in ((q_weight, nq), (k_weight, nk)):
        _need(w is None or w.numel() == n, "a projection's norm weight must have the projection's size")
    if q_weight is not None and k_weight is not None:
        _need(q_weight.dtype == k_weight.dtype, "the two norm weights must be of one type")
    wt = q_weight if q_weight is not None else k_weight
    _check(_load("rowwise").cw_qk_rownorm_store(
        _ptr(proj), dtype_code(proj.dtype), width, q_off, k_off, v_off, nq, nk, nv, _ptr(q_weight), _ptr(k_weight),
        dtype_code(wt.dtype) if wt is not None else 0, float(eps), _ptr(slots), _ptr(k_cache), _ptr(v_cache), cache_rows, T,
        _stream()), "qk_rownorm_store")


# ---------------------------------------------------------------------------------------------
def sink_attention_max_run(heads: int, kv_heads: int, dim: int, vdim: int) -> int:
    """The most query tokens a workgroup of the sink-attention kernel takes for this geometry
    (0: the geometry is beyond the kernel)."""
    return int(_load("sink_attention").cw_sink_attention_max_bq(heads, kv_heads, dim, vdim))


def sink_attention(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int, run: int,
                   r1, r2, sink, talk, heads: int, kv_heads: int, dim: int, vdim: int, block_size: int, window: int,
                   scale: float) -> None:
    """Attention of the step's queries (``q`` [T, q_stride], a token's heads * dim query elements
    first) over paged keys [rows, kv_heads, dim] and values [rows, kv_heads, vdim], into ``out``
    [T, heads * vdim]. Options (each None: off): ``r1``/``r2`` float32 [heads], the score loses
    r1 * log(1 + r2 * distance); ``sink`` float32 [heads], exp(sink) joins the softmax
    denominator; ``talk`` float32 [heads, heads], the normalised weights are mixed across heads.
    ``items`` int32 [n_items, 4]: (request, first token, tokens <= run, 0)."""
    _gpu(q, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, r1, r2, sink, talk)
    T = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == q_stride and heads * dim <= q_stride, "q must be [T, q_stride] with the query heads first")
    _need(tuple(out.shape) == (T, heads * vdim) and out.dtype == q.dtype, "out must be [T, heads * vdim]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache and activations differ in type")
    _need(tuple(k_cache.shape[-2:]) == (kv_heads, dim) and tuple(v_cache.shape[-2:]) == (kv_heads, vdim),
          "the planes must be [..., kv_heads, dim] and [..., kv_heads, vdim]")
    rows = k_cache.numel() // (kv_heads * dim)
    _need(rows == v_cache.numel() // (kv_heads * vdim), "key and value planes must hold the same number of rows")
    R = ctx_lens.numel()
    _i32(ctx_lens, R, "ctx_lens")
    _i32(cu_q, R + 1, "cu_q")
    _i32(items, 4 * n_items, "items")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= R, "block tables must be int32 [R, width]")
    for t, n, what in ((r1, heads, "r1"), (r2, heads, "r2"), (sink, heads, "sink"), (talk, heads * heads, "talk")):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == n), f"{what} must be float32 with {n} elements")
    _need((r1 is None) == (r2 is None), "the distance bias takes r1 and r2 together")
    _check(_load("sink_attention").cw_sink_attention(
        dtype_code(q.dtype), _ptr(q), q_stride, _ptr(out), _ptr(k_cache), _ptr(v_cache), rows, _ptr(block_tables),
        block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, run, _ptr(r1), _ptr(r2), _ptr(sink),
        _ptr(talk), heads, kv_heads, dim, vdim, block_size, int(window), float(scale), _stream()), "sink_attention")


def linear_recurrence_supported(dim: int, vdim: int) -> bool:
    return bool(_load("linear_recurrence").cw_linear_recurrence_supported(dim, vdim))


RECURRENCE_DECAYS = {"sigmoid_power": 0, "double_exp": 1, "double_exp_tanh": 2}


def _recurrence_operands(proj, q_off, k_off, v_off, g_off, u_off, a2, a2_bias, norm_weight, state, heads, dim, vdim, decay, bonus,
                         decay_input):
    """Checks shared by the two recurrence entry points; returns (T, row stride, the five offsets
    in elements, the trailing arguments of the C call after eps)."""
    _need(decay in RECURRENCE_DECAYS, f"decay {decay!r}: expected one of {sorted(RECURRENCE_DECAYS)}")
    if proj.dim() == 3:
        # planes one behind the other, [planes, T, heads * dim]: an offset names a plane
        P, T, width = proj.shape
        _need(proj.is_contiguous() and width == heads * dim and dim == vdim, "planes hold rows of heads * dim (== heads * vdim) elements")
        _need(decay_input is not None, "with planes the decay input is a tensor of its own")
        _need(all(0 <= o < P for o in (q_off, k_off, v_off)) and g_off < P, "an offset names a plane")
        _need(P * T * width < 2 ** 31, "the planes outgrow 32-bit offsets")
        plane = T * width
        q_off, k_off, v_off, g_off = q_off * plane, k_off * plane, v_off * plane, (g_off * plane if g_off >= 0 else -1)
        u_off = 0
    else:
        T, width = proj.shape
    _need(a2.dim() == 2 and a2.shape[0] == heads * dim and a2.dtype == proj.dtype, "a2 must be [heads * dim, rank] in the activation type")
    _need(a2_bias is None or (a2_bias.dtype == torch.float32 and a2_bias.numel() == heads * dim), "the decay bias must be float32 [heads * dim]")
    _need(norm_weight is None or (norm_weight.dtype == torch.float32 and norm_weight.numel() in (vdim, heads * vdim)),
          "the norm weight must be float32 [vdim] or [heads * vdim]")
    _need(bonus is None or (bonus.dtype == torch.float32 and bonus.numel() == heads * dim), "the bonus must be float32 [heads, dim]")
    _need(state.dtype == torch.float32 and state.dim() >= 2 and state.is_contiguous() and state[0].numel() >= heads * dim * vdim,
          "the state must be float32 [slots, >= heads * dim * vdim]")
    u_stride = 0
    if decay_input is not None:
        _need(tuple(decay_input.shape) == (T, a2.shape[1]) and decay_input.dtype == proj.dtype and decay_input.is_contiguous(),
              "the decay input must be [T, rank] in the activation type")
        u_stride = a2.shape[1]
    per_head = norm_weight is not None and norm_weight.numel() == heads * vdim and heads > 1
    tail = (RECURRENCE_DECAYS[decay], _ptr(bonus), vdim if per_head else 0, _ptr(decay_input), u_stride, state[0].numel())
    return T, width, (int(q_off), int(k_off), int(v_off), int(g_off), int(u_off)), tail


def linear_recurrence(proj, q_off: int, k_off: int, v_off: int, g_off: int, u_off: int, a2, a2_bias, norm_weight, state,
                      state_slots, cu_q, n_requests: int, heads: int, dim: int, vdim: int, q_scale: float, tau: float,
                      eps: float, decay: str = "sigmoid_power", bonus=None, decay_input=None) -> torch.Tensor:
    """The decayed recurrence S <- diag(a) S + k v^T, o = S^T (q_scale q) over the step's tokens,
    request by request from each request's slot of ``state`` (float32 [slots, ...]: a slot's
    first heads * dim * vdim floats are the matrices, updated in place). Rows of ``proj`` hold q,
    k (heads * dim), v, the output gate (heads * vdim; ``g_off`` < 0: none) and the decay's
    low-rank input (``a2`` [heads * dim, rank] maps it to z; a = sigmoid(z + bias)^(1/tau)). The
    outputs are RMS-normed over vdim with ``norm_weight`` ([vdim] for all heads or [heads * vdim];
    None: not) and multiplied by silu(gate). Returns [T, heads * vdim].

    ``proj`` [planes, T, heads * dim]: q, k, v and the gate are planes, the offsets their numbers.
    ``decay_input`` [T, rank]: the decay's input as a tensor of its own. ``decay`` "double_exp":
    a = exp(-exp(a2 input + bias)); "double_exp_tanh": a = exp(-exp(a2 tanh(input) + bias)). ``bonus`` float32 [heads, dim]: the output reads the
    state before the token joins it and the token itself through the bonus,
    o = (S + diag(bonus) k v^T)^T q, then S <- diag(a) S + k v^T."""
    _gpu(proj, a2, a2_bias, norm_weight, state, state_slots, cu_q, bonus, decay_input)
    T, width, offs, tail = _recurrence_operands(proj, q_off, k_off, v_off, g_off, u_off, a2, a2_bias, norm_weight, state, heads,
                                                dim, vdim, decay, bonus, decay_input)
    _i32(state_slots, n_requests, "state_slots")
    _i32(cu_q, n_requests + 1, "cu_q")
    out = torch.empty((T, heads * vdim), dtype=proj.dtype, device=proj.device)
    _check(_load("linear_recurrence").cw_linear_recurrence(
        dtype_code(proj.dtype), _ptr(proj), width, *offs, _ptr(a2), _ptr(a2_bias),
        _ptr(norm_weight), _ptr(state), state.shape[0], _ptr(state_slots), _ptr(cu_q), _ptr(out), n_requests, heads, dim,
        vdim, a2.shape[1], float(q_scale), 1.0 / float(tau), float(eps), *tail, _stream()), "linear_recurrence")
    return out


def linear_recurrence_segments_supported(dim: int, vdim: int) -> bool:
    return bool(_load("linear_recurrence").cw_linear_recurrence_segments_supported(dim, vdim))


def linear_recurrence_segments(proj, q_off: int, k_off: int, v_off: int, g_off: int, u_off: int, a2, a2_bias, norm_weight,
                               state, state_slots, cu_q, seg_items, n_segments: int, seg_tokens: int, req_first,
                               n_requests: int, heads: int, dim: int, vdim: int, q_scale: float, tau: float,
                               eps: float, decay: str = "sigmoid_power", bonus=None, decay_input=None) -> torch.Tensor:
    """``linear_recurrence`` for steps with long portions: the tokens are cut into segments that
    are walked side by side (each from a zero state, then the segments' start states are carried
    from the request's slot, then each is walked again for its outputs). ``seg_items`` int32
    [n_segments, 4]: (request, first token of the segment in the request's portion, tokens, 0),
    a request's segments in order and together, none longer than ``seg_tokens``; ``req_first`` int32 [R + 1]: where each
    request's segments begin. The same arguments and result otherwise."""
    _gpu(proj, a2, a2_bias, norm_weight, state, state_slots, cu_q, seg_items, req_first, bonus, decay_input)
    T, width, offs, tail = _recurrence_operands(proj, q_off, k_off, v_off, g_off, u_off, a2, a2_bias, norm_weight, state, heads,
                                                dim, vdim, decay, bonus, decay_input)
    _i32(state_slots, n_requests, "state_slots")
    _i32(cu_q, n_requests + 1, "cu_q")
    _i32(seg_items, 4 * n_segments, "seg_items")
    _i32(req_first, n_requests + 1, "req_first")
    lib = _load("linear_recurrence")
    need = lib.cw_linear_recurrence_segments_workspace_floats(T, n_segments, heads, dim, vdim)
    workspace = torch.empty(max(int(need), 1), dtype=torch.float32, device=proj.device)
    out = torch.empty((T, heads * vdim), dtype=proj.dtype, device=proj.device)
    _check(lib.cw_linear_recurrence_segments(
        dtype_code(proj.dtype), _ptr(proj), width, *offs, _ptr(a2), _ptr(a2_bias),
        _ptr(norm_weight), _ptr(state), state.shape[0], _ptr(state_slots), _ptr(cu_q), _ptr(seg_items), n_segments,
        int(seg_tokens), _ptr(req_first), _ptr(workspace), _ptr(out), n_requests, T, heads, dim, vdim, a2.shape[1], float(q_scale),
        1.0 / float(tau), float(eps), *tail, _stream()), "linear_recurrence_segments")
    return out


def tanh_(x: torch.Tensor) -> torch.Tensor:
    """x <- tanh(x), in place, float32 inside."""
    _gpu(x)
    _need(x.is_contiguous(), "tanh_ takes a dense tensor")
    _check(_load("rowwise").cw_tanh(_ptr(x), dtype_code(x.dtype), x.numel(), _stream()), "tanh")
    return x


SHIFT_MIX_TOKENS = 16   # tokens of one request that a work item of ``shift_mix`` holds


def shift_mix(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, prev_off: int, state_slots, cu_q, items,
              n_items: int) -> torch.Tensor:
    """[n, T, W]: out[s, t] = x[t] + (before[t] - x[t]) * mu[s], ``before`` the row of the request's
    token one position earlier: the row above, or for the first token of a request's portion the
    W floats that the request's slot of ``state`` (float32 [slots, ...]) holds from ``prev_off``
    (zeros in a fresh slot). The portion's last row is then left there for the next step. ``mu``
    [n, W]; ``items`` int32 [n_items, 4]: (request, first token, tokens, 0), a request's first item
    beginning at its token 0, at most ``SHIFT_MIX_TOKENS`` tokens each."""
    _gpu(x, mu, state, state_slots, cu_q, items)
    T, W = x.shape
    _need(x.is_contiguous() and mu.dim() == 2 and mu.shape[1] == W and mu.is_contiguous(), "mu must be [n, W]")
    _need(state.dtype == torch.float32 and state.dim() >= 2 and state.is_contiguous() and 0 <= prev_off
          and prev_off + W <= state[0].numel(), "the state must be float32 [slots, >= prev_off + W]")
    R = state_slots.numel()
    _i32(state_slots, R, "state_slots")
    _i32(cu_q, R + 1, "cu_q")
    _i32(items, 4 * n_items, "items")
    out = torch.empty((mu.shape[0], T, W), dtype=x.dtype, device=x.device)
    _check(_load("rowwise").cw_shift_mix(_ptr(x), dtype_code(x.dtype), _ptr(mu), dtype_code(mu.dtype), mu.shape[0], _ptr(state),
                                         state[0].numel(), int(prev_off), state.shape[0], _ptr(state_slots), _ptr(cu_q),
                                         _ptr(items), int(n_items), _ptr(out), T, W, _stream()), "shift_mix")
    return out


def stream_beside_input(resid: torch.Tensor, pending, model_input: torch.Tensor, dtype, extra: int = 0, hot: int = -1) -> torch.Tensor:
    """Adds what is still ``pending`` (None, a tensor, a :class:`PendingPair` or
    :class:`PartialSums`) to the float32 stream ``resid`` in place and returns [T, 2 H + extra] in
    ``dtype``: the stream beside the model's input (float32 [T, H]), then ``extra`` columns of
    zeros with a one in column ``hot`` (which lets the product that follows add one of ``extra``
    learned rows exactly, in its own float32 sums)."""
    a = b = None
    if isinstance(pending, PendingPair):
        a, b = pending.first, pending.second
    elif pending is not None:
        a = pending
    a = a.sum(dtype) if isinstance(a, PartialSums) else a
    b = b.sum(dtype) if isinstance(b, PartialSums) else b
    _gpu(resid, a, b, model_input)
    T, H = resid.shape
    _need(resid.dtype == torch.float32 and model_input.dtype == torch.float32 and tuple(model_input.shape) == (T, H)
          and resid.is_contiguous() and model_input.is_contiguous(), "stream and input must be float32 [T, H]")
    for t in (a, b):
        _need(t is None or (tuple(t.shape) == (T, H) and t.dtype == dtype and t.is_contiguous()), "a pending output must be [T, H] in the activation type")
    _need(extra >= 0 and -1 <= hot < max(extra, 1), "the one must lie inside the extra columns")
    image = torch.empty((T, 2 * H + extra), dtype=dtype, device=resid.device)
    _check(_load("rowwise").cw_stream_beside_input(_ptr(resid), _ptr(a), _ptr(b), _ptr(model_input), _ptr(image), dtype_code(dtype),
                                                   T, H, int(extra), int(hot), _stream()), "stream_beside_input")
    return image


SINK_DECODE_MAX_RUN = 128


def sink_decode_supported(heads: int, kv_heads: int, dim: int, vdim: int) -> bool:
    return bool(_load("sink_attention").cw_sink_decode_supported(heads, kv_heads, dim, vdim))


def sink_attention_decode(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, n_requests: int,
                          run_keys: int, n_runs: int, r1, r2, sink, talk, heads: int, kv_heads: int, dim: int, vdim: int,
                          block_size: int, window: int, scale: float) -> None:
    """``sink_attention`` for the step's requests of one token each (others are left alone): the
    keys a token sees are cut into ``n_runs`` runs of ``run_keys`` keys (the most any request of
    the step has), a workgroup each; three kernels (scores and their sums, values, merge)."""
    _gpu(q, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, r1, r2, sink, talk)
    T = q.shape[0]
    _need(q.dim() == 2 and q.shape[1] == q_stride and heads * dim <= q_stride, "q must be [T, q_stride] with the query heads first")
    _need(tuple(out.shape) == (T, heads * vdim) and out.dtype == q.dtype, "out must be [T, heads * vdim]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache and activations differ in type")
    _need(tuple(k_cache.shape[-2:]) == (kv_heads, dim) and tuple(v_cache.shape[-2:]) == (kv_heads, vdim),
          "the planes must be [..., kv_heads, dim] and [..., kv_heads, vdim]")
    rows = k_cache.numel() // (kv_heads * dim)
    _need(rows == v_cache.numel() // (kv_heads * vdim), "key and value planes must hold the same number of rows")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests, "block tables must be int32 [R, width]")
    for t, n, what in ((r1, heads, "r1"), (r2, heads, "r2"), (sink, heads, "sink"), (talk, heads * heads, "talk")):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == n), f"{what} must be float32 with {n} elements")
    _need((r1 is None) == (r2 is None), "the distance bias takes r1 and r2 together")
    _need(1 <= run_keys <= SINK_DECODE_MAX_RUN and n_runs >= 1, "runs of 1 to 128 keys, at least one")
    lib = _load("sink_attention")
    need = lib.cw_sink_decode_workspace_floats(n_requests, n_runs, run_keys, heads, vdim)
    workspace = torch.empty(max(int(need), 1), dtype=torch.float32, device=q.device)
    _check(lib.cw_sink_decode(
        dtype_code(q.dtype), _ptr(q), q_stride, _ptr(out), _ptr(k_cache), _ptr(v_cache), rows, _ptr(block_tables),
        block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), n_requests, run_keys, n_runs, _ptr(workspace), _ptr(r1), _ptr(r2),
        _ptr(sink), _ptr(talk), heads, kv_heads, dim, vdim, block_size, int(window), float(scale), _stream()),
        "sink_attention_decode")


def sink_prefill_mfma_supported(heads: int, kv_heads: int, dim: int, vdim: int, dtype) -> bool:
    """Is there a matrix-core build of the sink-attention kernel for portions of this geometry?
    (bfloat16; key and value sizes of 64 or 128; up to 16 heads.)"""
    return dtype == torch.bfloat16 and bool(_load("sink_attention").cw_sink_prefill_mfma_supported(heads, kv_heads, dim, vdim))


def sink_attention_prefill(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
                           r1, r2, sink, talk, heads: int, kv_heads: int, dim: int, vdim: int, block_size: int, window: int,
                           scale: float, compute_units: int = 256) -> None:
    """``sink_attention`` on the matrix cores for bfloat16 portions: ``items`` are runs of up to
    16 tokens; a launch of fewer runs than ``compute_units`` gives each run two workgroups. Scores, softmax and the mixing across heads are float32; the mixed weights meet
    the values as two bfloat16 operands (leading bits and rest)."""
    _gpu(q, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, r1, r2, sink, talk)
    T = q.shape[0]
    _need(q.dtype == torch.bfloat16 and q.dim() == 2 and q.shape[1] == q_stride and heads * dim <= q_stride and q_stride % 8 == 0,
          "q must be bfloat16 [T, q_stride], q_stride a multiple of 8, with the query heads first")
    _need(tuple(out.shape) == (T, heads * vdim) and out.dtype == q.dtype, "out must be [T, heads * vdim]")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache and activations differ in type")
    _need(tuple(k_cache.shape[-2:]) == (kv_heads, dim) and tuple(v_cache.shape[-2:]) == (kv_heads, vdim),
          "the planes must be [..., kv_heads, dim] and [..., kv_heads, vdim]")
    rows = k_cache.numel() // (kv_heads * dim)
    _need(rows == v_cache.numel() // (kv_heads * vdim), "key and value planes must hold the same number of rows")
    R = ctx_lens.numel()
    _i32(ctx_lens, R, "ctx_lens")
    _i32(cu_q, R + 1, "cu_q")
    _i32(items, 4 * n_items, "items")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= R, "block tables must be int32 [R, width]")
    for t, n, what in ((r1, heads, "r1"), (r2, heads, "r2"), (sink, heads, "sink"), (talk, heads * heads, "talk")):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == n), f"{what} must be float32 with {n} elements")
    _need((r1 is None) == (r2 is None), "the distance bias takes r1 and r2 together")
    _check(_load("sink_attention").cw_sink_prefill_mfma(
        _ptr(q), q_stride, _ptr(out), _ptr(k_cache), _ptr(v_cache), rows, _ptr(block_tables), block_tables.shape[1],
        _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, _ptr(r1), _ptr(r2), _ptr(sink), _ptr(talk), heads, kv_heads, dim,
        vdim, block_size, int(window), float(scale), int(compute_units), _stream()), "sink_attention_prefill")


# ---------------------------------------------------------------------------------------------
class WithStreamInput:
    """A pending branch output (or None) together with a float32 stream [T, H] that joins the
    residual sum right after it: what a norm that ``accepts_stream_input`` adds before it norms.
    The model hands it to the first norm of a run entry that begins a repeated pass."""

    __slots__ = ("delta", "extra")

    def __init__(self, delta, extra) -> None:
        self.delta, self.extra = delta, extra


def add_dynamic_tanh(resid, delta, delta_scale: float, extra, weight, bias, alpha, out, rows=None) -> torch.Tensor:
    """resid += delta_scale * delta (+ extra), out = tanh(alpha * resid) * weight + bias, float32
    inside; ``alpha`` is one float32 element on the device. With ``rows`` only those rows are
    normed into out[i] and resid is left alone."""
    _gpu(resid, delta, extra, weight, bias, alpha, out, rows)
    T, H = resid.shape
    _need(resid.dtype == torch.float32, "the residual stream is float32")
    n = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "rows")
    _need(tuple(out.shape) == (n, H), f"out must be [{n}, {H}]")
    _need(weight.numel() == H and (bias is None or (bias.numel() == H and bias.dtype == weight.dtype)),
          "norm weight and bias must have the row's size and one type")
    _need(alpha.dtype == torch.float32 and alpha.numel() == 1, "alpha must be one float32 element")
    if delta is not None:
        _need(tuple(delta.shape) == (T, H) and delta.dtype == out.dtype, "the pending branch must be [T, H] in the activation type")
    if extra is not None:
        _need(tuple(extra.shape) == (T, H) and extra.dtype == torch.float32, "the stream input must be [T, H] float32")
    _check(_load("rowwise").cw_add_dyt(_ptr(resid), _ptr(delta), dtype_code(delta.dtype) if delta is not None else 0,
                                       float(delta_scale), _ptr(extra), _ptr(weight), _ptr(bias), dtype_code(weight.dtype),
                                       _ptr(alpha), _ptr(out), dtype_code(out.dtype), _ptr(rows), n, H, _stream()),
           "add_dynamic_tanh")
    return out


def linear_gelu(x: torch.Tensor, weight: torch.Tensor, policy: "ProductPolicy | None" = None) -> torch.Tensor:
    """gelu(x @ weight.T), the erf form. Few bfloat16 rows: the weight-streaming product with the
    activation in its epilogue, applied to the float32 sums (one launch); else the product and the
    activation kernel."""
    _gpu(x, weight)
    M, K = x.shape
    N = weight.shape[0]
    if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.shape[1] == K and M <= STREAM_MAX_ROWS
            and K % 8 == 0):
        lib = _load("gemm")
        if lib.cw_gemm_bf16_skinny_fast(4, M, N, K):
            out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            _check(lib.cw_gemm_bf16_skinny(4, _ptr(x), K, _ptr(weight), _ptr(out), N, M, N, K, 0, _stream()), "gemm_bf16_skinny(gelu)")
            return out
    return gelu_erf_(linear(x, weight, policy=policy))


def gelu_erf_(x: torch.Tensor) -> torch.Tensor:
    """x <- 0.5 x (1 + erf(x / sqrt 2)), in place."""
    _gpu(x)
    _check(_load("rowwise").cw_gelu_erf(_ptr(x), dtype_code(x.dtype), x.numel(), _stream()), "gelu_erf")
    return x


def sigmoid_mul_(a: torch.Tensor, z: torch.Tensor, z_off: int, group: int = 1) -> torch.Tensor:
    """a[t, j] <- a[t, j] * sigmoid(z[t, z_off + j // group]), in place on ``a`` [T, n]; ``z``
    [T, width]. ``group`` 1: a gate an element; g: one gate for every run of g elements (a head)."""
    _gpu(a, z)
    T, n = a.shape
    _need(group >= 1 and n % group == 0, "the gated runs must tile the row")
    _need(z.dim() == 2 and z.shape[0] == T and z.dtype == a.dtype and 0 <= z_off and z_off + n // group <= z.shape[1],
          "the gates must be [T, width] columns of the activations' type")
    _check(_load("rowwise").cw_sigmoid_mul(_ptr(a), _ptr(z), dtype_code(a.dtype), z.shape[1], int(z_off), T, n, int(group),
                                           _stream()), "sigmoid_mul")
    return a


def bias_store(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, nq: int, nk: int, nv: int, bias, slots,
               k_plane, v_plane) -> None:
    """Rows of ``proj`` [T, width] hold a token's query, key and value projections at the given
    columns. ``bias`` ([width] or None) is added: queries in place, keys and values into the cache
    rows ``k_plane[slots[t]]`` / ``v_plane[slots[t]]`` (flat [rows, nk] and [rows, nv]); a negative
    slot writes nothing."""
    _gpu(proj, bias, slots, k_plane, v_plane)
    T, width = proj.shape
    _i32(slots, T, "slots")
    _need(bias is None or bias.numel() == width, "the bias must have one element per column of the projection")
    _need(k_plane.dtype == proj.dtype and v_plane.dtype == proj.dtype, "cache and activations differ in type")
    _need(k_plane.numel() % nk == 0 and v_plane.numel() % nv == 0 and k_plane.numel() // nk == v_plane.numel() // nv,
          "key and value planes must hold the same number of rows")
    _check(_load("rowwise").cw_bias_store(_ptr(proj), dtype_code(proj.dtype), width, q_off, k_off, v_off, nq, nk, nv,
                                          _ptr(bias), dtype_code(bias.dtype) if bias is not None else 0, _ptr(slots),
                                          _ptr(k_plane), _ptr(v_plane), k_plane.numel() // nk, T, _stream()), "bias_store")


def latent_store(proj: torch.Tensor, dq_off: int, nq: int, dkv_off: int, rank: int, rot: int, rot_dims: int, q_weight,
                 kv_weight, eps: float, positions, freq, slots, cq: torch.Tensor, plane) -> None:
    """Rows of ``proj`` hold ``nq`` elements of a low-rank query step at ``dq_off`` and
    ``rank + rot`` elements of the key/value one at ``dkv_off``: cq[t] = RMS(dq) * q_weight; the
    cache row ``plane[slots[t]]`` ([rows, rank + rot]) gets RMS(dkv[:rank]) * kv_weight and then
    the ``rot`` other elements, the first ``rot_dims`` of them rotated by the token's position
    (half-split pairs, angle = position * freq[i], ``freq`` float32 [rot_dims / 2])."""
    _gpu(proj, q_weight, kv_weight, positions, freq, slots, cq, plane)
    T, width = proj.shape
    _i32(positions, T, "positions")
    _i32(slots, T, "slots")
    _need(tuple(cq.shape) == (T, nq) and cq.dtype == proj.dtype, "cq must be [T, nq] in the activations' type")
    _need(q_weight.numel() == nq and kv_weight.numel() == rank and q_weight.dtype == kv_weight.dtype, "norm weights must fit")
    _need(plane.dtype == proj.dtype and plane.numel() % (rank + rot) == 0, "the plane must hold rows of rank + rot elements")
    _need(rot_dims == 0 or (freq is not None and freq.dtype == torch.float32 and freq.numel() >= rot_dims // 2),
          "freq must be float32 with rot_dims / 2 elements")
    _check(_load("rowwise").cw_latent_store(_ptr(proj), dtype_code(proj.dtype), width, dq_off, nq, dkv_off, rank, rot, rot_dims,
                                            _ptr(q_weight), _ptr(kv_weight), dtype_code(q_weight.dtype), float(eps),
                                            _ptr(positions), _ptr(freq), _ptr(slots), _ptr(cq), _ptr(plane),
                                            plane.numel() // (rank + rot), T, _stream()), "latent_store")


def rotate_part(src: torch.Tensor, src_strides, src_off: int, dst: torch.Tensor, dst_strides, dst_off: int, heads: int,
                n: int, rot_dims: int, positions, freq) -> None:
    """dst(t, h, dst_off + j) = src(t, h, src_off + j) for j < n, the first ``rot_dims`` of them
    rotated by the token's position (half-split pairs, angle = position * freq[i]). Element
    (t, h, e) of a tensor lies at ``flatten()[t * strides[0] + h * strides[1] + e]``: token-major
    and head-major tensors alike."""
    _gpu(src, dst, positions, freq)
    T = positions.numel()
    _i32(positions, T, "positions")
    _need(dst.dtype == src.dtype, "src and dst must be of one type")
    for t, (st, sh), off in ((src, src_strides, src_off), (dst, dst_strides, dst_off)):
        _need(st >= 1 and sh >= 1 and off >= 0 and (T == 0 or (T - 1) * st + (heads - 1) * sh + off + n <= t.numel()),
              "rotate_part strides reach outside a tensor")
    _need(rot_dims == 0 or (freq is not None and freq.dtype == torch.float32 and freq.numel() >= rot_dims // 2),
          "freq must be float32 with rot_dims / 2 elements")
    _check(_load("rowwise").cw_rotate_part(_ptr(src), dtype_code(src.dtype), int(src_strides[0]), int(src_strides[1]), src_off,
                                           _ptr(dst), int(dst_strides[0]), int(dst_strides[1]), dst_off, heads, n, rot_dims,
                                           _ptr(positions), _ptr(freq), T, _stream()), "rotate_part")


MASK_KINDS = {"causal": 0, "window": 1, "segments": 2}


def rows_attention_supported(heads: int, kv_heads: int, dim: int, vdim: int, maps: int = 1, alias: bool = False) -> bool:
    lib = _load("rows_attention")
    return bool(lib.cw_rows_attention_key_chunk(maps, dim, vdim, int(alias))
                and lib.cw_rows_attention_heads_per_group(heads, kv_heads, maps))


def rows_attention_tokens_per_item(heads: int, kv_heads: int, maps: int = 1) -> int:
    """Tokens of one request that a work item of ``rows_attention`` may hold."""
    return int(_load("rows_attention").cw_rows_attention_tokens_per_item(heads, kv_heads, maps))


ROWS_MFMA_TOKENS = 16   # tokens of one request that a work item of the matrix-core kernel holds


def rows_mfma_supported(dim: int, vdim: int, maps: int, dtype, alias: bool = False) -> bool:
    """Does the matrix-core kernel take this geometry? bfloat16; one or two maps with key rows of 64
    or 128 elements a map and value rows of 64, 128 or 256; or one map whose values lie inside the
    key row (``alias``): key rows of 160, 320 or 576 elements, values their first 128, 256 or 512."""
    return dtype == torch.bfloat16 and bool(_load("rows_attention").cw_rows_mfma_supported(maps, dim, vdim, int(alias)))


def rows_mfma_key_runs(n_items: int, longest: int, heads: int, kv_heads: int, dim: int, vdim: int, maps: int,
                       compute_units: int, alias: bool = False) -> int:
    """Into how many runs the matrix-core kernel cuts every item's keys: as many as there are idle
    compute units for while the longest key range gives each run 128 keys, 64 at most (a step of
    single tokens, or a short portion behind a long context, would leave most of the card idle)."""
    per_run = n_items * int(_load("rows_attention").cw_rows_mfma_grid_y(heads, kv_heads, maps, dim, vdim, int(alias)))
    if per_run <= 0:
        return 1
    return int(max(1, min(compute_units // per_run, longest // 128, 64)))


def heads_linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[h] = x[h] @ weight[h].T for every head: ``x`` [heads, T, n_in], ``weight``
    [heads, n_out, n_in], ``out`` [heads, T, n_out]; x and out may be views whose rows lie apart
    (a slice of each head's columns), their last dimension dense. The library's batched product,
    float32 accumulation (full float32 for float32 operands), always with the library's default
    kernel: its tuner times candidates on copies of the operands that it sizes as
    max(batch stride, rows * columns) * batch elements, which a slice of wider rows outgrows (rows
    lie a whole token apart, heads a few columns), so a tuning run would read past its copy."""
    _need(x.dim() == 3 and weight.dim() == 3 and out.dim() == 3 and x.shape[0] == weight.shape[0] == out.shape[0]
          and x.shape[2] == weight.shape[2] and out.shape[2] == weight.shape[1] and x.shape[1] == out.shape[1],
          "heads_linear shapes")
    _need(x.dtype == weight.dtype == out.dtype and x.stride(2) == 1 and out.stride(2) == 1, "heads_linear types and strides")
    if x.shape[1]:
        import torch.cuda.tunable as tunable

        tuning = tunable.is_enabled() and tunable.tuning_is_enabled()
        if tuning:
            tunable.tuning_enable(False)
        try:
            torch.bmm(x, weight.transpose(1, 2), out=out)
        finally:
            if tuning:
                tunable.tuning_enable(True)
    return out


def rows_attention(q, q_strides, out, out_strides, k_plane, v_plane, block_tables, ctx_lens, cu_q, items, n_items: int,
                   heads: int, kv_heads: int, dim: int, vdim: int, block_size: int, scale: float, maps: int = 1,
                   mask: str = "causal", mask_size: int = 0, sink=None, lam=None, head_norm_eps=None,
                   post_mult: float = 1.0, mfma: bool = False, key_runs: int = 1, keep_first: int = 0,
                   softcap: float = 0.0, head_gate=None) -> None:
    """Softmax attention of the step's queries over paged rows. Query (t, head, map, d) lies at
    ``q.flatten()[t * q_strides[0] + head * q_strides[1] + map * dim + d]``, output (t, head, c) at
    ``out.flatten()[t * out_strides[0] + head * out_strides[1] + c]`` (token-major or head-major
    tensors alike). ``k_plane`` [rows, >= kv_heads * maps * dim] holds a
    token's keys [kv head][map][dim]; ``v_plane`` [rows, >= kv_heads * vdim] its values, or None:
    the values are the first ``vdim`` elements of the key row (``maps`` 1).
    ``mask``: "causal", "window" (the ``mask_size`` latest positions) or "segments" (the earlier
    tokens of the token's segment of ``mask_size`` positions, segments counted from position 0).
    ``keep_first`` n (with a window): the request's first n positions stay visible to every later
    token. ``softcap`` c > 0: scores are squashed, c * tanh(scale * q . k / c), before the softmax.
    ``head_gate`` (z, offset): head h of token t is multiplied by logistic(z[t, offset + h]), z [T, width]
    in the queries' type. ``sink`` float32 [heads]: exp(sink) joins the denominator. ``maps`` 2: the head's output is
    map 0 minus ``lam`` (one float32 element) times map 1. ``head_norm_eps`` not None: the head's
    output is divided by its root mean square and multiplied by ``post_mult``. ``items`` int32
    [n_items, 4]: (request, first token, tokens, 0) with at most
    ``rows_attention_tokens_per_item`` tokens each. ``mfma``: the matrix-core kernel
    (``rows_mfma_supported``; items of up to ``ROWS_MFMA_TOKENS`` tokens), every item's keys cut
    into ``key_runs`` runs that a second kernel puts together."""
    alias = v_plane is None
    _gpu(q, out, k_plane, v_plane, block_tables, ctx_lens, cu_q, items, sink, lam)
    qs, qh = int(q_strides[0]), int(q_strides[1])
    os_, oh = int(out_strides[0]), int(out_strides[1])
    _need(out.dtype == q.dtype, "queries and output differ in type")
    # the furthest element a token row of the step can touch must lie inside the tensors
    def _fits(t, tok_stride, head_stride, width, tokens):
        return tokens == 0 or (tokens - 1) * tok_stride + (heads - 1) * head_stride + width <= t.numel()
    tokens = out.numel() // (heads * vdim)
    _need(_fits(q, qs, qh, maps * dim, tokens) and _fits(out, os_, oh, vdim, tokens), "q / out strides reach outside the tensors")
    k2 = k_plane.reshape(k_plane.shape[0], -1)
    _need(k2.dtype == q.dtype and k2.shape[1] >= kv_heads * maps * dim, "the key plane must be [rows, >= kv_heads * maps * dim]")
    rows = k2.shape[0]
    v_row = 0
    if not alias:
        v2 = v_plane.reshape(v_plane.shape[0], -1)
        _need(v2.dtype == q.dtype and v2.shape[0] == rows and v2.shape[1] >= kv_heads * vdim,
              "the value plane must be [rows, >= kv_heads * vdim]")
        v_row = v2.shape[1]
    else:
        _need(maps == 1 and kv_heads == 1 and vdim <= dim, "values inside the key row: one map, one key/value head, vdim <= dim")
    R = ctx_lens.numel()
    _i32(ctx_lens, R, "ctx_lens")
    _i32(cu_q, R + 1, "cu_q")
    _i32(items, 4 * n_items, "items")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= R, "block tables must be int32 [R, width]")
    _need(sink is None or (sink.dtype == torch.float32 and sink.numel() == heads), f"sink must be float32 with {heads} elements")
    _need((maps == 1 and lam is None) or (maps == 2 and lam is not None and lam.dtype == torch.float32 and lam.numel() == 1),
          "two maps take one float32 lambda, one map none")
    _need(mask in MASK_KINDS and (mask == "causal" or mask_size >= 1), f"mask {mask!r} of size {mask_size}")
    _need(keep_first >= 0 and (keep_first == 0 or mask == "window"), "first positions are kept visible behind a window only")
    _need(softcap >= 0.0, "a score cap is positive (0: none)")
    gate, gate_stride, gate_off = None, 0, 0
    if head_gate is not None:
        gate, gate_off = head_gate
        _gpu(gate)
        _need(gate.dim() == 2 and gate.dtype == q.dtype and gate.shape[0] >= tokens and gate.is_contiguous()
              and 0 <= gate_off and gate_off + heads <= gate.shape[1], "the gates must be [T, width] with a column a head")
        gate_stride = gate.shape[1]
    if mfma:
        lib = _load("rows_attention")
        _need(rows_mfma_supported(dim, vdim, maps, q.dtype, alias), "the matrix-core kernel does not take this geometry")
        need = int(lib.cw_rows_mfma_workspace_floats(n_items, heads, kv_heads, maps, dim, vdim, int(alias), key_runs))
        workspace = torch.empty(need, dtype=torch.float32, device=q.device) if need else None
        _check(lib.cw_rows_attention_mfma(
            _ptr(q), qs, qh, _ptr(out), os_, oh, _ptr(k_plane), _ptr(k_plane if alias else v_plane), k2.shape[1], v_row, rows,
            _ptr(block_tables), block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, _ptr(sink), _ptr(lam),
            heads, kv_heads, dim, vdim, maps, block_size, MASK_KINDS[mask], int(mask_size), float(scale),
            0 if head_norm_eps is None else 1, float(head_norm_eps or 0.0), float(post_mult), int(key_runs), _ptr(workspace), need,
            int(keep_first), float(softcap), _ptr(gate), int(gate_stride), int(gate_off), _stream()), "rows_attention_mfma")
        return
    _check(_load("rows_attention").cw_rows_attention(
        dtype_code(q.dtype), _ptr(q), qs, qh, _ptr(out), os_, oh, _ptr(k_plane), _ptr(k_plane if alias else v_plane), k2.shape[1],
        v_row, rows, _ptr(block_tables), block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, _ptr(sink),
        _ptr(lam), heads, kv_heads, dim, vdim, maps, block_size, MASK_KINDS[mask], int(mask_size), float(scale),
        0 if head_norm_eps is None else 1, float(head_norm_eps or 0.0), float(post_mult), int(keep_first), float(softcap),
        _ptr(gate), int(gate_stride), int(gate_off), _stream()), "rows_attention")


# ---------------------------------------------------------------------------------------------
class StreamImage:
    """The residual stream as it stands, in the activation type: what a block whose sublayers read
    the stream itself hands on instead of a pending branch output (nothing is left to add)."""

    __slots__ = ("image",)

    def __init__(self, image) -> None:
        self.image = image


def branch_norm_add(resid, branch, weight, weight_offset: float, eps: float, scale: float, image=None):
    """resid += scale * branch / sqrt(mean(branch^2) + eps) * (weight_offset + weight), float32
    inside; ``image`` ([T, H] in the activation type, or None) receives the stream after that.
    ``branch`` None: nothing is added (the image alone is made)."""
    _gpu(resid, branch, weight, image)
    T, H = resid.shape
    _need(resid.dtype == torch.float32, "the residual stream is float32")
    act = branch if branch is not None else image
    _need(act is not None, "a branch or an image, or both")
    if branch is not None:
        _need(tuple(branch.shape) == (T, H), "the branch must be [T, H]")
        _need(weight is not None and weight.numel() == H, "the norm's weight must have the row's size")
    if image is not None:
        _need(tuple(image.shape) == (T, H) and image.dtype == act.dtype, "the image must be [T, H] in the activation type")
    _check(_load("rowwise").cw_branch_norm_add(_ptr(resid), _ptr(branch), _ptr(weight),
                                               dtype_code(weight.dtype) if weight is not None else 0, float(weight_offset),
                                               float(eps), float(scale), _ptr(image), dtype_code(act.dtype), T, H, _stream()),
           "branch_norm_add")
    return image


def stream_norm(resid, weight, weight_offset: float, eps: float, out, rows=None) -> torch.Tensor:
    """out[i] = resid[r] / sqrt(mean(resid[r]^2) + eps) * (weight_offset + weight), r = rows[i] (or i),
    the product in float32 and rounded once; the stream is left as it is."""
    _gpu(resid, weight, out, rows)
    T, H = resid.shape
    _need(resid.dtype == torch.float32, "the residual stream is float32")
    n = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "rows")
    _need(tuple(out.shape) == (n, H) and weight.numel() == H, f"out must be [{n}, {H}], the weight [{H}]")
    _check(_load("rowwise").cw_stream_norm(_ptr(resid), _ptr(weight), dtype_code(weight.dtype), float(weight_offset), float(eps),
                                           _ptr(out), dtype_code(out.dtype), _ptr(rows), n, H, _stream()), "stream_norm")
    return out


HEAD_PAIRINGS = {"halves": 0, "neighbours": 1}
HEAD_NORMS = {"none": 0, "before": 1, "after": 2}


def headnorm_rope_store(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, n_q_vectors: int, n_k_vectors: int, dim: int,
                        nv: int, bias, q_weight, k_weight, eps: float, positions, freq, rot_dims: int, slots, k_plane,
                        v_plane, values_from_keys: bool = False, pairing: str = "halves", norm=None,
                        query_temperature=None) -> None:
    """Rows of ``proj`` [T, width] hold a token's query vectors (``n_q_vectors`` of ``dim`` elements
    from column q_off), key vectors (``n_k_vectors`` from k_off) and value projection (``nv``
    elements from v_off). ``bias`` ([width] or None) is added; every query and key vector by itself
    is divided by its root mean square and multiplied by ``q_weight`` / ``k_weight`` ([dim], both or
    neither), its first ``rot_dims`` elements rotated by the token's position (half-split pairs,
    angle = position * freq[i], ``freq`` float32 [rot_dims / 2]). Queries are rewritten in place,
    keys go to ``k_plane[slots[t]]``, values to ``v_plane[slots[t]]``: the biased value projection,
    or with ``values_from_keys`` the biased key projection before norm and rotation. ``slots``
    None or a negative slot: no cache row is written.

    ``pairing`` "neighbours": elements 2i and 2i + 1 turn together by freq[i] (instead of i and
    i + rot_dims / 2). ``norm``: "before" (the norm, then the rotation), "after" (the rotated vector is
    divided by its own root mean square), "none"; None: "before" if weights are given, else
    "none". The weights may be absent with either norm. ``query_temperature`` (coef, every): every
    query is multiplied, last, by 1 + coef * ln(floor((position + 1) / every) + 1)."""
    _gpu(proj, bias, q_weight, k_weight, positions, freq, slots, k_plane, v_plane)
    T, width = proj.shape
    if positions is not None:
        _i32(positions, T, "positions")
    if slots is not None:
        _i32(slots, T, "slots")
    _need(bias is None or bias.numel() == width, "the bias must have one element per column of the projection")
    _need((q_weight is None) == (k_weight is None), "norm weights for queries and keys, or for neither")
    if q_weight is not None:
        _need(q_weight.numel() == dim and k_weight.numel() == dim and q_weight.dtype == k_weight.dtype, "norm weights must be [dim]")
    _need(rot_dims == 0 or (freq is not None and positions is not None and freq.dtype == torch.float32
                            and freq.numel() >= rot_dims // 2), "freq must be float32 with rot_dims / 2 elements")
    _need(pairing in HEAD_PAIRINGS, f"pairing {pairing!r}: expected one of {sorted(HEAD_PAIRINGS)}")
    if norm is None:
        norm = "before" if q_weight is not None else "none"
    _need(norm in HEAD_NORMS and (norm != "none" or q_weight is None), f"norm {norm!r}: 'before', 'after' or 'none' (which takes no weights)")
    coef, every = query_temperature if query_temperature is not None else (0.0, 0)
    _need(int(every) >= 0 and (int(every) == 0 or positions is not None), "a query temperature needs positions and a positive period")
    rows = 0
    if slots is not None:
        nk = n_k_vectors * dim
        _need(k_plane is not None and k_plane.dtype == proj.dtype and k_plane.numel() % nk == 0, "the key plane must hold rows of the keys' width")
        rows = k_plane.numel() // nk
        _need(nv == 0 or (v_plane is not None and v_plane.dtype == proj.dtype and v_plane.numel() == rows * nv),
              "key and value planes must hold the same number of rows")
    _check(_load("rowwise").cw_headnorm_rope_store(
        _ptr(proj), dtype_code(proj.dtype), width, int(q_off), int(k_off), int(v_off), int(n_q_vectors), int(n_k_vectors), int(dim),
        int(nv), _ptr(bias), dtype_code(bias.dtype) if bias is not None else 0, _ptr(q_weight), _ptr(k_weight),
        dtype_code(q_weight.dtype) if q_weight is not None else 0, float(eps), _ptr(positions), _ptr(freq), int(rot_dims),
        _ptr(slots), _ptr(k_plane), _ptr(v_plane), int(bool(values_from_keys)), rows, T, HEAD_PAIRINGS[pairing], HEAD_NORMS[norm],
        float(coef), int(every), _stream()), "headnorm_rope_store")


def relu_squared_(x: torch.Tensor) -> torch.Tensor:
    """x <- max(x, 0)^2, in place."""
    _gpu(x)
    _check(_load("rowwise").cw_relu_squared(_ptr(x), dtype_code(x.dtype), x.numel(), _stream()), "relu_squared")
    return x


def linear_relu_squared(x: torch.Tensor, weight: torch.Tensor, policy: "ProductPolicy | None" = None) -> torch.Tensor:
    """max(x @ weight.T, 0)^2. Few bfloat16 rows: the weight-streaming product with the activation
    in its epilogue, applied to the float32 sums (one launch); else the product, then the
    activation in place."""
    _gpu(x, weight)
    M, K = x.shape
    N = weight.shape[0]
    if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.shape[1] == K and M <= STREAM_MAX_ROWS
            and K % 8 == 0):
        lib = _load("gemm")
        if lib.cw_gemm_bf16_skinny_fast(5, M, N, K):
            out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            _check(lib.cw_gemm_bf16_skinny(5, _ptr(x), K, _ptr(weight), _ptr(out), N, M, N, K, 0, _stream()), "gemm_bf16_skinny(relu2)")
            return out
    # a long portion: the wide-tile kernel with the activation in its epilogue, from the sizes at
    # which it takes the gate/up product of a gated feed-forward (the same kernel, the same gain)
    if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.shape[1] == K and M >= WIDE_SWIGLU_MIN_ROWS
            and x.stride(1) == 1 and x.stride(0) % 8 == 0 and weight.is_contiguous()):
        lib = _load("gemm_tile")
        if lib.cw_gemm_bf16_wide_tiles(5, M, N, K, x.stride(0)) >= WIDE_SWIGLU_MIN_TILES:
            out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            _check(lib.cw_gemm_bf16_wide(5, _ptr(x), x.stride(0), _ptr(weight), None, 0, _ptr(out), N, M, N, K,
                                         _compute_units(x.device), _stream()), "gemm_bf16_wide(relu2)")
            return out
    return relu_squared_(linear(x, weight, policy=policy))


def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    """x <- s * x, in place on float32 (logits)."""
    _gpu(x)
    _need(x.dtype == torch.float32, "scale_ takes float32")
    _check(_load("rowwise").cw_scale(_ptr(x), x.numel(), float(s), _stream()), "scale")
    return x


# ---------------------------------------------------------------------------------------------
ROUTER_KINDS = {"sigmoid": 0, "softmax": 1}


def moe_route(x: torch.Tensor, router: torch.Tensor, top: int, kind: str = "sigmoid", renormalize: bool = False,
              correction=None, groups=None, extra: int = 0, renorm_eps: float = 0.0):
    """(choice int32 [T, top], score float32 [T, top]): the ``top`` experts with the largest
    logistic (or softmax) of router x, the lower index first among equals, in falling order;
    ``renormalize``: the chosen scores are divided by their sum (plus ``renorm_eps``). float32 sums.

    ``correction`` float32 [experts]: added to the scores for the choice only. ``groups``
    (count, kept, top): the experts lie in ``count`` equal runs of neighbours, a run's score is the
    sum of its ``top`` largest choice scores, and only experts of the ``kept`` best runs can be
    chosen. ``extra`` n: the router's matrix has n more rows behind the experts' (gates that
    read the same input); their logistic values come back as a third result, float32 [T, n]."""
    _gpu(x, router, correction)
    T, H = x.shape
    E = router.shape[0] - int(extra)
    _need(router.dim() == 2 and router.shape[1] == H and router.dtype == x.dtype and extra >= 0 and E >= 1,
          "the router must be [experts (+ extra), H] in x's type")
    _need(1 <= top <= E and kind in ROUTER_KINDS, f"top {top} of {E} experts, router kind {kind!r}")
    _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == E), "the correction must be float32 [experts]")
    count, kept, run_top = groups if groups is not None else (1, 1, 1)
    _need(count >= 1 and E % count == 0 and 1 <= kept <= count and run_top >= 1 and (E // count) * kept >= top,
          f"{E} experts in {count} runs of which {kept} are kept cannot give {top} experts")
    choice = torch.empty((T, top), dtype=torch.int32, device=x.device)
    score = torch.empty((T, top), dtype=torch.float32, device=x.device)
    gates = torch.empty((T, extra), dtype=torch.float32, device=x.device) if extra else None
    _check(_load("moe").cw_moe_route(_ptr(x), _ptr(router), dtype_code(x.dtype), T, H, E, top, ROUTER_KINDS[kind],
                                     int(bool(renormalize)), _ptr(choice), _ptr(score), _ptr(correction), int(count), int(kept),
                                     int(run_top), int(extra), _ptr(gates), float(renorm_eps), _stream()), "moe_route")
    return (choice, score, gates) if extra else (choice, score)


MOE_KERNELS = {"plain": 0, "stream": 1, "wide": 2, "grouped": 3}
# rows an expert from which a step's experts run on the wide tiles of the matrix-core kernel
MOE_WIDE_FROM = 48
# rows an expert from which they run as row tiles of the dense products' wide-tile kernel
MOE_GROUPED_FROM = 256


def moe_kernel_for(dtype, n_pairs: int, experts: int, hidden: int, ff: int) -> str:
    """Which kernel runs the experts' products of a step: by type, sizes and the step's shape alone
    (never by what the router chose), so a captured step replays. bfloat16 with widths that are a
    multiple of 8 runs on the matrix cores: "wide" tiles of 128 rows from ``MOE_WIDE_FROM`` rows an
    expert on average, else "stream" (tiles of 16 rows, the expert's matrix read once a tile);
    from ``MOE_GROUPED_FROM`` rows an expert, with widths that are a multiple of 64 and at least 256,
    "grouped": the rows laid out expert by expert in tiles of 256 and multiplied by the kernel of
    the dense products of long portions, every row tile with its expert's matrix. Everything else,
    float32 included, "plain" arithmetic."""
    if dtype != torch.bfloat16 or hidden % 8 or ff % 8:
        return "plain"
    grouped_rows = (n_pairs // 256 + min(n_pairs, experts)) * 256   # the most rows its tiles can hold
    if n_pairs >= MOE_GROUPED_FROM * experts and moe_grouped_ok(hidden, ff) and grouped_rows * max(hidden, ff) * 2 < 2 ** 32:
        return "grouped"
    return "wide" if n_pairs >= MOE_WIDE_FROM * experts else "stream"


def moe_grouped_ok(hidden: int, ff: int) -> bool:
    """Does the grouped product take experts of these widths (both are a K of one of its products)?"""
    return min(hidden, ff) >= 256 and hidden % 64 == 0 and ff % 64 == 0 and 2 * ff * hidden * 2 < 2 ** 32


class ExpertRows:
    """The (token, choice) pairs of a step sorted by expert (``moe_plan``): ``row_pair`` int32
    [max_rows] (pair index or -1), ``tile_expert`` int32 [max_tiles], ``n_tiles`` int32 [1], all on
    the device; every tile of ``tile_rows`` rows belongs to one expert. ``kernel`` names the kernel
    whose tiles these are."""

    __slots__ = ("row_pair", "tile_expert", "n_tiles", "max_tiles", "max_rows", "n_pairs", "kernel", "tile_rows")


def moe_plan(choice: torch.Tensor, experts: int, kernel: str = "plain") -> ExpertRows:
    _gpu(choice)
    _need(choice.dtype == torch.int32, "choices are int32")
    _need(kernel in MOE_KERNELS, f"kernel {kernel!r}: one of {sorted(MOE_KERNELS)}")
    lib = _load("moe")
    plan = ExpertRows()
    plan.kernel = kernel
    plan.tile_rows = int(lib.cw_moe_tile_rows(MOE_KERNELS[kernel]))
    plan.n_pairs = choice.numel()
    plan.max_tiles = int(lib.cw_moe_max_tiles(plan.n_pairs, experts, plan.tile_rows))
    plan.max_rows = plan.max_tiles * plan.tile_rows
    plan.row_pair = torch.empty(max(plan.max_rows, 1), dtype=torch.int32, device=choice.device)
    plan.tile_expert = torch.empty(max(plan.max_tiles, 1), dtype=torch.int32, device=choice.device)
    plan.n_tiles = torch.empty(1, dtype=torch.int32, device=choice.device)
    _check(lib.cw_moe_plan(_ptr(choice), plan.n_pairs, experts, plan.tile_rows, _ptr(plan.row_pair), plan.max_rows,
                           _ptr(plan.tile_expert), plan.max_tiles, _ptr(plan.n_tiles), _stream()), "moe_plan")
    return plan


def moe_gate_up(x: torch.Tensor, gate_up: torch.Tensor, plan: ExpertRows, score: torch.Tensor, top: int,
                scale_input: bool) -> torch.Tensor:
    """inner [max_rows, ff] = silu(gate_e u) * (up_e u) for every row of the plan, u the row's token
    of ``x`` [T, H] (times the pair's score, rounded to x's type, with ``scale_input``); ``gate_up``
    [experts, 2 * ff, H], gate rows first. Rows that hold no pair are zero."""
    _gpu(x, gate_up, score)
    T, H = x.shape
    _need(gate_up.dim() == 3 and gate_up.shape[2] == H and gate_up.shape[1] % 2 == 0 and gate_up.dtype == x.dtype,
          "gate_up must be [experts, 2 * ff, H] in x's type")
    _need(plan.n_pairs == T * top and score.numel() == T * top and score.dtype == torch.float32, "one score a pair")
    ff = gate_up.shape[1] // 2
    inner = torch.empty((max(plan.max_rows, 1), ff), dtype=x.dtype, device=x.device)
    if plan.kernel == "grouped":
        _need(x.dtype == torch.bfloat16 and moe_grouped_ok(H, ff), "the grouped product takes bfloat16 and widths that are a multiple of 64")
        rows = torch.empty((max(plan.max_rows, 1), H), dtype=x.dtype, device=x.device)
        _check(_load("moe").cw_moe_gather(_ptr(x), _ptr(rows), dtype_code(x.dtype), _ptr(plan.row_pair), _ptr(plan.n_tiles),
                                          plan.max_tiles, plan.tile_rows, _ptr(score), top, H, int(bool(scale_input)), _stream()),
               "moe_gather")
        _check(_load("gemm_tile").cw_gemm_bf16_wide_grouped(2, _ptr(rows), H, _ptr(gate_up), gate_up.stride(0), _ptr(inner), ff,
                                                            2 * ff, H, _ptr(plan.tile_expert), _ptr(plan.n_tiles), plan.max_tiles,
                                                            None, None, _compute_units(x.device), _stream()), "moe_gate_up")
        return inner
    _check(_load("moe").cw_moe_expert_product(0, MOE_KERNELS[plan.kernel], _ptr(x), _ptr(gate_up), _ptr(inner), dtype_code(x.dtype), _ptr(plan.row_pair),
                                              _ptr(plan.tile_expert), _ptr(plan.n_tiles), plan.max_tiles, _ptr(score), top, H, ff,
                                              int(bool(scale_input)), _stream()), "moe_gate_up")
    return inner


def moe_down(inner: torch.Tensor, down: torch.Tensor, plan: ExpertRows, score: torch.Tensor, top: int, scale_output: bool,
             out: torch.Tensor) -> torch.Tensor:
    """out[pair] = down_e inner[row] for every row that holds a pair (times the pair's score with
    ``scale_output``); ``down`` [experts, H, ff], ``out`` [pairs, H]."""
    _gpu(inner, down, score, out)
    ff = inner.shape[1]
    _need(down.dim() == 3 and down.shape[2] == ff and down.dtype == inner.dtype, "down must be [experts, H, ff] in the rows' type")
    H = down.shape[1]
    _need(inner.shape[0] >= plan.max_rows and tuple(out.shape) == (plan.n_pairs, H) and out.dtype == inner.dtype, "out must be [pairs, H]")
    if plan.kernel == "grouped":
        _need(inner.dtype == torch.bfloat16 and moe_grouped_ok(H, ff) and inner.is_contiguous(), "the grouped product takes bfloat16 and widths that are a multiple of 64")
        _check(_load("gemm_tile").cw_gemm_bf16_wide_grouped(0, _ptr(inner), ff, _ptr(down), down.stride(0), _ptr(out), H, H, ff,
                                                            _ptr(plan.tile_expert), _ptr(plan.n_tiles), plan.max_tiles,
                                                            _ptr(plan.row_pair), _ptr(score) if scale_output else None,
                                                            _compute_units(inner.device), _stream()), "moe_down")
        return out
    _check(_load("moe").cw_moe_expert_product(1, MOE_KERNELS[plan.kernel], _ptr(inner), _ptr(down), _ptr(out), dtype_code(inner.dtype), _ptr(plan.row_pair),
                                              _ptr(plan.tile_expert), _ptr(plan.n_tiles), plan.max_tiles, _ptr(score), top, ff, H,
                                              int(bool(scale_output)), _stream()), "moe_down")
    return out


def moe_combine(y: torch.Tensor, top: int, out: torch.Tensor, always=None, always_gate=None) -> torch.Tensor:
    """out[t] = y[t * top] + ... + y[t * top + top - 1], added in that order in float32; then
    ``always`` [T, H] (the output of an expert that every token uses) joins, times
    ``always_gate[t, 0]`` (float32 [T, n]) if given."""
    _gpu(y, out, always, always_gate)
    T, H = out.shape
    _need(tuple(y.shape) == (T * top, H) and y.dtype == out.dtype, "y must be [T * top, H]")
    _need(always is None or (tuple(always.shape) == (T, H) and always.dtype == out.dtype and always.is_contiguous()),
          "the expert of every token must be [T, H] in the output's type")
    stride = 0
    if always_gate is not None:
        _need(always is not None and always_gate.dtype == torch.float32 and always_gate.dim() == 2 and always_gate.shape[0] == T
              and always_gate.is_contiguous(), "the gate must be float32 [T, n]")
        stride = always_gate.shape[1]
    _check(_load("moe").cw_moe_combine(_ptr(y), _ptr(out), dtype_code(out.dtype), T, top, H, _ptr(always), _ptr(always_gate),
                                       int(stride), _stream()), "moe_combine")
    return out
