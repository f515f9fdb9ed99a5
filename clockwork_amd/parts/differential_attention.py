"""Attention with two score maps a head over shared values (``DifferentialAttentionSpec``).

Steps: one fused q/k/v product; one kernel adds the biases, rewrites the queries and writes keys
and values to their pages (every token of the step is cached before any query reads; with
``qk_norm`` or a position encoding the same kernel norms every query and key vector, each map of
each head by itself, and rotates it by the token's position); the
attention kernel runs both maps of a head in one workgroup, subtracts the second from the first
with the layer's lambda, norms the head's output and scales it; output product. Keys
[kv_heads, 2, key_dim] and values [kv_heads, value_dim] are two planes of a ``PagedRowsSpec``;
with a segment mask the pages before the running segment are given back while the request runs.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import PagedRowsSpec, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.sink_attention import longest_key_range, query_runs
from clockwork_amd.parts.specs import DifferentialAttentionSpec

MAPS = 2


class DifferentialAttention(Part):
    graph_safe = True

    def __init__(self, spec: DifferentialAttentionSpec) -> None:
        self.spec = spec
        self.q_width = spec.num_heads * MAPS * spec.key_dim
        self.k_width = spec.num_kv_heads * MAPS * spec.key_dim
        self.v_width = spec.num_kv_heads * spec.value_dim

    def param_specs(self):
        s = self.spec
        width = self.q_width + self.k_width + self.v_width
        specs = {
            "qkv_weight": ParamSpec((width, s.hidden_size)),
            "out_weight": ParamSpec((s.hidden_size, s.num_heads * s.value_dim)),
        }
        if s.qkv_bias:
            specs["qkv_bias"] = ParamSpec((width,), precision="stored", init=("normal", 0.02))
        if s.out_bias:
            specs["out_bias"] = ParamSpec((s.hidden_size,), precision="compute", init=("normal", 0.02))
        if s.qk_norm:
            specs["q_norm"] = ParamSpec((s.key_dim,), precision="stored", init=("one_plus_uniform", 0.3))
            specs["k_norm"] = ParamSpec((s.key_dim,), precision="stored", init=("one_plus_uniform", 0.3))
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = ParamSpec((s.key_dim,), precision="float32", init=("normal", 0.1))
        return specs

    def cache_need(self):
        s = self.spec
        return PagedRowsSpec((("k", (s.num_kv_heads, MAPS * s.key_dim)), ("v", (s.num_kv_heads, s.value_dim))),
                             window=s.window, segment=s.segment)

    def kernel_libraries(self) -> list:
        return [("rowwise", None), ("rows_attention", None)]

    def mask(self) -> tuple:
        s = self.spec
        if s.segment is not None:
            return "segments", s.segment
        return ("window", s.window) if s.window is not None else ("causal", 0)

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        self.qkv_weight, self.qkv_bias = params["qkv_weight"], params.get("qkv_bias")
        self.out_weight, self.out_bias = params["out_weight"], params.get("out_bias")
        self.q_norm, self.k_norm = params.get("q_norm"), params.get("k_norm")
        # rotation frequencies base^(-2i / n), made on the host in float64 and rounded once
        self.rot_dims = s.position.rotary_dim if s.position is not None else 0
        self.freq = None
        if self.rot_dims:
            freq = torch.tensor([float(s.position.theta) ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)],
                                dtype=torch.float64)
            self.freq = freq.to(torch.float32).to(device)
        # lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init: one float32 number a layer
        lam = (torch.exp((params["lq1"].float() * params["lk1"].float()).sum())
               - torch.exp((params["lq2"].float() * params["lk2"].float()).sum()) + s.lambda_init)
        self.lam = lam.reshape(1).to(device=device, dtype=torch.float32).contiguous()
        self.dtype = dtype
        if not ops.rows_attention_supported(s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, maps=MAPS):
            raise ValueError(f"two-map attention with keys of {s.key_dim} and values of {s.value_dim} elements is beyond "
                             "the attention kernel for paged rows (value_dim up to 512, tiles of 150 KB of LDS)")
        # bfloat16 with the common head sizes runs on the matrix cores (16-byte loads: rows begin at multiples of 8)
        self.mfma = (ops.rows_mfma_supported(s.key_dim, s.value_dim, MAPS, dtype)
                     and (self.q_width + self.k_width + self.v_width) % 8 == 0)
        self.run = ops.ROWS_MFMA_TOKENS if self.mfma else ops.rows_attention_tokens_per_item(s.num_heads, s.num_kv_heads, MAPS)

    def _plan(self, ctx):
        """(work items, their number, runs that every item's keys are cut into)."""
        s = self.spec
        key = ("two-map attention", s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, s.segment, s.window, self.mfma)
        plan = ctx.plans.get(key)
        if plan is None:
            items, n_items = query_runs(ctx, self.run)
            runs = 1
            if self.mfma:
                runs = ops.rows_mfma_key_runs(n_items, longest_key_range(ctx, s.window, s.segment), s.num_heads, s.num_kv_heads,
                                              s.key_dim, s.value_dim, MAPS, ctx.num_compute_units)
            plan = ctx.plans[key] = (items, n_items, runs)
        return plan

    def prepare(self, ctx) -> None:
        self._plan(ctx)

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        if not cache.writes:
            raise NotImplementedError("this mixer writes its own keys and values: it cannot borrow another entry's cache")
        k_plane, v_plane = cache.planes["k"], cache.planes["v"]
        qkv = ops.linear(x, self.qkv_weight, policy=policy)
        if s.qk_norm or self.rot_dims:
            ops.headnorm_rope_store(qkv, 0, self.q_width, self.q_width + self.k_width, s.num_heads * MAPS, s.num_kv_heads * MAPS,
                                    s.key_dim, self.v_width, self.qkv_bias, self.q_norm, self.k_norm, s.norm_eps, ctx.positions,
                                    self.freq, self.rot_dims, ctx.slots[cache.group], k_plane, v_plane)
        else:
            ops.bias_store(qkv, 0, self.q_width, self.q_width + self.k_width, self.q_width, self.k_width, self.v_width,
                           self.qkv_bias, ctx.slots[cache.group], k_plane, v_plane)
        out = torch.empty((x.shape[0], s.num_heads * s.value_dim), dtype=x.dtype, device=x.device)
        items, n_items, runs = self._plan(ctx)
        kind, size = self.mask()
        ops.rows_attention(qkv, (qkv.shape[1], MAPS * s.key_dim), out, (out.shape[1], s.value_dim), k_plane, v_plane,
                           ctx.block_tables[cache.group], ctx.ctx_lens, ctx.cu_q, items, n_items, s.num_heads, s.num_kv_heads,
                           s.key_dim, s.value_dim, cache.block_size, s.scale, maps=MAPS, mask=kind, mask_size=size, lam=self.lam,
                           head_norm_eps=s.norm_eps, post_mult=1.0 - s.lambda_init, mfma=self.mfma, key_runs=runs)
        return ops.linear(out, self.out_weight, self.out_bias, policy=policy)
