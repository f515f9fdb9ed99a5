"""Grouped attention with per-head query/key norms, values that may be the keys themselves and an
output gate (``GatedAttentionSpec``).

Steps: one fused product for queries, keys, values (if they have a projection of their own) and
the gate; one kernel adds the biases, norms every head's query and key vector, rotates them by the
token's position, rewrites the queries and writes keys and values to their pages (every token of
the step is cached before any query reads; with ``values="keys"`` the value row is the key
projection as it left the product); attention over the paged rows; the heads times the logistic
function of the gate columns; output product. Keys [kv_heads, key_dim] and values
[kv_heads, value_dim] are two planes of a ``PagedRowsSpec``; with a window the pages behind it are
given back while the request runs.

bfloat16 steps whose head size the kernels for plain grouped attention are built for run on
those (the two planes have the layout of a key/value cache); everything else, float32 included,
on the kernel for paged rows, which is also the one that knows kept first positions behind a
window and a cap on the scores. The norm may come before or after the rotation and may lack
weights, the rotation may pair halves or neighbours, queries may carry a factor that grows with
the logarithm of their position, and the gate may be one number a head: all in the same kernels.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import PagedRowsSpec, ParamSpec
from clockwork_amd.parts.attention import attention_plan
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.sink_attention import longest_key_range, query_runs
from clockwork_amd.parts.specs import GatedAttentionSpec, RopePairsSpec


class GatedAttention(Part):
    graph_safe = True

    def __init__(self, spec: GatedAttentionSpec) -> None:
        self.spec = spec
        self.q_width = spec.num_heads * spec.key_dim
        self.k_width = spec.num_kv_heads * spec.key_dim
        self.v_width = spec.num_kv_heads * spec.value_dim
        self.own_values = spec.values == "projection"
        self.out_width = spec.num_heads * spec.value_dim
        # columns of the fused product: queries, keys, values (if projected), gate (if any)
        self.v_off = self.q_width + self.k_width
        self.g_off = self.v_off + (self.v_width if self.own_values else 0)
        self.gate_width = 0 if not spec.output_gate else (spec.num_heads if spec.gate_per_head else self.out_width)
        self.in_width = self.g_off + self.gate_width

    def param_specs(self):
        s = self.spec
        specs = {
            "in_weight": ParamSpec((self.in_width, s.hidden_size)),
            "out_weight": ParamSpec((s.hidden_size, self.out_width)),
        }
        if s.qkv_bias:
            specs["in_bias"] = ParamSpec((self.in_width,), precision="stored", init=("normal", 0.02))
        if s.out_bias:
            specs["out_bias"] = ParamSpec((s.hidden_size,), precision="compute", init=("normal", 0.02))
        if s.qk_norm and s.qk_norm_weight:
            specs["q_norm"] = ParamSpec((s.key_dim,), precision="stored", init=("one_plus_uniform", 0.3))
            specs["k_norm"] = ParamSpec((s.key_dim,), precision="stored", init=("one_plus_uniform", 0.3))
        return specs

    def cache_need(self):
        s = self.spec
        return PagedRowsSpec((("k", (s.num_kv_heads, s.key_dim)), ("v", (s.num_kv_heads, s.value_dim))), window=s.window,
                             keep_first=s.keep_first)

    def _plain_kernels(self, dtype) -> bool:
        """Do the kernels for plain grouped attention take these heads? bfloat16, keys and values
        of one size that they are built for."""
        s = self.spec
        # (the product's rows are padded to 16 bytes when the part is bound; those kernels know a
        # window and a cap on the scores, but no kept first positions)
        return (dtype == torch.bfloat16 and s.key_dim == s.value_dim and s.key_dim % 32 == 0 and 32 <= s.key_dim <= 256
                and not s.keep_first)

    def kernel_libraries(self) -> list:
        # the library of plain grouped attention is loaded (and, if missing, built) when the part is
        # bound as bfloat16 with a head size it takes: a float32 engine never needs it
        return [("rowwise", None), ("rows_attention", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        self.in_weight, self.in_bias = params["in_weight"], params.get("in_bias")
        self.out_weight, self.out_bias = params["out_weight"], params.get("out_bias")
        self.q_norm, self.k_norm = params.get("q_norm"), params.get("k_norm")
        self.rot_dims = s.position.rotary_dim if s.position is not None else 0
        self.pairing = "neighbours" if isinstance(s.position, RopePairsSpec) else "halves"
        self.norm_order = "none" if not s.qk_norm else ("after" if s.qk_norm_after_rotation else "before")
        self.freq = None
        if self.rot_dims:
            # base^(-2i / n), made on the host in float64 and rounded once
            freq = torch.tensor([float(s.position.theta) ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)],
                                dtype=torch.float64)
            self.freq = freq.to(torch.float32).to(device)
        self.dtype = dtype
        pad = (-self.in_width) % 8
        if pad and dtype == torch.bfloat16:
            # rows of the product that begin at multiples of 16 bytes (a few gate columns a head
            # leave odd widths): the kernels behind it load 16 bytes a lane
            self.in_weight = torch.cat([self.in_weight, self.in_weight.new_zeros((pad, s.hidden_size))])
            if self.in_bias is not None:
                self.in_bias = torch.cat([self.in_bias, self.in_bias.new_zeros(pad)])
        self.plain = self._plain_kernels(dtype) and ops.prefill_attention_supported(s.key_dim, dtype) \
            and ops.decode_attention_supported(s.key_dim, dtype)
        # the matrix-core kernel for paged rows: bfloat16 heads of 64 or 128 elements with values of 64 to 256
        self.rows_mfma = not self.plain and ops.rows_mfma_supported(s.key_dim, s.value_dim, 1, dtype)
        # a gate a head without a bias is applied where the attention kernel stores a head
        self._gate_inside = s.output_gate and s.gate_per_head and self.in_bias is None
        if self.rows_mfma:
            self.run = ops.ROWS_MFMA_TOKENS
        elif not self.plain:
            if not ops.rows_attention_supported(s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, maps=1):
                raise ValueError(f"attention with keys of {s.key_dim} and values of {s.value_dim} elements is beyond the "
                                 "attention kernel for paged rows (value_dim up to 512, tiles of 150 KB of LDS)")
            self.run = ops.rows_attention_tokens_per_item(s.num_heads, s.num_kv_heads, 1)

    def _plan(self, ctx):
        if self.plain:
            hd = self.spec.key_dim
            return attention_plan(ctx, self.spec.num_heads, self.spec.num_kv_heads, narrow_ok=ops.prefill_row_blocks_ok(hd, 2))
        if not self.rows_mfma:
            return (*query_runs(ctx, self.run), 1)
        s = self.spec
        key = ("gated attention", s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, s.window, s.keep_first)
        plan = ctx.plans.get(key)
        if plan is None:
            items, n_items = query_runs(ctx, self.run)
            # every item's keys are cut into runs where the step would leave most of the compute units idle
            longest = longest_key_range(ctx, s.window) + (s.keep_first if s.window is not None else 0)
            runs = ops.rows_mfma_key_runs(n_items, longest, s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, 1,
                                          ctx.num_compute_units)
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
        proj = ops.linear(x, self.in_weight, policy=policy)
        ops.headnorm_rope_store(proj, 0, self.q_width, self.v_off, s.num_heads, s.num_kv_heads, s.key_dim, self.v_width,
                                self.in_bias, self.q_norm, self.k_norm, s.norm_eps, ctx.positions, self.freq, self.rot_dims,
                                ctx.slots[cache.group], k_plane, v_plane, values_from_keys=not self.own_values,
                                pairing=self.pairing, norm=self.norm_order, query_temperature=s.query_temperature)
        out = torch.empty((x.shape[0], self.out_width), dtype=x.dtype, device=x.device)
        if self.plain:
            self._attend_plain(proj, out, ctx, cache, k_plane, v_plane)
        else:
            items, n_items, runs = self._plan(ctx)
            ops.rows_attention(proj, (proj.shape[1], s.key_dim), out, (out.shape[1], s.value_dim), k_plane, v_plane,
                               ctx.block_tables[cache.group], ctx.ctx_lens, ctx.cu_q, items, n_items, s.num_heads, s.num_kv_heads,
                               s.key_dim, s.value_dim, cache.block_size, s.scale, maps=1,
                               mask="window" if s.window is not None else "causal", mask_size=s.window or 0,
                               keep_first=s.keep_first, softcap=s.softcap or 0.0, mfma=self.rows_mfma, key_runs=runs,
                               head_gate=(proj, self.g_off) if self._gate_inside else None)
        if s.output_gate and not (self._gate_inside and not self.plain):
            bias_free = self.in_bias is None
            if not bias_free:
                raise NotImplementedError("an output gate with a bias")
            ops.sigmoid_mul_(out, proj, self.g_off, group=s.value_dim if s.gate_per_head else 1)
        return ops.linear(out, self.out_weight, self.out_bias, policy=policy)

    def _attend_plain(self, q, out, ctx, cache, k_plane, v_plane) -> None:
        """The kernels of plain grouped attention on the two planes (each [rows, kv_heads, size])."""
        s = self.spec
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.key_dim
        T = q.shape[0]
        plan = self._plan(ctx)
        common = dict(
            q=q, q_stride=q.shape[1], out=out, k_cache=k_plane, v_cache=v_plane,
            block_tables=ctx.block_tables[cache.group], ctx_lens=ctx.ctx_lens, cu_q=ctx.cu_q,
            nh=nh, nkv=nkv, hd=hd, block_size=cache.block_size, window=s.window or 0,
            scale=s.scale, n_tokens=T, n_requests=ctx.num_requests, softcap=s.softcap or 0.0,
        )
        if plan.n_wide:
            workspace = None
            if plan.mfma_parts > 1:
                need = ops.prefill_attention_workspace_floats(hd, plan.n_mfma, nh, nkv, plan.mfma_row_blocks)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention_prefill(items=plan.mfma_items, n_items=plan.n_mfma, row_blocks=plan.mfma_row_blocks,
                                  workspace=workspace, **common)
        if plan.n_single:
            workspace = None
            if plan.decode_splits > 1:
                need = ops.decode_attention_workspace_floats(hd, plan.n_single, nh, nkv, plan.decode_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention_decode(items=plan.single_items, n_items=plan.n_single, n_splits=plan.decode_splits,
                                 workspace=workspace, identity=plan.single_identity,
                                 split_keys=plan.decode_split_keys, max_ctx=plan.decode_max_ctx, **common)
