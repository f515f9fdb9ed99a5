"""Linear attention with a matrix state per head and a decay per key channel
(``DecayedLinearAttentionSpec``): S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.

One product makes q, k, v, the output gate and the low-rank input of the decay for every token
of the step; one kernel walks each request's tokens in order from the request's state slot
(float32 [heads, key_dim, value_dim], zero at a request's start), makes the decays
(sigmoid(z)^(1/tau) through log-sigmoid, float32), norms and gates the outputs; output product.
A step with a portion of more than 64 tokens cuts every request's tokens into segments of 32 that
are walked side by side: each from a zero state, then the start states are carried from segment
to segment, then each segment is walked again for its outputs (the same sums, other parentheses).
The state is all the mixer keeps: a ``StateSpec``.
"""

from __future__ import annotations

import numpy as np
import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec, StateSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.specs import DecayedLinearAttentionSpec


# tokens of a segment, and the longest portion that is still walked token by token in one piece
SEGMENT_TOKENS = 32
SEGMENT_MIN_TOKENS = 64


class DecayedLinearAttention(Part):
    graph_safe = True

    def __init__(self, spec: DecayedLinearAttentionSpec) -> None:
        self.spec = spec
        qk, v = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        # columns of the input product: q, k, v, gate, decay input
        self.q_off, self.k_off, self.v_off, self.g_off, self.u_off = 0, qk, 2 * qk, 2 * qk + v, 2 * qk + 2 * v
        self.in_width = 2 * qk + 2 * v + spec.decay_rank

    def param_specs(self):
        s = self.spec
        return {
            "in_weight": ParamSpec((self.in_width, s.hidden_size)),
            "decay_weight": ParamSpec((s.num_heads * s.key_dim, s.decay_rank), init=("normal", 0.5)),
            "decay_bias": ParamSpec((s.num_heads * s.key_dim,), precision="float32", init=("normal", 1.0)),
            "norm_weight": ParamSpec((s.value_dim,), precision="float32", init=("one_plus_uniform", 0.1)),
            "out_weight": ParamSpec((s.hidden_size, s.num_heads * s.value_dim)),
        }

    def cache_need(self):
        s = self.spec
        return StateSpec((s.num_heads, s.key_dim, s.value_dim), "float32")

    def kernel_libraries(self) -> list:
        return [("linear_recurrence", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        if not ops.linear_recurrence_supported(s.key_dim, s.value_dim):
            raise ValueError(f"a state of {s.key_dim} x {s.value_dim} a head is beyond the recurrence kernel "
                             "(value_dim up to 256, key_dim up to 128 rows a thread)")
        self.segments_ok = ops.linear_recurrence_segments_supported(s.key_dim, s.value_dim)
        self.in_weight = params["in_weight"]
        self.decay_weight = params["decay_weight"]
        self.decay_bias = params["decay_bias"]
        self.norm_weight = params["norm_weight"]
        self.out_weight = params["out_weight"]

    def _segments(self, ctx):
        """The step's segments when it holds a long portion and the state fits the kernel that
        walks segments side by side, else None (every request is then walked token by token by
        one workgroup a head). Made once a step, kept in ``ctx.plans``."""
        if max(ctx.h_q_lens, default=0) <= SEGMENT_MIN_TOKENS or not self.segments_ok:
            return None
        key = ("recurrence segments", SEGMENT_TOKENS)
        plan = ctx.plans.get(key)
        if plan is None:
            items, first = [], [0]
            for r, q_len in enumerate(ctx.h_q_lens):
                tok0 = np.arange(0, q_len, SEGMENT_TOKENS, dtype=np.int32)
                rows = np.zeros((tok0.size, 4), dtype=np.int32)
                rows[:, 0] = r
                rows[:, 1] = tok0
                rows[:, 2] = np.minimum(SEGMENT_TOKENS, q_len - tok0)
                rows[:, 3] = np.arange(tok0.size)
                items.append(rows.reshape(-1))
                first.append(first[-1] + tok0.size)
            device_items, device_first = ctx.upload([np.concatenate(items), first])
            plan = ctx.plans[key] = (device_items, first[-1], device_first)
        return plan

    def prepare(self, ctx) -> None:
        self._segments(ctx)

    def shape_class(self, q_lens, ctx_lens):
        return "segments" if max(q_lens, default=0) > SEGMENT_MIN_TOKENS and self.segments_ok else "token by token"

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        proj = ops.linear(x, self.in_weight, policy=policy)
        common = (proj, self.q_off, self.k_off, self.v_off, self.g_off, self.u_off, self.decay_weight, self.decay_bias,
                  self.norm_weight, cache.state, ctx.state_slots, ctx.cu_q)
        sizes = (ctx.num_requests, s.num_heads, s.key_dim, s.value_dim, s.key_dim ** -0.5, s.tau, s.norm_eps)
        plan = self._segments(ctx)
        if plan is not None:
            items, n_segments, first = plan
            out = ops.linear_recurrence_segments(*common, items, n_segments, SEGMENT_TOKENS, first, *sizes)
        else:
            out = ops.linear_recurrence(*common, *sizes)
        return ops.linear(out, self.out_weight, policy=policy)


class ShiftedRecurrence(Part):
    """A matrix recurrence a head whose inputs are mixes of a token with the one before it
    (``ShiftedRecurrenceSpec``).

    One kernel makes the five mixes of the step's tokens (the row before a portion's first token
    waits in the request's state slot, and the portion's last row is left there); the products
    for r, k, v and the gate are one batched product over four planes, the decay's low-rank input
    a product of its own; the recurrence kernels of :class:`DecayedLinearAttention` walk the tokens
    in their other form (the decay exp(-exp(.)) of the tanh of that input, the output read from the
    state before the token joins it, the token itself through the bonus), norm every head's output
    with the head's own weights and gate it; output product. Long portions are cut into segments
    that are walked side by side, as there. A request's slot is float32
    [heads * dim * dim + hidden]: the matrices, then the last input row."""

    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, spec) -> None:
        self.spec = spec
        self.inner = spec.num_heads * spec.head_dim

    def param_specs(self):
        s = self.spec
        return {
            # the mixing vectors of r, k, v, g, w one behind the other
            "mix": ParamSpec((len(self.MIXES) * s.hidden_size,), precision="float32", init=("uniform", 0.0, 1.0)),
            "rkvg_weight": ParamSpec((4 * self.inner, s.hidden_size)),
            "decay_in_weight": ParamSpec((s.decay_rank, s.hidden_size), init=("normal", 0.1)),
            "decay_weight": ParamSpec((self.inner, s.decay_rank), init=("normal", 0.5)),
            "decay_bias": ParamSpec((self.inner,), precision="float32", init=("uniform", -3.0, 0.5)),
            "bonus": ParamSpec((s.num_heads, s.head_dim), precision="float32", init=("normal", 0.5)),
            "norm_weight": ParamSpec((self.inner,), precision="float32", init=("one_plus_uniform", 0.1)),
            "out_weight": ParamSpec((s.hidden_size, self.inner)),
        }

    def cache_need(self):
        s = self.spec
        return StateSpec((s.num_heads * s.head_dim * s.head_dim + s.hidden_size,), "float32")

    def kernel_libraries(self) -> list:
        return [("linear_recurrence", None), ("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        if not ops.linear_recurrence_supported(s.head_dim, s.head_dim):
            raise ValueError(f"a state of {s.head_dim} x {s.head_dim} a head is beyond the recurrence kernel "
                             "(head_dim up to 256)")
        self.segments_ok = ops.linear_recurrence_segments_supported(s.head_dim, s.head_dim)
        self.mix = params["mix"].view(len(self.MIXES), s.hidden_size)
        self.rkvg = params["rkvg_weight"].view(4, self.inner, s.hidden_size)
        self.decay_in = params["decay_in_weight"]
        self.decay_weight, self.decay_bias = params["decay_weight"], params["decay_bias"]
        self.bonus, self.norm_weight = params["bonus"], params["norm_weight"]
        self.out_weight = params["out_weight"]

    def _items(self, ctx):
        from clockwork_amd.parts.sink_attention import query_runs

        return query_runs(ctx, ops.SHIFT_MIX_TOKENS)

    _segments = DecayedLinearAttention._segments

    def prepare(self, ctx) -> None:
        self._items(ctx)
        self._segments(ctx)

    def shape_class(self, q_lens, ctx_lens):
        return "segments" if max(q_lens, default=0) > SEGMENT_MIN_TOKENS and self.segments_ok else "token by token"

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        T = x.shape[0]
        state = cache.state
        items, n_items = self._items(ctx)
        mixes = ops.shift_mix(x, self.mix, state, s.num_heads * s.head_dim * s.head_dim, ctx.state_slots, ctx.cu_q, items, n_items)
        planes = torch.empty((4, T, self.inner), dtype=x.dtype, device=x.device)
        ops.heads_linear(mixes[:4], self.rkvg, planes)
        decay_input = ops.linear(mixes[4], self.decay_in, policy=policy)
        common = (planes, 0, 1, 2, 3, 0, self.decay_weight, self.decay_bias, self.norm_weight, state, ctx.state_slots, ctx.cu_q)
        sizes = (ctx.num_requests, s.num_heads, s.head_dim, s.head_dim, 1.0, 1.0, s.norm_eps)
        plan = self._segments(ctx)
        if plan is not None:
            # a long portion: the tanh once an element, ahead of the kernel that makes every channel's decay from all of them
            seg_items, n_segments, first = plan
            out = ops.linear_recurrence_segments(*common, seg_items, n_segments, SEGMENT_TOKENS, first, *sizes, decay="double_exp",
                                                 bonus=self.bonus, decay_input=ops.tanh_(decay_input))
        else:
            out = ops.linear_recurrence(*common, *sizes, decay="double_exp_tanh", bonus=self.bonus, decay_input=decay_input)
        return ops.linear(out, self.out_weight, policy=policy)
