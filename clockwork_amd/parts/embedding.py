"""The two ends of the decoder: token ids to the residual stream, final rows to logits.

Both are parts like any other (clockwork/engine/model.py:200 and 216-233 are the plain table
lookup and the plain product that these two implement); another architecture registers its own
(a scaled embedding, positions added at the input, a capped or biased output) under its own spec.

Interfaces: an embedding has ``forward(ctx) -> resid`` (float32 [T, hidden], the residual
stream of the step's tokens) and may offer ``table()``, the [vocab, hidden] matrix a tied head
uses. A head has ``forward(rows, ctx) -> logits`` (float32 [n, vocab]) for the normed rows the
step wants logits of; a head whose spec has ``tied`` set is handed the embedding part through
``use_embedding(part)`` before it is bound.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import LinearHeadSpec, PositionTableEmbeddingSpec, TokenEmbeddingSpec


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, spec: TokenEmbeddingSpec) -> None:
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.device = device

    def table(self) -> torch.Tensor:
        return self.weight

    def forward(self, ctx) -> torch.Tensor:
        resid = torch.empty((ctx.num_tokens, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        return ops.embedding(self.weight, ctx.token_ids, resid)


class PositionTableEmbedding(Part):
    """scale * table[id] + positions[p] in float32, p the token's index in its request
    (``ctx.positions``); a tied head gets the table itself, without the scale."""

    graph_safe = True

    def __init__(self, spec: PositionTableEmbeddingSpec) -> None:
        self.spec = spec

    def param_specs(self):
        specs = {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}
        if self.spec.max_positions is not None:
            specs["positions"] = ParamSpec((self.spec.max_positions, self.spec.hidden_size))
        return specs

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.position_table = params.get("positions")
        self.device = device

    def table(self) -> torch.Tensor:
        return self.weight

    def forward(self, ctx) -> torch.Tensor:
        resid = torch.empty((ctx.num_tokens, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        return ops.embedding_positions(self.weight, ctx.token_ids, ctx.positions, self.position_table, self.spec.scale, resid)


class LinearHead(Part):
    graph_safe = True

    def __init__(self, spec: LinearHeadSpec) -> None:
        self.spec = spec
        self._embedding = None
        self.shares_embedding = False

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def use_embedding(self, embedding) -> None:
        self._embedding = embedding

    def bind(self, params, device, dtype) -> None:
        own = params.get("weight")
        if not self.spec.tied:
            if own is None:
                raise RuntimeError("the output head's matrix is missing and the embeddings are not tied")
            self.weight = own
            return
        # one buffer, two uses (clockwork/engine/model.py:217-218). A tied checkpoint may still
        # carry the head's tensor; the reference loads it into the shared parameter, so it has to
        # be the table itself: it is checked and let go, not kept as a second matrix.
        table = getattr(self._embedding, "table", lambda: None)() if self._embedding is not None else None
        if table is None:
            raise RuntimeError("a tied output head needs an embedding part that offers its table()")
        if own is not None and not (own.shape == table.shape and torch.equal(own, table)):
            raise ValueError(
                "the checkpoint ties the output head to the embedding (tie_word_embeddings) but "
                "carries an lm_head tensor that differs from the embedding table"
            )
        self.weight = table
        self.shares_embedding = True

    def matrices(self) -> list:
        """The matrices a step streams through this part (for the step's byte count)."""
        return [self.weight]

    def forward(self, rows: torch.Tensor, ctx) -> torch.Tensor:
        logits = ops.linear(rows, self.weight, out_dtype=torch.float32, policy=getattr(ctx, "products", None))
        if self.spec.scale is not None:
            ops.scale_(logits, self.spec.scale)
        if self.spec.softcap is not None:
            ops.softcap_(logits, self.spec.softcap)
        return logits

    def kernel_libraries(self) -> list:
        return [("rowwise", None)] if self.spec.softcap is not None or self.spec.scale is not None else []


class StreamReentry(Part):
    """The stream made anew from itself and the model's input before a pass of a repeated run of
    layers (``StreamReentrySpec``): x <- R [x; x0] + s_n.

    One kernel adds what the block before left pending to the float32 stream and writes
    [x, x0, e_n] in the activation type, e_n a one in column n of a few extra columns; one product
    with [R | s^T] then yields R [x; x0] + s_n with the learned row inside the product's float32
    sums. The result is the new float32 stream."""

    graph_safe = True

    def __init__(self, spec) -> None:
        self.spec = spec
        self.extra = -(-spec.passes // 8) * 8   # the operand's rows stay a multiple of 16 bytes

    def param_specs(self):
        H = self.spec.hidden_size
        return {"in_weight": ParamSpec((H, 2 * H), init=("normal", 0.7 / (2 * H) ** 0.5 * 2 ** 0.5)),
                "step": ParamSpec((self.spec.passes, H), init=("normal", 0.1))}

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        H, P = self.spec.hidden_size, self.spec.passes
        weight = torch.zeros((H, 2 * H + self.extra), dtype=dtype, device=device)
        weight[:, : 2 * H] = params["in_weight"]
        weight[:, 2 * H : 2 * H + P] = params["step"].to(dtype).t()
        self.weight = weight
        self.dtype = dtype

    def forward(self, resid: torch.Tensor, pending, model_input: torch.Tensor, pass_no: int, ctx) -> torch.Tensor:
        """The new float32 stream [T, hidden]; ``pending`` has joined the old one on the way."""
        if not 0 <= pass_no < self.spec.passes:
            raise ValueError(f"pass {pass_no} of {self.spec.passes}")
        image = ops.stream_beside_input(resid, pending, model_input, self.dtype, self.extra, pass_no)
        return ops.linear(image, self.weight, out_dtype=torch.float32, policy=getattr(ctx, "products", None))
