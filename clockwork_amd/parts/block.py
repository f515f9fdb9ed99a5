"""Block arrangements: how norms, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

from clockwork_amd import ops


class PreNormBlock:
    """x = x + mixer(norm(x)); x = x + ffn(norm(x)) (clockwork/engine/model.py:139-154).

    The residual stream is float32 and is only ever touched by the norms' fused add, so
    each branch output is added exactly once, in float32. ``forward`` takes the previous
    block's pending output ``delta`` and returns its own. A block without a feed-forward (and
    without its norm) is the first half alone.
    """

    def __init__(self, mixer, mixer_norm, feed_forward=None, ffn_norm=None) -> None:
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a pre-norm block has a feed-forward and its norm, or neither")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ffn_norm = ffn_norm

    def parts(self) -> dict:
        parts = {"mixer": self.mixer}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
        parts["mixer_norm"] = self.mixer_norm
        if self.ffn_norm is not None:
            parts["ffn_norm"] = self.ffn_norm
        return parts

    def first_norm(self):
        """The norm that takes what the block before hands on (may it be two pending outputs?)."""
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache):
        x = self.mixer_norm.forward(resid, delta)
        a = self.mixer.forward(x, ctx, cache)
        if self.feed_forward is None:
            return a
        # Few rows: the second norm can run inside the feed-forward's first product, which saves a
        # launch. That kernel writes no residual, so the mixer's output stays pending and is
        # handed on together with the feed-forward's (the next norm must be able to take both).
        fuses = getattr(self.feed_forward, "fuses_input_norm", None)
        lazy = getattr(self.ffn_norm, "lazy", None)
        if (fuses is not None and lazy is not None and getattr(ctx, "next_norm_accepts_pending", False)
                and fuses(resid.shape[0], x.dtype, a)):
            return ops.PendingPair(a, self.feed_forward.forward(lazy(resid, a), ctx))
        x = self.ffn_norm.forward(resid, a)
        return self.feed_forward.forward(x, ctx)


class BranchGate:
    """Sigmoid gates on a block's branches (``BranchGateSpec``): one product of the block's normed
    input with all gates' matrices; the sigmoids and the biases are applied where the branches are
    added to the residual stream (``ops.GatedBranches``)."""

    graph_safe = True

    def __init__(self, spec) -> None:
        self.spec = spec

    def param_specs(self):
        from clockwork_amd.config.spec import ParamSpec

        n = self.spec.branches * self.spec.hidden_size
        return {"weight": ParamSpec((n, self.spec.hidden_size)),
                "bias": ParamSpec((n,), precision="float32", init=("normal", 0.5))}

    def cache_need(self):
        return None

    def kernel_libraries(self) -> list:
        return [("rowwise", None)]

    def bind(self, params, device, dtype) -> None:
        self.weight, self.bias = params["weight"], params["bias"]

    def forward(self, x, ctx):
        """The gates' products [T, branches * hidden] (before bias and sigmoid)."""
        return ops.linear(x, self.weight, policy=getattr(ctx, "products", None))


class ParallelBlock:
    """One norm, mixer and feed-forward side by side on its output:
    x = x + g1 * mixer(norm(x)) + g2 * ffn(norm(x)), with g = sigmoid(W norm(x) + c) from the
    block's ``gate`` part, or 1 without one; the feed-forward may be absent.

    The residual stream is float32. The block hands its branches on unadded, as
    ``ops.GatedBranches``, when the norm that comes next adds them inside its own kernel
    (``accepts_gated``); else it adds them itself with one kernel."""

    def __init__(self, mixer, mixer_norm, feed_forward=None, gate=None) -> None:
        self.mixer, self.mixer_norm, self.feed_forward, self.gate = mixer, mixer_norm, feed_forward, gate
        if gate is not None and gate.spec.branches != (2 if feed_forward is not None else 1):
            raise ValueError("a block's gate needs one set of gates per branch")

    def parts(self) -> dict:
        parts = {"mixer": self.mixer, "mixer_norm": self.mixer_norm}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
        if self.gate is not None:
            parts["gate"] = self.gate
        return parts

    def first_norm(self):
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache):
        x = self.mixer_norm.forward(resid, delta)
        a = self.mixer.forward(x, ctx, cache)
        b = self.feed_forward.forward(x, ctx) if self.feed_forward is not None else None
        z = self.gate.forward(x, ctx) if self.gate is not None else None
        pending = ops.GatedBranches(z, self.gate.bias if self.gate is not None else None, a, b)
        if getattr(ctx, "next_norm_accepts_gated", False):
            return pending
        ops.gated_residual_add(resid, pending)
        return None


class TwoNormParallelBlock:
    """x = x + mixer(norm1(x)) + ffn(norm2(x)): mixer and feed-forward side by side, each behind a
    norm of its own of the same x; the feed-forward and its norm may be absent.

    The residual stream is float32. Both outputs are handed on unadded (``ops.PendingPair``) when
    the norm that comes next adds them inside its kernel; else the block adds them itself. The
    first norm takes what the block before left pending; the second then norms the same, updated
    stream."""

    def __init__(self, mixer, mixer_norm, feed_forward=None, ffn_norm=None) -> None:
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a block has a feed-forward and its norm, or neither")
        self.mixer, self.mixer_norm, self.feed_forward, self.ffn_norm = mixer, mixer_norm, feed_forward, ffn_norm

    def parts(self) -> dict:
        parts = {"mixer": self.mixer}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
        parts["mixer_norm"] = self.mixer_norm
        if self.ffn_norm is not None:
            parts["ffn_norm"] = self.ffn_norm
        return parts

    def first_norm(self):
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache):
        both = getattr(self.mixer_norm, "forward_pair", None)
        if self.feed_forward is not None and both is not None and type(self.ffn_norm) is type(self.mixer_norm):
            x, y = both(resid, delta, self.ffn_norm)   # one kernel: the two norms share the row's statistics
        else:
            x = self.mixer_norm.forward(resid, delta)
            y = self.ffn_norm.forward(resid, None) if self.feed_forward is not None else None
        a = self.mixer.forward(x, ctx, cache)
        if self.feed_forward is None:
            return a
        b = self.feed_forward.forward(y, ctx)
        if isinstance(a, ops.PartialSums):
            a = a.sum(x.dtype)
        if getattr(ctx, "next_norm_accepts_pending", False):
            return ops.PendingPair(a, b)
        ops.gated_residual_add(resid, ops.GatedBranches(None, None, a, b))
        return None


class BranchNormBlock:
    """x = x + c * N1(mixer(x)); x = x + c * N2(ffn(x)): mixer and feed-forward read the stream
    itself, and what is normed is their output (``BranchRMSNorm``, whose spec holds c). The
    feed-forward and its norm may be absent.

    The stream is float32; the sublayers read its image in the activation type, which the kernel
    that adds a normed branch writes beside the stream. So the block has nothing pending when it
    is done: it hands on the image (``ops.StreamImage``), which the next block of this kind reads
    instead of making it again."""

    def __init__(self, mixer, mixer_norm, feed_forward=None, ffn_norm=None) -> None:
        if (feed_forward is None) != (ffn_norm is None):
            raise ValueError("a block has a feed-forward and its norm, or neither")
        for norm in (mixer_norm, ffn_norm):
            if norm is not None and not (hasattr(norm, "join") and hasattr(norm, "image")):
                raise TypeError("the norms of a 'branchnorm' block norm a branch as it joins the stream (join / image)")
        self.mixer, self.mixer_norm, self.feed_forward, self.ffn_norm = mixer, mixer_norm, feed_forward, ffn_norm

    def parts(self) -> dict:
        parts = {"mixer": self.mixer}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
        parts["mixer_norm"] = self.mixer_norm
        if self.ffn_norm is not None:
            parts["ffn_norm"] = self.ffn_norm
        return parts

    def forward(self, resid, delta, ctx, cache):
        if isinstance(delta, ops.StreamImage):
            x = delta.image
        elif delta is None:
            x = self.mixer_norm.image(resid)
        else:
            raise TypeError("a 'branchnorm' block cannot add the pending output of a block of another kind")
        x = self.mixer_norm.join(resid, self.mixer.forward(x, ctx, cache))
        if self.feed_forward is not None:
            x = self.ffn_norm.join(resid, self.feed_forward.forward(x, ctx))
        return ops.StreamImage(x)
