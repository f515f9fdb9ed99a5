"""Specs of the built-in part kinds: their sizes and constants, nothing else.

Importing this module needs neither torch nor the HIP libraries, so
configuration code and CPU tests can build and inspect a model description.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class RMSNormSpec:
    """y = weight * cast(x / sqrt(mean(x^2) + eps)); statistics in float32."""

    size: int
    eps: float


@dataclass(frozen=True)
class RopeNeoxSpec:
    """Rotary position encoding, half-split pairing (i, i + rotary_dim/2).

    inv_freq[j] = 1 / theta^(2j / rotary_dim); the first ``rotary_dim`` elements
    of each head are rotated, the rest pass through.
    """

    rotary_dim: int
    theta: float


@dataclass(frozen=True)
class RopePairsSpec:
    """Rotary position encoding over neighbouring elements: (2i, 2i + 1) turn together by the angle
    position / theta^(2i / rotary_dim); the first ``rotary_dim`` elements of each head are rotated,
    the rest pass through."""

    rotary_dim: int
    theta: float


@dataclass(frozen=True)
class AttentionSpec:
    """Softmax attention with grouped query heads over a paged key/value cache."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    qkv_bias: bool
    out_bias: bool
    scale: float
    window: Optional[int] = None
    position: Any = None  # a position-encoding spec, or None for no encoding

    def __post_init__(self):
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError(
                f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}"
            )
        if self.head_dim % 16 != 0 or not 16 <= self.head_dim <= 256:
            raise ValueError(
                f"head_dim {self.head_dim} is not supported: the attention kernels take "
                "multiples of 16 from 16 to 256"
            )
        if self.window is not None and self.window < 1:
            raise ValueError(f"window must be positive, got {self.window}")


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), no biases."""

    hidden_size: int
    intermediate_size: int


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    """The residual stream starts as row ``id`` of a [vocab, hidden] table: no scaling, nothing added."""

    vocab_size: int
    hidden_size: int


@dataclass(frozen=True)
class LinearHeadSpec:
    """logits = rows @ W^T with W [vocab, hidden], no bias, float32 logits. ``tied``: W is the
    embedding's table (one buffer, two uses) unless the checkpoint brings a head of its own.
    ``softcap`` c: the logits are capped, c * tanh(logits / c). ``scale`` s: the logits are
    multiplied by s (before a cap)."""

    vocab_size: int
    hidden_size: int
    tied: bool = False
    softcap: Optional[float] = None  # logits <- softcap * tanh(logits / softcap)
    scale: Optional[float] = None    # logits <- scale * logits


@dataclass(frozen=True)
class LayerNormSpec:
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias; statistics in float32."""

    size: int
    eps: float
    bias: bool = True


@dataclass(frozen=True)
class PositionTableEmbeddingSpec:
    """The residual stream starts as scale * table[id] + positions[p], p the token's index in its
    request; ``max_positions`` None: no position table (a scaled lookup)."""

    vocab_size: int
    hidden_size: int
    scale: float = 1.0
    max_positions: Optional[int] = None


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x)), no biases; ``activation`` "silu" or "gelu_tanh"
    (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))))."""

    hidden_size: int
    intermediate_size: int
    activation: str = "gelu_tanh"

    def __post_init__(self):
        if self.activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"activation {self.activation!r}: expected 'silu' or 'gelu_tanh'")


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Softmax attention with grouped query heads over a paged cache of keys [kv_heads, key_dim]
    and values [kv_heads, value_dim], with options that plain attention has not:

    * ``qk_norm``: "projection" - queries and keys are RMS-normed as whole projections (all heads
      of a token as one vector, a weight of that size each) before they are cut into heads; None.
    * ``distance_bias``: the score of query i and key j of head h loses r1[h] * log(1 + r2[h] * (i - j)).
    * ``sink``: the softmax denominator of head h has the extra term exp(sink[h]): no key, no value.
    * ``talking_heads``: the normalised weights are mixed across heads by a learned
      [heads, heads] matrix before they are applied; head h applies its mixed weights to the
      values of its own key/value head.
    * ``window`` W: a token sees itself and the W - 1 tokens before it; None: all of them.

    No rotation or other position encoding is applied, no biases."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    window: Optional[int] = None
    qk_norm: Optional[str] = "projection"
    qk_norm_eps: float = 1e-6
    distance_bias: bool = True
    sink: bool = True
    talking_heads: bool = True

    def __post_init__(self):
        if self.num_heads < 1 or self.num_kv_heads < 1 or self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        if self.key_dim < 1 or self.value_dim < 1:
            raise ValueError("key_dim and value_dim must be positive")
        if self.window is not None and self.window < 1:
            raise ValueError(f"window must be positive, got {self.window}")
        if self.qk_norm not in (None, "projection"):
            raise ValueError(f"qk_norm {self.qk_norm!r}: expected 'projection' or None")


@dataclass(frozen=True)
class DecayedLinearAttentionSpec:
    """Linear attention with a matrix state per head and a decay per key channel:
    S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_t * key_dim^-1/2), S float32, zero at a
    request's start. a_t = sigmoid(A2 (A1 x_t) + b)^(1/tau) with A1 [decay_rank, hidden]. Each
    head's o_t is RMS-normed over value_dim with one weight shared by the heads, the heads are
    concatenated, multiplied by silu(G x_t) and projected back to hidden_size."""

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    decay_rank: int
    tau: float
    norm_eps: float

    def __post_init__(self):
        if min(self.num_heads, self.key_dim, self.value_dim, self.decay_rank) < 1:
            raise ValueError("heads, key_dim, value_dim and decay_rank must be positive")
        if not self.tau > 0:
            raise ValueError(f"tau must be positive, got {self.tau}")


@dataclass(frozen=True)
class PairMixerSpec:
    """Two mixers side by side on the same input; the result is the mean of their outputs, each
    first RMS-normed over the model width with a weight of its own."""

    hidden_size: int
    left: Any
    right: Any
    eps: float


@dataclass(frozen=True)
class BranchGateSpec:
    """Sigmoid gates on a block's branches: branch b's output is multiplied element by element by
    sigmoid(W_b x + c_b), x the block's normed input; ``branches`` gates of hidden_size each."""

    hidden_size: int
    branches: int = 2


@dataclass(frozen=True)
class DynamicTanhSpec:
    """y = tanh(alpha * x) * weight + bias with one learned scalar alpha: a norm that takes no mean
    or variance of the row. ``delta_scale``: what the norm adds to the residual stream first (the
    pending branch output) is multiplied by it (a model-wide residual multiplier)."""

    size: int
    delta_scale: float = 1.0
    bias: bool = True


@dataclass(frozen=True)
class DenseMLPSpec:
    """down(act(up(x))), no gate, no biases; ``activation`` "gelu" (the erf form) or "relu2"
    (max(z, 0)^2)."""

    hidden_size: int
    intermediate_size: int
    activation: str = "gelu"

    def __post_init__(self):
        if self.activation not in ("gelu", "relu2"):
            raise ValueError(f"activation {self.activation!r}: expected 'gelu' or 'relu2'")


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Grouped softmax attention in which every query head has two score maps over the same
    values: queries [heads, 2, key_dim], keys [kv_heads, 2, key_dim], values [kv_heads, value_dim],
    all from biased projections (``qkv_bias``). The head's output is A_1 - lambda * A_2 with
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + ``lambda_init`` (four learned vectors of key_dim, one
    number a layer), then divided by its root mean square over value_dim (``norm_eps`` inside the
    root, no weight) and multiplied by 1 - ``lambda_init``.

    ``qk_norm``: every query and key vector of key_dim elements (each map of each head by itself)
    is divided by its root mean square (``norm_eps``) and multiplied by a weight of key_dim
    elements, one for all query vectors and one for all key vectors, after the bias and before the
    rotation. ``position``: a ``RopeNeoxSpec``, applied to every query and key vector by itself
    (its first ``rotary_dim`` elements); None: no position encoding. ``out_bias``: the output
    projection has a bias.

    What a token sees: ``segment`` S: the earlier tokens of its own run of S positions (runs
    counted from position 0); ``window`` W: itself and the W - 1 before it; neither: all earlier ones."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    lambda_init: float
    norm_eps: float
    segment: Optional[int] = None
    window: Optional[int] = None
    qkv_bias: bool = True
    qk_norm: bool = False
    position: Any = None
    out_bias: bool = False

    def __post_init__(self):
        if self.num_heads < 1 or self.num_kv_heads < 1 or self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        if self.key_dim < 1 or self.value_dim < 1:
            raise ValueError("key_dim and value_dim must be positive")
        if self.position is not None and not 0 <= self.position.rotary_dim <= self.key_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds key_dim {self.key_dim}")
        if self.segment is not None and self.window is not None:
            raise ValueError("an attention mask has segments or a window, not both")
        for name in ("segment", "window"):
            if getattr(self, name) is not None and getattr(self, name) < 1:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are made from one cached latent a token. Queries:
    RMS-normed low-rank step of ``q_rank``, then [heads, key_dim + rope_dim]. Keys/values: a
    projection to ``kv_rank + rope_dim`` elements; the first kv_rank, RMS-normed with a weight, are
    the latent c, the others one rotated key part that all heads share. Head a's key is
    [uk_a c, rotated part], its value uv_a c (value_dim). The rope_dim parts of queries and keys
    are rotated by position: the first ``rotary_dims`` of them in half-split pairs with base
    ``rope_base``. ``sink``: exp(sink[a]) joins head a's softmax denominator. ``output_gate``: the
    concatenated heads are multiplied by the sigmoid of a projection of the mixer's input.
    Only the latent and the rotated part are cached: kv_rank + rope_dim elements a token."""

    hidden_size: int
    num_heads: int
    key_dim: int
    rope_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    rope_base: float
    rotary_dims: int
    norm_eps: float
    sink: bool = True
    output_gate: bool = True
    window: Optional[int] = None

    def __post_init__(self):
        if min(self.num_heads, self.key_dim, self.value_dim, self.q_rank, self.kv_rank) < 1 or self.rope_dim < 0:
            raise ValueError("heads, key_dim, value_dim, q_rank and kv_rank must be positive, rope_dim not negative")
        if self.rotary_dims % 2 or not 0 <= self.rotary_dims <= self.rope_dim:
            raise ValueError(f"rotary_dims {self.rotary_dims} must be even and at most rope_dim {self.rope_dim}")
        if self.window is not None and self.window < 1:
            raise ValueError(f"window must be positive, got {self.window}")


@dataclass(frozen=True)
class BranchRMSNormSpec:
    """An RMS norm whose weight is kept as its distance from ``weight_offset``:
    N(y) = y / sqrt(mean(y^2) + eps) * (weight_offset + w), float32 throughout. It has two uses.
    On a branch: a sublayer's OUTPUT is normed and joins the float32 stream multiplied by
    ``branch_scale``, x <- x + branch_scale * N(branch) (the "branchnorm" block arrangement, whose
    sublayers read the stream itself). On the stream: N(x) of chosen rows (a model's final norm)."""

    size: int
    eps: float
    branch_scale: float = 1.0
    weight_offset: float = 1.0


@dataclass(frozen=True)
class GatedAttentionSpec:
    """Grouped softmax attention over paged key rows [kv_heads, key_dim] and value rows
    [kv_heads, value_dim], with options that plain attention has not:

    * ``qk_norm``: every head's query and key vector is divided by its root mean square
      (``norm_eps`` inside the root) and multiplied by a weight of key_dim elements (one for all
      query heads, one for all key heads), before the rotation.
    * ``position``: a ``RopeNeoxSpec`` (the first ``rotary_dim`` elements of every head's query
      and key are rotated) or None.
    * ``values``: "projection" (a value projection of its own) or "keys": the values are the key
      projections as they leave the product, before norm and rotation (value_dim == key_dim, no
      value matrix).
    * ``output_gate``: the concatenated heads are multiplied by the logistic function of one more
      projection of the mixer's input before the output projection.
    * ``window`` W: a token sees itself and the W - 1 tokens before it; None: all of them.
    * ``qkv_bias`` / ``out_bias``.
    * ``qk_norm_weight`` False: the query/key norm has no weights. ``qk_norm_after_rotation``: the
      vectors are rotated first and the rotated vector is normed.
    * ``position`` may also be a ``RopePairsSpec`` (neighbouring elements turn together).
    * ``keep_first`` n (with a window): the first n positions of a request stay visible to every
      later token, at their true positions.
    * ``softcap`` c: scores are squashed before the softmax, c * tanh(scale * q . k / c).
    * ``query_temperature`` (coef, every): the query at position p is multiplied by
      1 + coef * ln(floor((p + 1) / every) + 1), after its norm.
    * ``gate_per_head`` (with ``output_gate``): the gate is one number a head, not one an element."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    norm_eps: float = 1e-6
    window: Optional[int] = None
    qk_norm: bool = True
    position: Any = None
    values: str = "projection"
    output_gate: bool = False
    qkv_bias: bool = False
    out_bias: bool = False
    qk_norm_weight: bool = True
    qk_norm_after_rotation: bool = False
    keep_first: int = 0
    softcap: Optional[float] = None
    query_temperature: Optional[tuple] = None
    gate_per_head: bool = False

    def __post_init__(self):
        if self.num_heads < 1 or self.num_kv_heads < 1 or self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}")
        if self.key_dim < 1 or self.value_dim < 1:
            raise ValueError("key_dim and value_dim must be positive")
        if self.values not in ("projection", "keys"):
            raise ValueError(f"values {self.values!r}: expected 'projection' or 'keys'")
        if self.values == "keys" and self.value_dim != self.key_dim:
            raise ValueError(f"values that are the keys have the keys' size: value_dim {self.value_dim} != key_dim {self.key_dim}")
        if self.position is not None and not 0 <= self.position.rotary_dim <= self.key_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds key_dim {self.key_dim}")
        if self.window is not None and self.window < 1:
            raise ValueError(f"window must be positive, got {self.window}")
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise ValueError("first positions are kept visible behind a window only, and their number is not negative")
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError(f"softcap must be positive, got {self.softcap}")
        if self.query_temperature is not None and (len(self.query_temperature) != 2 or int(self.query_temperature[1]) < 1):
            raise ValueError(f"query_temperature is (coef, every) with every >= 1, got {self.query_temperature!r}")
        if self.gate_per_head and not self.output_gate:
            raise ValueError("a gate a head is an output gate")


@dataclass(frozen=True)
class ShiftedRecurrenceSpec:
    """A recurrence over a matrix state a head whose inputs are mixes of a token with the one
    before it. With h' the mixer's input one position earlier (zeros before a request's first
    token) each of r, k, v, g, w reads m_s = h + (h' - h) * mu_s. r, k, v = W_s m_s, cut into
    ``num_heads`` heads of ``head_dim``; gate = silu(W_g m_g); decay d = exp(-exp(w2 tanh(w1 m_w) +
    w0)), one number a head and key channel, w1 of ``decay_rank`` rows. A head with state S
    [head_dim, head_dim], zero at a request's start, float32: o = (S + diag(bonus) k v^T)^T r, then
    S <- diag(d) S + k v^T. Every head's o is divided by its root mean square (``norm_eps``); the
    concatenated heads are multiplied by a weight and by the gate, and projected back. The state a
    request keeps is the matrices and the last input row."""

    hidden_size: int
    num_heads: int
    head_dim: int
    decay_rank: int
    norm_eps: float

    def __post_init__(self):
        if min(self.hidden_size, self.num_heads, self.head_dim, self.decay_rank) < 1:
            raise ValueError("hidden_size, heads, head_dim and decay_rank must be positive")


@dataclass(frozen=True)
class StreamReentrySpec:
    """The stream made anew from itself and the model's input: x <- R [x; x0] + s_n, with x0 what
    the embedding part made of the step's tokens, R [hidden, 2 hidden] (x's columns first) and s
    [passes, hidden], n the number of the pass that begins (``RunEntry.reenter``)."""

    hidden_size: int
    passes: int

    def __post_init__(self):
        if self.hidden_size < 1 or self.passes < 1:
            raise ValueError("hidden_size and passes must be positive")


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A feed-forward made of ``num_experts`` small gated ones, E(u) = down(silu(gate u) * (up u)),
    no biases, of which every token uses ``top_k``: r = ``router``(W_r x) in float32 ("sigmoid":
    the logistic function of each logit by itself; "softmax": over the experts), the top_k
    largest r chosen (compared through their logits, which still differ where two r round to 1;
    the lower index first among equals), divided by their sum if
    ``renormalize``. ``weight_on`` "input": the result is the sum of E_e(r_e x); "output": the sum
    of r_e E_e(x).

    ``choice_correction``: a learned float32 number an expert joins r for the choice only; the
    weights stay r. ``groups`` (count, kept, top): the experts lie in ``count`` equal runs of
    neighbours; a run's score is the sum of its ``top`` largest choice scores and only experts of
    the ``kept`` best runs can be chosen. ``renorm_eps`` joins the sum that ``renormalize``
    divides by. ``shared_intermediate`` n: one more expert of inner width n runs for every token
    and its output is added, times logistic(w_sg x) (one number a token) if ``shared_gate``."""

    hidden_size: int
    intermediate_size: int
    num_experts: int
    top_k: int
    router: str = "sigmoid"
    renormalize: bool = False
    weight_on: str = "input"
    choice_correction: bool = False
    groups: Optional[tuple] = None
    renorm_eps: float = 0.0
    shared_intermediate: Optional[int] = None
    shared_gate: bool = False

    def __post_init__(self):
        if min(self.hidden_size, self.intermediate_size, self.num_experts) < 1:
            raise ValueError("hidden_size, intermediate_size and num_experts must be positive")
        if not 1 <= self.top_k <= self.num_experts:
            raise ValueError(f"top_k {self.top_k} must be between 1 and num_experts {self.num_experts}")
        if self.router not in ("sigmoid", "softmax"):
            raise ValueError(f"router {self.router!r}: expected 'sigmoid' or 'softmax'")
        if self.weight_on not in ("input", "output"):
            raise ValueError(f"weight_on {self.weight_on!r}: expected 'input' or 'output'")
        if self.groups is not None:
            if len(self.groups) != 3:
                raise ValueError(f"groups is (count, kept, top), got {self.groups!r}")
            count, kept, run_top = self.groups
            if count < 1 or self.num_experts % count or not 1 <= kept <= count or run_top < 1:
                raise ValueError(f"{self.num_experts} experts do not lie in {count} equal runs of which {kept} are kept")
            if (self.num_experts // count) * kept < self.top_k:
                raise ValueError(f"{kept} runs of {self.num_experts // count} experts cannot give {self.top_k} experts a token")
        if self.shared_intermediate is not None and self.shared_intermediate < 1:
            raise ValueError("the shared expert's inner width must be positive")
        if self.shared_gate and self.shared_intermediate is None:
            raise ValueError("a gate on the shared expert needs a shared expert")
