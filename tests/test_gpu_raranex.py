"""Raranex on the GPU against the plain implementation (tests/plain/raranex_plain.py): each new
mechanism alone (both attention mixers over many head geometries whole, in portions down to two
tokens and token by token; windows' edges and the kept first tokens with weights made so that one
key decides the output; a far key among hundreds; the shifted recurrence over several state shapes,
its state carried over hundreds of tokens; the router's correction, expert runs and shared expert;
the stream's re-entry; the block of two norms), then whole models of four small configurations
replayed whole, as prefill then single tokens, in portions and as mixed batches on tight page pools
and few state slots, in both dtypes; models drawn at random; long decoding as graph replays; greedy
generation through the engine's entry point, the command line and the trace program."""

import json
import subprocess
import sys
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

from clockwork_amd import ops
from clockwork_amd.parts.specs import (GatedAttentionSpec, PairMixerSpec, RMSNormSpec, RopePairsSpec, RoutedExpertsSpec,
                                       ShiftedRecurrenceSpec, StreamReentrySpec)
from clockwork_amd.registry import build_arrangement, build_part
from tests import replay
from tests.configs import RARANEX_CONFIGS, random_raranex_config
from tests.plain import raranex_plain as plain
from tests.test_gpu_fuvavik import _step_through, bind, close

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPO = Path(__file__).resolve().parents[1]
EPS = 1e-5


# ------------------------------------------------------------------------------- the two attention mixers
def _window_spec(hidden, heads, kv_heads, dim, vdim, window, keep_first, rot_dims, base=1000.0, scale=0.21):
    return GatedAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim, scale=scale,
                              norm_eps=EPS, window=window, keep_first=keep_first, qk_norm=True, qk_norm_weight=False,
                              qk_norm_after_rotation=True, position=RopePairsSpec(rot_dims, base) if rot_dims else None,
                              output_gate=True, gate_per_head=True)


def _capped_spec(hidden, heads, kv_heads, dim, vdim, softcap=4.0, coef=0.4, every=5, scale=0.21):
    return GatedAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim, scale=scale,
                              norm_eps=EPS, qk_norm=True, softcap=softcap, query_temperature=(coef, every), output_gate=True,
                              gate_per_head=True)


def _attention_names(w, spec):
    nq, nk, nv = spec.num_heads * spec.key_dim, spec.num_kv_heads * spec.key_dim, spec.num_kv_heads * spec.value_dim
    m = w["in_weight"]
    names = {"q": m[:nq], "k": m[nq : nq + nk], "v": m[nq + nk : nq + nk + nv], "g": m[nq + nk + nv :], "o": w["out_weight"]}
    if "q_norm" in w:
        names.update({"q.norm": w["q_norm"], "k.norm": w["k_norm"]})
    return names


def _window_sizes(spec):
    rot = {"base": spec.position.theta, "dims": spec.position.rotary_dim} if spec.position is not None else {"base": 1.0, "dims": 0}
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim, "scale": spec.scale,
            "mask": {"size": spec.window, "keep_first": spec.keep_first}, "rot": rot}


def _capped_sizes(spec):
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim, "scale": spec.scale,
            "softcap": spec.softcap, "q_temp": {"coef": spec.query_temperature[0], "every": spec.query_temperature[1]}}


CUTS = lambda T: ([T], [5, 1, 1, 17, 2, 1, 2, T - 29], [1] * T)  # noqa: E731

# heads, kv_heads, dim, vdim, window, kept first tokens, rotated elements, hidden: grouped heads, a
# group larger than a workgroup takes at once, sizes of 1 and 2, a window longer than the sequence
# and one of 1, more kept tokens than the window holds, rotation of all, a part and nothing
WINDOW_SHAPES = [(6, 2, 16, 24, 9, 3, 8, 96), (3, 1, 40, 8, 17, 1, 40, 100), (5, 5, 12, 20, 1, 4, 12, 64), (1, 1, 2, 1, 16, 0, 2, 48),
                 (4, 2, 24, 24, 300, 7, 0, 64), (20, 2, 8, 16, 12, 20, 4, 64), (8, 2, 64, 64, 33, 5, 32, 128),
                 (4, 4, 128, 64, 25, 2, 128, 64), (6, 3, 64, 64, 5, 9, 64, 66), (2, 1, 96, 48, 40, 40, 64, 72),
                 # nothing kept and keys and values of one size: in bfloat16 the kernels of plain grouped attention
                 (8, 2, 64, 64, 33, 0, 32, 128), (4, 4, 32, 32, 9, 0, 32, 64), (6, 1, 96, 96, 20, 0, 48, 72), (2, 2, 256, 256, 7, 0, 64, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", WINDOW_SHAPES)
def test_window_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, vdim, window, keep_first, rot_dims, hidden = shape
    spec = _window_spec(hidden, heads, kv_heads, dim, vdim, window, keep_first, rot_dims)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.15)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.window_attention(x.double(), _attention_names(w, spec), "", _window_sizes(spec), EPS)
    for cuts in CUTS(T):
        close(_step_through(part, part.cache_need(), x, cuts, dtype), want, dtype)


# heads, kv_heads, dim, vdim, hidden
CAPPED_SHAPES = [(8, 1, 24, 12, 96), (3, 3, 40, 8, 100), (1, 1, 2, 1, 48), (20, 2, 8, 16, 64), (8, 2, 64, 64, 128), (4, 4, 128, 64, 64),
                 (2, 1, 96, 48, 72), (5, 5, 12, 130, 64), (6, 2, 32, 32, 64), (3, 1, 160, 160, 40), (4, 2, 64, 256, 64), (16, 1, 16, 16, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", CAPPED_SHAPES)
def test_capped_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, vdim, hidden = shape
    spec = _capped_spec(hidden, heads, kv_heads, dim, vdim)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.15)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(5)).to(dtype)
    want = plain.capped_attention(x.double(), _attention_names(w, spec), "", _capped_sizes(spec), EPS)
    for cuts in CUTS(T):
        close(_step_through(part, part.cache_need(), x, cuts, dtype), want, dtype)


@pytest.mark.parametrize("kind", ["window", "capped"])
@pytest.mark.parametrize("shape", [(8, 2, 64, 64), (4, 1, 128, 128), (6, 3, 64, 128), (16, 2, 128, 64)])
def test_the_attention_kernels_agree_on_long_requests(kind, shape):
    """bfloat16, 700 tokens: the matrix-core kernels (for paged rows; for plain grouped heads where
    keys and values have one size and nothing is kept) against the plain-arithmetic kernel on the
    same steps and against the plain implementation, with the keys of single tokens and short
    portions cut into runs (a GPU of 256 compute units is what the plan sizes them by)."""
    heads, kv_heads, dim, vdim = shape
    hidden, T, dtype = 64, 700, torch.bfloat16
    if kind == "window":
        spec = _window_spec(hidden, heads, kv_heads, dim, vdim, 130, 70, 32)
        sizes, oracle = _window_sizes(spec), plain.window_attention
    else:
        spec = _capped_spec(hidden, heads, kv_heads, dim, vdim, softcap=3.0, coef=0.3, every=64)
        sizes, oracle = _capped_sizes(spec), plain.capped_attention
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(16)).to(dtype)
    outs = {}
    for kernel in ("fast", "arithmetic"):
        part = build_part(spec)
        w = bind(part, dtype, seed=3, matrix_std=0.2)
        assert part.plain == (kind == "capped" and dim == vdim) and part.rows_mfma == (not part.plain)
        if kernel == "arithmetic":
            part.plain = part.rows_mfma = False
            part.run = ops.rows_attention_tokens_per_item(heads, kv_heads, 1)
        for cuts in ([T], [600, 5, 2, 1, 1, 60] + [1] * 31):
            got = _step_through(part, part.cache_need(), x, cuts, dtype, block_size=16, num_blocks=64, compute_units=256)
            outs[(kernel, len(cuts))] = got
    want = oracle(x.double(), _attention_names(w, spec), "", sizes, EPS)
    for got in outs.values():
        close(got, want, dtype)


def test_the_attention_options_each_matter():
    """Every option of the two mixers switched off or changed by itself moves the output: the cap,
    the query's factor and its period, the kept tokens, the window, the order of norm and rotation
    (with weights), the pairing, the gate a head."""
    hidden, T = 64, 50
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(6))
    base = dict(hidden_size=hidden, num_heads=4, num_kv_heads=2, key_dim=16, value_dim=8, scale=0.6, norm_eps=EPS, qk_norm=True,
                output_gate=True, gate_per_head=True)
    variants = {
        "base": dict(base, softcap=2.0, query_temperature=(0.8, 4)),
        "no cap": dict(base, query_temperature=(0.8, 4)),
        "cap": dict(base, softcap=1.0, query_temperature=(0.8, 4)),
        "no factor": dict(base, softcap=2.0),
        "period": dict(base, softcap=2.0, query_temperature=(0.8, 9)),
    }
    outs = {}
    for key, kw in variants.items():
        part = build_part(GatedAttentionSpec(**kw))
        bind(part, torch.float32, seed=1, matrix_std=0.5)
        outs[key] = _step_through(part, part.cache_need(), x, [T], torch.float32)
    for key in variants:
        if key != "base":
            assert float((outs[key] - outs["base"]).abs().max()) > 1e-3, key
    wbase = dict(base, window=6, keep_first=3, position=RopePairsSpec(16, 50.0), qk_norm_after_rotation=True)
    variants = {
        "base": wbase,
        "nothing kept": dict(wbase, keep_first=0),
        "one more kept": dict(wbase, keep_first=4),
        "window": dict(wbase, window=7),
        "norm first": dict(wbase, qk_norm_after_rotation=False),
        "halves": dict(wbase, position=__import__("clockwork_amd.parts.specs", fromlist=["RopeNeoxSpec"]).RopeNeoxSpec(16, 50.0)),
        "no rotation": dict(wbase, position=None),
    }
    outs = {}
    for key, kw in variants.items():
        part = build_part(GatedAttentionSpec(**kw))
        bind(part, torch.float32, seed=2, matrix_std=0.5)
        outs[key] = _step_through(part, part.cache_need(), x, [T], torch.float32)
    for key in variants:
        if key != "base":
            assert float((outs[key] - outs["base"]).abs().max()) > 1e-3, key


def _loud_part(dim, window, keep_first, dtype, hidden=32, capped=False):
    """One head whose query is e0 for every token and whose key is ``10 * x[1] * e0``... made so:
    q reads input column 0, k input column 1, v input columns 2.. ; gate wide open; output = values."""
    vdim = 4
    if capped:
        spec = GatedAttentionSpec(hidden_size=hidden, num_heads=1, num_kv_heads=1, key_dim=dim, value_dim=vdim, scale=1.0, norm_eps=1e-12,
                                  qk_norm=False, softcap=30.0, output_gate=True, gate_per_head=True)
    else:
        spec = GatedAttentionSpec(hidden_size=hidden, num_heads=1, num_kv_heads=1, key_dim=dim, value_dim=vdim, scale=1.0, norm_eps=1e-12,
                                  window=window, keep_first=keep_first, qk_norm=False, output_gate=True, gate_per_head=True)
    part = build_part(spec)

    def change(values):
        m = torch.zeros_like(values["in_weight"])
        m[0, 0] = 1.0                      # q[0] = x[0]
        m[dim, 1] = 1.0                    # k[0] = x[1]
        for c in range(vdim):
            m[2 * dim + c, 2 + c] = 1.0    # v = x[2 : 2 + vdim]
        m[2 * dim + vdim, 6] = 1.0         # gate logit = x[6]
        values["in_weight"] = m
        o = torch.zeros_like(values["out_weight"])
        for c in range(vdim):
            o[c, c] = 1.0
        values["out_weight"] = o

    bind(part, dtype, change=change)
    return part, spec


def _loud_input(T, loud, hidden=32, score=16.0):
    """Every token asks with q = 1; the token at ``loud`` answers with a key of ``score``, all others
    with 0; the loud token's values are (1, 2, 3, 4), the others' 0; gates open (logit 16)."""
    x = torch.zeros(T, hidden)
    x[:, 0] = 1.0
    x[loud, 1] = score
    x[loud, 2:6] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    x[:, 6] = 16.0
    return x


@pytest.mark.parametrize("window, keep_first", [(1, 0), (5, 0), (16, 3), (17, 16), (40, 8), (4, 9)])
@pytest.mark.parametrize("cuts", ["whole", "portions", "single"])
def test_one_loud_key_at_the_windows_edge_and_among_the_kept_first_tokens(window, keep_first, cuts):
    """A key that takes all the weight wherever it is seen: just inside the window the output is
    its value, just outside it is nothing of it; the same for the last kept token and the first
    that is not kept. Pages of 8 tokens, given back behind the window while the request runs."""
    T = 75
    how = {"whole": [T], "portions": [3, 9, 2, 16, 5, 2, 31, 7], "single": [1] * T}[cuts]
    part, spec = _loud_part(8, window, keep_first, torch.float32)
    for loud in sorted({0, keep_first - 1, keep_first, 20, 33} - {-1}):
        x = _loud_input(T, loud)
        got = _step_through(part, part.cache_need(), x, how, torch.float32, block_size=8, num_blocks=16)
        for i in range(T):
            seen = loud <= i and (i - loud < window or loud < keep_first)
            want = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=torch.float64) if seen else torch.zeros(4, dtype=torch.float64)
            # unseen: the weight is shared by the silent keys, whose values are 0
            assert float((got[i, :4] - want).abs().max()) < 1e-4, (loud, i, got[i, :4])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_and_the_cap(dtype):
    """Position 3 holds the loud key, 700 tokens follow: every later token's output is its value
    as far as the cap lets the score stand out (cap 30: all of it)."""
    T = 703
    part, spec = _loud_part(8, None, 0, dtype, capped=True)
    x = _loud_input(T, 3, score=28.0)
    for cuts in ([T], [400] + [1] * (T - 400), [100, 2, 300, 301]):
        got = _step_through(part, part.cache_need(), x, cuts, dtype, block_size=16, num_blocks=48)
        want = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=torch.float64)
        assert float((got[3:, :4] - want).abs().max()) < (1e-4 if dtype == torch.float32 else 3e-2)
        assert float(got[:3, :4].abs().max()) < 1e-6


# ------------------------------------------------------------------------------- the shifted recurrence
def _recurrence_names(w, spec):
    inner, W = spec.num_heads * spec.head_dim, spec.hidden_size
    m = w["rkvg_weight"]
    names = {f"mu.{s}": w["mix"][i * W : (i + 1) * W] for i, s in enumerate(("r", "k", "v", "g", "w"))}
    names.update({"r": m[:inner], "k": m[inner : 2 * inner], "v": m[2 * inner : 3 * inner], "g": m[3 * inner :],
                  "w1": w["decay_in_weight"], "w2": w["decay_weight"], "w0": w["decay_bias"], "u": w["bonus"], "norm": w["norm_weight"],
                  "o": w["out_weight"]})
    return names


# heads, head size, rank, hidden: sizes that the segment kernels take and ones they do not
RECURRENCE_SHAPES = [(3, 16, 6, 96), (1, 18, 5, 100), (2, 4, 1, 48), (4, 32, 16, 64), (2, 64, 8, 128), (1, 128, 3, 72), (5, 8, 2, 64),
                     (1, 1, 1, 40)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", RECURRENCE_SHAPES)
def test_the_shifted_recurrence_whole_in_portions_and_token_by_token(dtype, shape):
    heads, dim, rank, hidden = shape
    if dim == 1 and dtype == torch.bfloat16:
        pytest.skip("a head of one element normed by itself is its sign: rounding flips it where the output is near 0")
    spec = ShiftedRecurrenceSpec(hidden_size=hidden, num_heads=heads, head_dim=dim, decay_rank=rank, norm_eps=EPS)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads + dim, matrix_std=0.2)
    T = 150
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(7)).to(dtype)
    want = plain.time_mixing(x.double(), _recurrence_names(w, spec), "", {"heads": heads, "dim": dim}, EPS)
    # whole (segments side by side where the state's shape allows), portions that end inside a
    # segment, down to two tokens, and single tokens
    for cuts in ([T], [5, 1, 1, 17, 2, 70, 2, 52], [100] + [1] * 50, [2] * 75):
        close(_step_through(part, part.cache_need(), x, cuts, dtype), want, dtype)


def test_the_recurrence_keeps_a_token_from_far_back_and_forgets_by_its_decay():
    """With the decay near one (bias -12: exp(-exp(-12))) what token 2 wrote is read 400 tokens
    later; with the decay near zero (bias 3) only the bonus term, the token itself, remains."""
    hidden, heads, dim, T = 32, 1, 8, 420
    outs = {}
    for bias in (-12.0, 3.0):
        spec = ShiftedRecurrenceSpec(hidden_size=hidden, num_heads=heads, head_dim=dim, decay_rank=2, norm_eps=EPS)
        part = build_part(spec)

        def change(values, bias=bias):
            values["decay_bias"] = torch.full_like(values["decay_bias"], bias)
            values["decay_weight"] = torch.zeros_like(values["decay_weight"])

        w = bind(part, torch.float32, seed=3, matrix_std=0.3, change=change)
        x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(8))
        names = _recurrence_names(w, spec)
        want = plain.time_mixing(x.double(), names, "", {"heads": heads, "dim": dim}, EPS)
        for cuts in ([T], [150, 2, 268], [300] + [1] * 120):
            close(_step_through(part, part.cache_need(), x, cuts, torch.float32), want, torch.float32)
        moved = x.clone()
        moved[2] += 1.0
        outs[bias] = float((plain.time_mixing(moved.double(), names, "", {"heads": heads, "dim": dim}, EPS) - want)[410:].abs().max())
    assert outs[-12.0] > 1e-3 and outs[3.0] < 1e-9


# ------------------------------------------------------------------------------- routed experts
def _routed_names(w, spec):
    E, F, H = spec.num_experts, spec.intermediate_size, spec.hidden_size
    gu = w["gate_up_weight"].view(E, 2, F, H)
    down = w["down_weight"].view(E, H, F)
    names = {"router": w["router_weight"][:E], "correction": w["correction"]}
    for e in range(E):
        names.update({f"e{e}.gate": gu[e, 0], f"e{e}.up": gu[e, 1], f"e{e}.down": down[e]})
    if spec.shared_intermediate is not None:
        S = spec.shared_intermediate
        names.update({"shared.gate": w["shared_gate_up_weight"][:S], "shared.up": w["shared_gate_up_weight"][S:],
                      "shared.down": w["shared_down_weight"], "shared.sg": w["router_weight"][E:]})
    return names


def _routed_mlp(spec):
    router = {"experts": spec.num_experts, "top": spec.top_k}
    if spec.groups is not None:
        router["groups"] = {"count": spec.groups[0], "keep": spec.groups[1]}
    return {"kind": "moe", "router": router, "shared": None if spec.shared_intermediate is None else {"ff": spec.shared_intermediate}}


# hidden, ff, experts, top, runs (count, kept) or None, shared width or None, tokens
ROUTED_SHAPES = [(96, 40, 6, 2, (3, 2), 48, 61), (100, 50, 4, 4, None, None, 37), (64, 1, 4, 1, (4, 2), 1, 9), (48, 24, 8, 3, (2, 1), 24, 130),
                 (128, 72, 16, 4, (4, 2), 64, 3), (64, 130, 7, 2, (1, 1), 10, 1), (72, 33, 40, 6, (8, 3), None, 20),
                 (128, 64, 4, 2, (2, 2), 128, 700)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ROUTED_SHAPES)
def test_routed_experts_with_correction_runs_and_a_shared_expert(dtype, shape):
    hidden, ff, experts, top, groups, shared, T = shape
    spec = RoutedExpertsSpec(hidden_size=hidden, intermediate_size=ff, num_experts=experts, top_k=top, renormalize=True,
                             weight_on="output", choice_correction=True, groups=None if groups is None else (*groups, 2),
                             renorm_eps=1e-20, shared_intermediate=shared, shared_gate=shared is not None)
    part = build_part(spec)

    def change(values):
        # corrections that are negative as well: a run that is not kept must count as minus
        # infinity, not as nothing
        values["correction"] = (values["correction"] * 6.0 - 0.7).to(torch.bfloat16).float()
        if dtype == torch.bfloat16:
            # rounded inputs flip close choices; here the corrections decide, far apart from one another
            values["correction"] = (torch.randperm(experts, generator=torch.Generator().manual_seed(1)).float() * 0.7 - 2.0)
            values["router_weight"][:experts] *= 0.05

    w = bind(part, dtype, seed=experts, matrix_std=1.5 / hidden ** 0.5, change=change)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(9)).to(dtype)
    names = _routed_names(w, spec)
    want = plain.routed_feed_forward(x.double(), names, "", _routed_mlp(spec))
    got = part.forward(x.to(DEV), SimpleNamespace()).double().cpu()
    close(got, want, dtype)
    chosen, weight = plain.routed_choice(x.double(), names, "", _routed_mlp(spec)["router"])
    choice, score, *_ = part.route(x.to(DEV))
    assert torch.equal(choice.cpu().long(), chosen)
    torch.testing.assert_close(score.double().cpu(), weight, rtol=2e-3 if dtype == torch.bfloat16 else 1e-5, atol=1e-6)


def test_the_routers_options_each_matter():
    hidden, T = 64, 40
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(10))
    base = dict(hidden_size=hidden, intermediate_size=24, num_experts=8, top_k=2, renormalize=True, weight_on="output",
                choice_correction=True, groups=(4, 2, 2), shared_intermediate=16, shared_gate=True)
    variants = {"base": base, "no runs": dict(base, groups=None), "one run kept": dict(base, groups=(4, 1, 2)),
                "runs by their best": dict(base, groups=(4, 2, 1)), "not renormalised": dict(base, renormalize=False),
                "no shared expert": dict(base, shared_intermediate=None, shared_gate=False), "no gate": dict(base, shared_gate=False)}
    outs = {}
    for key, kw in variants.items():
        part = build_part(RoutedExpertsSpec(**kw))
        gen = torch.Generator().manual_seed(11)
        params = {}
        for name, spec in part.param_specs().items():
            full = {"router_weight": (9, hidden)}.get(name, spec.shape)
            t = torch.randn(full, generator=gen) * (0.6 if name != "correction" else 0.8)
            params[name] = t[: spec.shape[0]].contiguous().to(DEV)
        part.bind(params, torch.device(DEV), torch.float32)
        outs[key] = part.forward(x.to(DEV), SimpleNamespace()).cpu()
    for key in variants:
        if key != "base":
            assert float((outs[key] - outs["base"]).abs().max()) > 1e-3, key


# ------------------------------------------------------------------------------- re-entry, the block, the pair
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, passes, T", [(100, 3, 37), (64, 1, 1), (256, 11, 300)])
def test_the_stream_re_entered_from_itself_and_the_input(dtype, hidden, passes, T):
    part = build_part(StreamReentrySpec(hidden, passes))
    w = bind(part, dtype, seed=passes, matrix_std=0.1)
    gen = torch.Generator().manual_seed(12)
    resid0, inp = torch.randn(T, hidden, generator=gen), torch.randn(T, hidden, generator=gen).to(dtype).float()
    a, b = (torch.randn(T, hidden, generator=gen)).to(dtype), (torch.randn(T, hidden, generator=gen)).to(dtype)
    for n in (0, passes - 1):
        for pending, extra in ((None, 0.0), (a.to(DEV), a.double()), (ops.PendingPair(a.to(DEV), b.to(DEV)), a.double() + b.double())):
            resid = resid0.clone().to(DEV)
            out = part.forward(resid, pending, inp.to(DEV), n, SimpleNamespace())
            assert out.dtype == torch.float32
            x = resid0.double() + extra
            torch.testing.assert_close(resid.double().cpu(), x, rtol=1e-6, atol=1e-6)   # what was pending has joined the old stream
            if dtype == torch.bfloat16:
                x = x.float().to(dtype).double()
            want = torch.cat([x, inp.double()], dim=-1) @ w["in_weight"].t() + w["step"][n]
            close(out.double().cpu(), want, dtype)
    with pytest.raises(ValueError):
        part.forward(resid0.to(DEV), None, inp.to(DEV), passes, SimpleNamespace())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_pair_of_capped_attention_and_recurrence(dtype):
    hidden = 72
    left = _capped_spec(hidden, 4, 2, 24, 16)
    right = ShiftedRecurrenceSpec(hidden_size=hidden, num_heads=3, head_dim=8, decay_rank=4, norm_eps=EPS)
    part = build_part(PairMixerSpec(hidden_size=hidden, left=left, right=right, eps=EPS))
    w = bind(part, dtype, seed=5, matrix_std=0.2)
    T = 90
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(13)).to(dtype)
    lw = {k[len("left."):]: v for k, v in w.items() if k.startswith("left.")}
    rw = {k[len("right."):]: v for k, v in w.items() if k.startswith("right.")}
    names = {"left." + k: v for k, v in _attention_names(lw, left).items()}
    names.update({"right." + k: v for k, v in _recurrence_names(rw, right).items()})
    names.update({"left.out": w["left_out_norm"], "right.out": w["right_out_norm"]})
    want = plain.side_by_side(x.double(), names, "", {"left": _capped_sizes(left), "right": {"heads": 3, "dim": 8}}, EPS)
    for cuts in ([T], [7, 2, 1, 70, 10], [1] * T):
        close(_step_through(part, part.cache_need(), x, cuts, dtype), want, dtype)


class _Twice:
    """A mixer or feed-forward that doubles or negates its input: shows which norm a branch read."""

    def __init__(self, factor):
        self.factor = factor

    def forward(self, x, ctx, cache=None):
        return (x.float() * self.factor).to(x.dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_block_of_two_norms_side_by_side(dtype):
    W, T = 96, 11
    n1, n2 = build_part(RMSNormSpec(W, 1e-3)), build_part(RMSNormSpec(W, 1e-3))
    w1, w2 = bind(n1, dtype, seed=1), bind(n2, dtype, seed=2)
    block = build_arrangement("twonorm", mixer=_Twice(2.0), mixer_norm=n1, feed_forward=_Twice(-0.5), ffn_norm=n2)
    gen = torch.Generator().manual_seed(14)
    x0 = torch.randn(T, W, generator=gen) * 3
    pending = (torch.randn(T, W, generator=gen)).to(dtype)
    for accepts in (True, False):
        resid = x0.clone().to(DEV)
        ctx = SimpleNamespace(next_norm_accepts_pending=accepts)
        out = block.forward(resid, pending.to(DEV), ctx, None)
        x = x0.double() + pending.double()
        a = 2.0 * plain.weighted_norm(x, w1["weight"], 1e-3)
        b = -0.5 * plain.weighted_norm(x, w2["weight"], 1e-3)
        if accepts:
            assert isinstance(out, ops.PendingPair)
            torch.testing.assert_close(resid.double().cpu(), x, rtol=1e-6, atol=1e-6)
            close(out.first.double().cpu(), a, dtype)
            close(out.second.double().cpu(), b, dtype)
        else:
            assert out is None
            close(resid.double().cpu(), x + a + b, dtype)


# ------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def raranex_dirs(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("raranex")
    return {name: write_random_model(root / name, cfg, seed) for name, (cfg, seed, _) in RARANEX_CONFIGS.items()}


def _requests(vocab, lengths, seed):
    gen = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=gen).tolist() for i, n in enumerate(lengths)}


def _check(got, ref, dtype, float32_bound=5e-5):
    """float32: element by element, which is the sharp test. bfloat16 on these small models:
    heads of a few elements that are divided by their own root mean square, and the pair's norms
    behind them, make single positions ill-conditioned under rounding (the plain implementation
    itself moves by a third of the logits' scale at such a position when only the recurrence's
    projections are rounded to bfloat16), so the errors are held by their distribution over the
    positions: half of them within 5 % of the scale and nine in ten within 15 %, where a wrong key,
    window, state or slot moves every position behind it by the scale itself. The kernels that
    only bfloat16 runs are held to the usual bounds part by part, above."""
    if dtype == "float32":
        replay.compare(got, ref, rtol=float32_bound, atol=float32_bound)
        return
    keys = sorted(got)
    want = torch.stack([ref[rid][pos] for rid, pos in keys]).float()
    rows = torch.stack([got[k] for k in keys])
    assert not bool(torch.isnan(rows).any()), "NaN in the logits"
    scale = float(want.square().mean().sqrt())
    per_row = (rows - want).abs().max(dim=1).values / scale
    half, most = float(per_row.quantile(0.5)), float(per_row.quantile(0.9))
    assert half < 5e-2 and most < 1.5e-1, f"errors against the scale: median {half:.3f}, nine in ten within {most:.3f}"


def _settle_the_choice(model_dir):
    """For bfloat16 runs: the routers scaled down and the corrections spread far apart, so that
    the rounding of a router's input does not flip a choice (which a comparison of logits cannot
    tell from a fault); the weights still follow the router."""
    from safetensors.torch import load_file, save_file

    path = str(Path(model_dir) / "model.safetensors")
    tensors = load_file(path)
    for key in list(tensors):
        if key.endswith("mlp.router"):
            tensors[key] = (tensors[key].float() * 0.05).to(tensors[key].dtype)
        if key.endswith("mlp.correction"):
            # unevenly spaced, so that no two pairs of them have the same sum (a run's score is one)
            n = tensors[key].numel()
            order = torch.randperm(n, generator=torch.Generator().manual_seed(n)).float()
            tensors[key] = (order * 0.6 + order * order * 0.05 - 1.0).to(tensors[key].dtype)
    save_file(tensors, path)


@pytest.fixture(scope="module")
def settled_dirs(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("raranex_settled")
    dirs = {}
    for name, (cfg, seed, _) in RARANEX_CONFIGS.items():
        dirs[name] = write_random_model(root / name, cfg, seed)
        _settle_the_choice(dirs[name])
    return dirs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
@pytest.mark.parametrize("name", list(RARANEX_CONFIGS))
def test_models_in_four_batching_modes(raranex_dirs, settled_dirs, name, mode, dtype):
    cfg, _, block_size = RARANEX_CONFIGS[name]
    model_dir = (settled_dirs if dtype == "bfloat16" else raranex_dirs)[name]
    requests = _requests(cfg["vocab"], [50, 9, 77, 30, 64, 1, 2], seed=11)
    # pages for the four longest requests and two more, four state slots: freed pages and slots are
    # used again (NaN-poisoned pools: a read outside a request's pages shows)
    runner = replay.make_runner(model_dir, dtype, block_size, replay.pages_needed(requests, 4, block_size) + 2)
    oracle = plain.PlainRaranex(model_dir)
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    assert len(got) == sum(len(t) for t in requests.values())
    _check(got, ref, dtype)
    assert not runner.manager.live_requests()
    assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("seed", range(3000, 3006))
def test_models_drawn_at_random(tmp_path, seed):
    """Models whose sizes, layer order, repeated run and constants are drawn at random, six requests
    of 1 to 420 tokens on pages of 64 barely enough for four of them, as mixed batches, in portions
    and as prefill then single tokens; float32 as the model stands, bfloat16 with the experts'
    choice settled by the corrections."""
    import random

    from clockwork_amd.weights.random_init import write_random_model

    cfg = random_raranex_config(seed)
    rng = random.Random(seed)
    lengths = [rng.randint(100, 420), rng.randint(2, 90), rng.randint(200, 330), rng.randint(40, 300), 1, 65]
    for dtype in ("float32", "bfloat16"):
        model_dir = write_random_model(tmp_path / dtype, cfg, seed)
        if dtype == "bfloat16":
            _settle_the_choice(model_dir)
        requests = _requests(cfg["vocab"], lengths, seed)
        oracle = plain.PlainRaranex(model_dir)
        ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
        for mode in ("mixed", "portions", "prefill_then_decode"):
            runner = replay.make_runner(model_dir, dtype, 64, replay.pages_needed(requests, 4, 64) + 1)
            got = replay.run_trace(runner, getattr(replay, mode)(requests))
            assert len(got) == sum(len(t) for t in requests.values())
            # up to ten layer runs of random weights: float32 sums of hundreds of terms, amplified
            _check(got, ref, dtype, float32_bound=2e-4)
            assert not runner.manager.live_requests()


def test_the_stream_after_every_layer_run(raranex_dirs):
    """Float32, one request: the residual stream after every layer run (a repeated layer counts
    each time) against the plain implementation's; what a block leaves pending is added first."""
    cfg, _, block_size = RARANEX_CONFIGS["RA"]
    runner = replay.make_runner(raranex_dirs["RA"], "float32", block_size, 16)
    tokens = _requests(cfg["vocab"], [40], seed=2)["q0"]
    seen = []
    for layer in runner.model.layers:
        inner = layer.forward

        def forward(resid, delta, ctx, cache, inner=inner):
            out = inner(resid, delta, ctx, cache)
            total = resid.clone()
            for part in ((out.first, out.second) if isinstance(out, ops.PendingPair) else (out,)):
                if part is not None:
                    total += part.float()
            seen.append(total.cpu())
            return out

        layer.forward = forward
    replay.run_trace(runner, replay.whole({"a": tokens}))
    want = plain.PlainRaranex(raranex_dirs["RA"]).streams(tokens)
    assert len(seen) == want.shape[0] == 5
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, rtol=3e-5, atol=3e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_replays_graphs_and_equals_eager_steps(raranex_dirs, settled_dirs, dtype):
    """A prompt, then 150 single tokens (windows of 9 and 33 pass over decoded tokens, pages behind
    them are given back, the kept first pages stay): with captured graphs, against the same steps
    run eagerly and against the plain implementation; two requests decode side by side."""
    cfg, _, block_size = RARANEX_CONFIGS["RA"]
    model_dir = (settled_dirs if dtype == "bfloat16" else raranex_dirs)["RA"]
    requests = _requests(cfg["vocab"], [200, 170], seed=12)
    steps = [{"entries": [{"id": rid, "tokens": toks[:20], "want": [19]}], "end": []} for rid, toks in requests.items()]
    for p in range(20, 170):
        steps.append({"entries": [{"id": rid, "tokens": toks[p : p + 1], "want": [0]} for rid, toks in requests.items()], "end": []})
    steps[-1]["end"] = list(requests)
    oracle = plain.PlainRaranex(model_dir)
    ref = {rid: oracle.logits(toks[:170]) for rid, toks in requests.items()}
    results = {}
    for graphs in (True, False):
        runner = replay.make_runner(model_dir, dtype, block_size, 64, use_graphs=graphs)
        results[graphs] = replay.run_trace(runner, steps)
        if graphs:
            assert any(isinstance(v, tuple) for v in runner._graphs.values()), "no decode step was captured"
        _check(results[graphs], ref, dtype)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=1e-5, atol=1e-5)


def test_greedy_generation_through_the_engine(raranex_dirs):
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    oracle = plain.PlainRaranex(raranex_dirs["RA"])
    prompts = [[3, 14, 15, 92, 65], list(range(100, 160)), [7], list(range(40))]
    want = [oracle.greedy(p, 8) for p in prompts]
    cfg = EngineConfig.defaults(str(raranex_dirs["RA"]), dtype="float32", block_size=8, num_blocks=64, max_num_batched_tokens=24)
    engine = LLMEngine(cfg)
    outs = engine.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    # once more on the same engine: pages and state slots of the first round are used again
    outs = engine.generate(prompts[::-1], SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want[::-1]


def test_the_command_line_and_the_trace_program(raranex_dirs, tmp_path):
    oracle = plain.PlainRaranex(raranex_dirs["RD"])
    prompt = [5, 17, 3, 60, 1]
    out = subprocess.run([sys.executable, str(REPO / "bin" / "clockwork-generate"), "--model", str(raranex_dirs["RD"]),
                          "--set", "dtype=float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5"],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert json.loads(out.stdout.splitlines()[-1])["token_ids"] == oracle.greedy(prompt, 5), out.stdout
    tokens = _requests(90, [45], seed=13)["q0"]
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": tokens[30:32], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": tokens[32:], "want": [12]}], "end": ["a"]})]
    run = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(raranex_dirs["RD"]), "--dtype", "float32",
                          "--out", str(tmp_path / "out"), "--max-tokens", "64"], input="\n".join(lines) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np

    ref = oracle.logits(tokens)
    first = torch.from_numpy(np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(2, -1))
    last = torch.from_numpy(np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (tmp_path / "out" / "1.f32").exists()
    torch.testing.assert_close(first, ref[[0, 29]], rtol=3e-5, atol=3e-5)
    torch.testing.assert_close(last, ref[[44]], rtol=3e-5, atol=3e-5)
