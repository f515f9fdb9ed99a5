"""Nenodra on the GPU against the plain implementation (tests/plain/nenodra_plain.py): each new
kernel and part alone, then whole models of three small configurations replayed whole, as prefill
then single tokens, in portions down to two tokens and as mixed batches on tight page pools, in
both dtypes; windows' edges and far keys with weights made so that one key decides the output;
experts chosen among equals; long decoding; forks; greedy generation through the engine's entry
point, the command line and the trace program."""

import json
import subprocess
import sys
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

from clockwork_amd import ops
from clockwork_amd.parts.specs import (BranchRMSNormSpec, DenseMLPSpec, DifferentialAttentionSpec, GatedAttentionSpec,
                                       LinearHeadSpec, RopeNeoxSpec, RoutedExpertsSpec)
from clockwork_amd.registry import build_part
from tests import replay
from tests.configs import NENODRA_CONFIGS
from tests.plain import nenodra_plain as plain
from tests.test_gpu_fuvavik import _step_through, bind, close

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPO = Path(__file__).resolve().parents[1]


# ------------------------------------------------------------------------------- norm, feed-forward, head
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [100, 257, 1024])
def test_the_norm_on_a_branch_on_the_stream_and_the_streams_image(dtype, width):
    part = build_part(BranchRMSNormSpec(size=width, eps=3e-4, branch_scale=0.3, weight_offset=1.0))
    w = bind(part, dtype, seed=width)
    gen = torch.Generator().manual_seed(1)
    T = 37
    resid0 = torch.randn(T, width, generator=gen) * 2
    branch = (torch.randn(T, width, generator=gen) * 5).to(dtype)
    # the stream's image alone: nothing is added
    resid = resid0.clone().to(DEV)
    image = part.image(resid)
    assert image.dtype == dtype
    torch.testing.assert_close(image.float().cpu(), resid0.to(dtype).float(), rtol=0, atol=0)
    torch.testing.assert_close(resid.cpu(), resid0, rtol=0, atol=0)
    # a branch joins: the float32 stream takes 0.3 * N(branch), the image is the stream rounded once
    image = part.join(resid, branch.to(DEV))
    summed = resid0.double() + 0.3 * plain.output_norm(branch.double(), w["weight"], 3e-4)
    torch.testing.assert_close(resid.cpu().double(), summed, rtol=1e-6, atol=2e-6)
    assert image.dtype == dtype
    torch.testing.assert_close(image.float().cpu(), resid.cpu().to(dtype).float(), rtol=0, atol=0)
    # the norm of the stream itself, of all rows and of chosen rows; the stream stays
    before = resid.clone()
    close(part.forward(resid, ops.StreamImage(image)).double().cpu(), plain.output_norm(summed, w["weight"], 3e-4), dtype)
    rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)
    close(part.forward(resid, None, rows=rows).double().cpu(), plain.output_norm(summed[[5, 0, 36]], w["weight"], 3e-4), dtype)
    assert torch.equal(resid, before)
    with pytest.raises(TypeError):
        part.forward(resid, branch.to(DEV))


def test_the_norms_constants_each_matter():
    x = torch.randn(5, 64, generator=torch.Generator().manual_seed(2))
    got = {}
    for key, spec in {"base": BranchRMSNormSpec(64, 1e-2, 0.5, 1.0), "offset": BranchRMSNormSpec(64, 1e-2, 0.5, 0.0),
                      "eps": BranchRMSNormSpec(64, 1.0, 0.5, 1.0), "scale": BranchRMSNormSpec(64, 1e-2, 1.0, 1.0)}.items():
        part = build_part(spec)
        w = bind(part, torch.float32, seed=3)
        resid = torch.zeros(5, 64, device=DEV)
        part.join(resid, (0.3 * x).to(DEV))
        got[key] = resid.cpu().double()
        want = spec.branch_scale * plain.unit_rms(0.3 * x.double(), spec.eps) * (spec.weight_offset + w["weight"])
        torch.testing.assert_close(got[key], want, rtol=1e-5, atol=1e-6)
    for key in ("offset", "eps", "scale"):
        assert float((got[key] - got["base"]).abs().max()) > 5e-2, key


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, rows", [(100, 41), (128, 8), (128, 1), (1024, 3), (128, 200)])
def test_squared_relu_feed_forward(dtype, hidden, rows):
    part = build_part(DenseMLPSpec(hidden_size=hidden, intermediate_size=72, activation="relu2"))
    w = bind(part, dtype, seed=2, matrix_std=0.05)
    x = torch.randn(rows, hidden, generator=torch.Generator().manual_seed(3)).to(dtype)
    got = part.forward(x.to(DEV), SimpleNamespace()).double().cpu()
    close(got, plain.dense_feed_forward(x.double(), {"up": w["up_weight"], "down": w["down_weight"]}, ""), dtype)
    if dtype == torch.bfloat16 and rows == 200:
        # the same activation in the epilogues of the up product: of the weight-streaming kernel
        # (few rows) and of the wide-tile kernel (a long portion of a wide layer), against the
        # product followed by the activation kernel
        for m, k, n in [(5, 256, 8704), (40, 512, 8704), (1100, 256, 8704), (1030, 384, 8650)]:
            gen = torch.Generator().manual_seed(m)
            a = torch.randn(m, k, generator=gen).to(dtype).to(DEV)
            wt = (torch.randn(n, k, generator=gen) / k ** 0.5).to(dtype).to(DEV)
            want = torch.relu(a.double() @ wt.double().t()).square().cpu()
            scale = float(want.square().mean().sqrt())
            for got in (ops.linear_relu_squared(a, wt), ops.relu_squared_(ops.linear(a, wt))):
                # squares reach far above their scale: an element is held to its own size
                assert bool(((got.double().cpu() - want).abs() <= 1.5e-2 * want.abs() + 1e-2 * scale).all())
    z = torch.tensor([-3.0, -0.0, 0.0, 0.5, 2.0, 64.0]).to(dtype).to(DEV)
    torch.testing.assert_close(ops.relu_squared_(z).float().cpu(), torch.tensor([0.0, 0.0, 0.0, 0.25, 4.0, 4096.0]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_head_with_a_factor_on_its_logits(dtype):
    head = build_part(LinearHeadSpec(vocab_size=77, hidden_size=40, scale=0.37))
    w = bind(head, dtype, matrix_std=0.3)
    rows = torch.randn(5, 40, generator=torch.Generator().manual_seed(4)).to(dtype)
    got = head.forward(rows.to(DEV), None)
    assert got.dtype == torch.float32
    close(got.double().cpu(), 0.37 * (rows.double() @ w["weight"].t()), dtype)


# ------------------------------------------------------------------------------- routed feed-forward
def _expert_names(w, spec):
    E, F, H = spec.num_experts, spec.intermediate_size, spec.hidden_size
    gu = w["gate_up_weight"].view(E, 2, F, H)
    down = w["down_weight"].view(E, H, F)
    names = {"router": w["router_weight"]}
    for e in range(E):
        names.update({f"e{e}.gate": gu[e, 0], f"e{e}.up": gu[e, 1], f"e{e}.down": down[e]})
    return names


# hidden, ff, experts, top, tokens: one expert, all experts, more experts than tokens, more tokens of
# an expert than a tile of rows holds, sizes that are no multiple of the kernels' tiles
ROUTED_SHAPES = [(96, 40, 5, 2, 61), (100, 50, 2, 1, 37), (64, 1, 1, 1, 9), (48, 24, 3, 3, 130), (128, 72, 16, 4, 3),
                 (224, 104, 9, 1, 200), (64, 130, 7, 2, 1), (72, 33, 40, 6, 20), (128, 64, 4, 2, 700), (72, 40, 6, 2, 33),
                 (200, 152, 3, 1, 400)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ROUTED_SHAPES)
def test_routed_experts_against_the_plain_sum(dtype, shape):
    hidden, ff, experts, top, T = shape
    spec = RoutedExpertsSpec(hidden_size=hidden, intermediate_size=ff, num_experts=experts, top_k=top)
    part = build_part(spec)
    w = bind(part, dtype, seed=experts, matrix_std=1.5 / hidden ** 0.5)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(5)).to(dtype)
    names = _expert_names(w, spec)
    mlp = {"router": {"top": top}}
    chosen, score = plain.routed_choice(x.double(), names, "", top)
    choice, got_score = part.route(x.to(DEV))
    if dtype == torch.float32:
        assert torch.equal(choice.cpu().long(), chosen)
        torch.testing.assert_close(got_score.cpu().double(), score, rtol=1e-5, atol=1e-6)
        got = part.forward(x.to(DEV), SimpleNamespace()).double().cpu()
        close(got, plain.routed_feed_forward(x.double(), names, "", mlp), dtype)
        return
    # bfloat16: the router's sums are float32 over the same rounded inputs, so a choice can differ
    # from float64's only between scores that are equal to five digits; the result is compared
    # through the experts that the engine chose
    r = plain.logistic(x.double() @ names["router"].t())
    want = torch.zeros(T, hidden, dtype=torch.float64)
    for t in range(T):
        mine = choice[t].tolist()
        if sorted(mine) != sorted(chosen[t].tolist()):
            assert float(score[t].min() - r[t][mine].min()) < 1e-5, f"token {t}: {mine} against {chosen[t].tolist()}"
        torch.testing.assert_close(got_score[t].cpu().double(), r[t][mine], rtol=1e-5, atol=1e-6)
        for e in mine:
            want[t] += plain.expert(r[t, e] * x[t].double(), names, f"e{e}.")
    close(part.forward(x.to(DEV), SimpleNamespace()).double().cpu(), want, dtype)


@pytest.mark.parametrize("shape", [(72, 40, 6, 2, 33), (128, 64, 4, 2, 700), (200, 152, 3, 1, 400), (192, 88, 10, 3, 5), (64, 8, 2, 2, 130)])
def test_the_three_kernels_of_the_experts_products_agree(shape):
    """bfloat16: plain arithmetic, the streaming kernel and the wide tiles of the matrix cores on the
    same step, each forced; they round alike and differ by the order of their float32 sums. Which
    one a step takes by itself follows from its shape alone."""
    hidden, ff, experts, top, T = shape
    spec = RoutedExpertsSpec(hidden_size=hidden, intermediate_size=ff, num_experts=experts, top_k=top)
    part = build_part(spec)
    w = bind(part, torch.bfloat16, seed=experts, matrix_std=1.5 / hidden ** 0.5)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(15)).to(torch.bfloat16).to(DEV)
    names = _expert_names(w, spec)
    choice, score = part.route(x)
    want = torch.zeros(T, hidden, dtype=torch.float64)
    for t in range(T):
        for e, r in zip(choice[t].tolist(), score[t].tolist()):
            want[t] += plain.expert(r * x[t].double().cpu(), names, f"e{e}.")
    got = {}
    for kernel in ("plain", "stream", "wide"):
        part.kernel = kernel
        got[kernel] = part.forward(x, SimpleNamespace()).double().cpu()
        close(got[kernel], want, torch.bfloat16)
    scale = float(want.square().mean().sqrt())
    for kernel in ("stream", "wide"):
        assert float((got[kernel] - got["plain"]).abs().max()) < 2e-2 * scale
    assert ops.moe_kernel_for(torch.bfloat16, 16, 8, 1536, 4480) == "stream"
    assert ops.moe_kernel_for(torch.bfloat16, 1024, 8, 1536, 4480) == "wide"
    assert ops.moe_kernel_for(torch.bfloat16, 4096, 8, 1536, 4480) == "grouped"
    assert ops.moe_kernel_for(torch.bfloat16, 4096, 8, 1536, 4488) == "wide"
    assert ops.moe_kernel_for(torch.float32, 4096, 8, 1536, 4480) == "plain"
    assert ops.moe_kernel_for(torch.bfloat16, 4096, 8, 100, 4480) == "plain"


@pytest.mark.parametrize("weight_on", ["input", "output"])
@pytest.mark.parametrize("shape", [(256, 384, 3, 2, 700), (320, 256, 5, 1, 300), (512, 256, 2, 2, 1030), (256, 256, 6, 3, 90)])
def test_the_experts_as_row_tiles_of_the_dense_products_kernel(shape, weight_on):
    """bfloat16, widths that are multiples of 64: the rows laid out expert by expert in tiles of 256
    and multiplied by the wide-tile kernel of the dense products, every tile with its expert's
    matrices; experts with more than a tile of rows, with a part of one, with none (the router of
    one expert is turned away from every token). Against the plain sum and the plain-arithmetic
    kernel, with the score on the expert's input and on its output."""
    hidden, ff, experts, top, T = shape
    spec = RoutedExpertsSpec(hidden_size=hidden, intermediate_size=ff, num_experts=experts, top_k=top, weight_on=weight_on)
    part = build_part(spec)

    def change(v):
        if experts > top + 1:
            v["router_weight"][experts - 2] = -8.0 * v["router_weight"][experts - 2].abs()   # with inputs > 0: never chosen

    w = bind(part, torch.bfloat16, seed=experts + 1, matrix_std=1.5 / hidden ** 0.5, change=change)
    x = (torch.randn(T, hidden, generator=torch.Generator().manual_seed(16)).abs() + 0.05).to(torch.bfloat16).to(DEV)
    names = _expert_names(w, spec)
    choice, score = part.route(x)
    if experts > top + 1:
        assert not bool((choice == experts - 2).any())
    want = torch.zeros(T, hidden, dtype=torch.float64)
    for t in range(T):
        for e, r in zip(choice[t].tolist(), score[t].tolist()):
            xt = x[t].double().cpu()
            want[t] += (r * plain.expert(xt, names, f"e{e}.") if weight_on == "output"
                        else plain.expert((r * xt).to(torch.bfloat16).double(), names, f"e{e}."))
    got = {}
    for kernel in ("plain", "grouped"):
        part.kernel = kernel
        got[kernel] = part.forward(x, SimpleNamespace()).double().cpu()
        close(got[kernel], want, torch.bfloat16)
    scale = float(want.square().mean().sqrt())
    # both round a value to bfloat16 once: they differ by the order of their float32 sums, which
    # moves an element by one step of its last bit at most
    assert float(((got["grouped"] - got["plain"]).abs() / (got["plain"].abs() + scale)).max()) < 2e-2
    # a second step of other tokens through the same part: fewer rows, other experts' tiles
    x2 = x[: max(T // 3, 1)].flip(0).contiguous()
    part.kernel = "plain"
    want2 = part.forward(x2, SimpleNamespace()).double().cpu()
    part.kernel = "grouped"
    assert float(((part.forward(x2, SimpleNamespace()).double().cpu() - want2).abs() / (want2.abs() + scale)).max()) < 2e-2


def test_routing_options_and_equal_scores():
    """The lower index wins among equal scores; the score weighs the expert's input, not its
    output (the experts are not linear, so the two differ); no renormalisation; each can be set
    otherwise by another design."""
    hidden, ff, experts, top = 64, 24, 6, 2
    x = torch.randn(11, hidden, generator=torch.Generator().manual_seed(6))
    results = {}
    for key, options in {"base": {}, "output": {"weight_on": "output"}, "renorm": {"renormalize": True},
                         "softmax": {"router": "softmax"}}.items():
        spec = RoutedExpertsSpec(hidden_size=hidden, intermediate_size=ff, num_experts=experts, top_k=top, **options)
        part = build_part(spec)

        def change(v):
            v["router_weight"][4] = v["router_weight"][1]      # experts 1 and 4 always score the same
            v["router_weight"][1] *= 3.0
            v["router_weight"][4] *= 3.0

        w = bind(part, torch.float32, seed=8, matrix_std=0.3, change=change)
        names = _expert_names(w, spec)
        choice, score = part.route(x.to(DEV))
        z = x.double() @ names["router"].t()
        r = torch.softmax(z, -1) if key == "softmax" else plain.logistic(z)
        order = torch.sort(r, dim=-1, descending=True, stable=True).indices[:, :top]
        assert torch.equal(choice.cpu().long(), order)
        rows = choice.cpu().tolist()
        assert any(row == [1, 4] for row in rows) and not any(row[0] == 4 and row[1] == 1 for row in rows)
        s = torch.gather(r, 1, order)
        if key == "renorm":
            s = s / s.sum(-1, keepdim=True)
        torch.testing.assert_close(score.cpu().double(), s, rtol=1e-5, atol=1e-6)
        want = torch.zeros(11, hidden, dtype=torch.float64)
        for t in range(11):
            for e, c in zip(order[t].tolist(), s[t]):
                want[t] += (c * plain.expert(x[t].double(), names, f"e{e}.") if key == "output"
                            else plain.expert(c * x[t].double(), names, f"e{e}."))
        results[key] = part.forward(x.to(DEV), SimpleNamespace()).double().cpu()
        torch.testing.assert_close(results[key], want, rtol=2e-5, atol=2e-5)
    for key in ("output", "renorm", "softmax"):
        assert float((results[key] - results["base"]).abs().max()) > 1e-2, key


def test_a_steps_experts_replay_as_a_graph():
    """Routing, the rows sorted by expert and the experts' products stay on the device: a captured
    step replays with other inputs, which choose other experts."""
    spec = RoutedExpertsSpec(hidden_size=64, intermediate_size=40, num_experts=5, top_k=2)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=9, matrix_std=0.3)
    names = _expert_names(w, spec)
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(19, 64, generator=gen).to(DEV)
    part.forward(x, SimpleNamespace())                       # libraries loaded before the capture
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            out = part.forward(x, SimpleNamespace())
    for _ in range(3):
        fresh = torch.randn(19, 64, generator=gen)
        x.copy_(fresh.to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        want = plain.routed_feed_forward(fresh.double(), names, "", {"router": {"top": 2}})
        torch.testing.assert_close(out.double().cpu(), want, rtol=2e-5, atol=2e-5)
        eager = part.forward(x, SimpleNamespace())
        torch.testing.assert_close(out, eager, rtol=0, atol=0)


# ------------------------------------------------------------------------------- the two mixers
def _two_map_spec(hidden, heads, kv_heads, dim, vdim, window, rot_dims, base=1000.0, scale=0.21, diff=0.35, eps=1e-5):
    return DifferentialAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim,
                                     scale=scale, lambda_init=diff, norm_eps=eps, window=window, qkv_bias=True, qk_norm=True,
                                     position=RopeNeoxSpec(rotary_dim=rot_dims, theta=base) if rot_dims else None, out_bias=True)


def _two_map_names(w, spec):
    nq = spec.num_heads * 2 * spec.key_dim
    nk = spec.num_kv_heads * 2 * spec.key_dim
    qkv, b = w["qkv_weight"], w["qkv_bias"]
    out = {"q": qkv[:nq], "k": qkv[nq : nq + nk], "v": qkv[nq + nk :], "q.b": b[:nq], "k.b": b[nq : nq + nk], "v.b": b[nq + nk :],
           "o": w["out_weight"], "o.b": w["out_bias"], "q.norm": w["q_norm"], "k.norm": w["k_norm"]}
    out.update({n: w[n] for n in ("lq1", "lk1", "lq2", "lk2")})
    return out


def _rot(spec):
    return {"base": spec.position.theta if spec.position else 1.0, "dims": spec.position.rotary_dim if spec.position else 0}


def _two_map_sizes(spec):
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim,
            "scale": spec.scale, "diff": spec.lambda_init, "mask": {"size": spec.window}, "rot": _rot(spec)}


def _gated_spec(hidden, heads, kv_heads, dim, window, rot_dims, base=1000.0, scale=0.21, eps=1e-5):
    return GatedAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=dim, scale=scale,
                              norm_eps=eps, window=window, qk_norm=True,
                              position=RopeNeoxSpec(rotary_dim=rot_dims, theta=base) if rot_dims else None, values="keys",
                              output_gate=True)


def _gated_names(w, spec):
    nq, nk = spec.num_heads * spec.key_dim, spec.num_kv_heads * spec.key_dim
    m = w["in_weight"]
    return {"q": m[:nq], "k": m[nq : nq + nk], "g": m[nq + nk :], "o": w["out_weight"], "q.norm": w["q_norm"], "k.norm": w["k_norm"]}


def _gated_sizes(spec):
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim,
            "scale": spec.scale, "mask": {"size": spec.window}, "rot": _rot(spec)}


# heads, kv_heads, dim, vdim, window, rotated elements, hidden: grouped heads, a group larger than a
# workgroup takes at once, sizes of 1, a window longer than the sequence and one of 1, rotation of
# all, of a part and of nothing
TWO_MAP_SHAPES = [(4, 2, 24, 16, 9, 12, 64), (6, 6, 16, 16, 33, 16, 96), (3, 1, 40, 24, 300, 2, 100), (2, 1, 8, 32, 1, 8, 48),
                  (1, 1, 32, 8, 17, 0, 48), (20, 2, 8, 20, 12, 4, 64), (2, 2, 64, 130, 16, 64, 64), (8, 2, 64, 128, 40, 32, 128),
                  (4, 2, 128, 128, 40, 128, 64), (3, 1, 128, 64, 16, 64, 64), (2, 1, 64, 256, 25, 64, 64), (10, 2, 64, 64, 21, 48, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", TWO_MAP_SHAPES)
def test_two_map_window_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, vdim, window, rot_dims, hidden = shape
    spec = _two_map_spec(hidden, heads, kv_heads, dim, vdim, window, rot_dims)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.15)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.two_map_window_attention(x.double(), _two_map_names(w, spec), "", _two_map_sizes(spec), 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 32], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)


# heads, kv_heads, dim, window, rotated elements, hidden; in bfloat16 the head sizes that are a
# multiple of 32 run on the kernels of plain grouped attention, the others on the kernel for paged rows
GATED_SHAPES = [(6, 2, 16, 9, 8, 96), (3, 1, 40, 17, 40, 100), (5, 5, 12, 1, 12, 64), (1, 1, 2, 16, 2, 48), (4, 2, 24, 300, 0, 64),
                (20, 2, 8, 12, 4, 64), (8, 2, 64, 33, 32, 128), (4, 4, 128, 25, 128, 64), (6, 2, 32, 5, 16, 64), (2, 1, 96, 40, 64, 72)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", GATED_SHAPES)
def test_gated_window_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, window, rot_dims, hidden = shape
    spec = _gated_spec(hidden, heads, kv_heads, dim, window, rot_dims)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.15)
    assert part.plain == (dtype == torch.bfloat16 and dim % 32 == 0)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.keys_as_values_attention(x.double(), _gated_names(w, spec), "", _gated_sizes(spec), 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 32], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)


def test_gated_attention_with_values_and_biases_of_its_own():
    """The part's other options (a value projection, biases, no gate, no norm, no window), which
    this design does not use, against the same equations written out here."""
    hidden, heads, kv_heads, dim, vdim = 64, 4, 2, 16, 24
    spec = GatedAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim, scale=0.3,
                              norm_eps=1e-5, window=None, qk_norm=False, position=RopeNeoxSpec(rotary_dim=8, theta=100.0),
                              values="projection", output_gate=False, qkv_bias=True, out_bias=True)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=3, matrix_std=0.2)
    T = 45
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(8))
    proj = x.double() @ w["in_weight"].t() + w["in_bias"]
    nq, nk = heads * dim, kv_heads * dim
    pos = list(range(T))
    q = plain.rotate_first(proj[:, :nq].reshape(T, heads, dim), pos, 100.0, 8)
    k = plain.rotate_first(proj[:, nq : nq + nk].reshape(T, kv_heads, dim), pos, 100.0, 8)
    v = proj[:, nq + nk :].reshape(T, kv_heads, vdim)
    outs = [plain.windowed_softmax_rows(q[:, a], k[:, a // 2], 0.3, T + 1) @ v[:, a // 2] for a in range(heads)]
    want = torch.cat(outs, -1) @ w["out_weight"].t() + w["out_bias"]
    for cuts in ([T], [3, 1, 20, 2, 19]):
        got = _step_through(part, part.cache_need(), x, cuts, torch.float32)
        torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)


def test_the_mixers_options_each_matter():
    """lambda, the biases, the norms' weights, the rotation, the window, the values' source and the
    gate each change the result by much more than the tolerance."""
    spec = _two_map_spec(64, 4, 2, 24, 16, 9, 12)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=7, matrix_std=0.15)
    x = torch.randn(30, 64, generator=torch.Generator().manual_seed(5))
    got = _step_through(part, part.cache_need(), x, [30], torch.float32)
    base, sizes = _two_map_names(w, spec), _two_map_sizes(spec)
    torch.testing.assert_close(got, plain.two_map_window_attention(x.double(), base, "", sizes, 1e-5), rtol=2e-5, atol=2e-5)
    for change in ({"lq1": base["lq1"] + 1.0}, {"q.b": base["q.b"] + 1.5 * (torch.arange(base["q.b"].numel()) % 3 - 1)},
                   {"v.b": base["v.b"] + 0.5}, {"o.b": base["o.b"] + 0.1}, {"q.norm": base["q.norm"] * 0 + 1.0},
                   {"k.norm": base["k.norm"].flip(0)}):
        other = plain.two_map_window_attention(x.double(), dict(base, **change), "", sizes, 1e-5)
        assert float((other - got).abs().max()) > 1e-2, list(change)
    for change in ({"diff": 0.6}, {"mask": {"size": 10}}, {"mask": {"size": 8}}, {"scale": 0.4}, {"rot": {"base": 1000.0, "dims": 8}},
                   {"rot": {"base": 10.0, "dims": 12}}):
        other = plain.two_map_window_attention(x.double(), base, "", dict(sizes, **change), 1e-5)
        assert float((other - got).abs().max()) > 1e-2, list(change)
    # the one-map mixer
    spec = _gated_spec(64, 6, 2, 16, 9, 8)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=7, matrix_std=0.15)
    got = _step_through(part, part.cache_need(), x, [30], torch.float32)
    base, sizes = _gated_names(w, spec), _gated_sizes(spec)
    torch.testing.assert_close(got, plain.keys_as_values_attention(x.double(), base, "", sizes, 1e-5), rtol=2e-5, atol=2e-5)
    for change in ({"g": base["g"] * 0}, {"q.norm": base["q.norm"] * 0 + 1.0}, {"k.norm": base["k.norm"].flip(0)}):
        other = plain.keys_as_values_attention(x.double(), dict(base, **change), "", sizes, 1e-5)
        assert float((other - got).abs().max()) > 3e-3, list(change)
    for change in ({"mask": {"size": 10}}, {"mask": {"size": 8}}, {"scale": 0.4}, {"rot": {"base": 1000.0, "dims": 16}},
                   {"rot": {"base": 10.0, "dims": 8}}):
        other = plain.keys_as_values_attention(x.double(), base, "", dict(sizes, **change), 1e-5)
        assert float((other - got).abs().max()) > 3e-3, list(change)
    # values that were the normed and rotated keys instead of the raw projections would show
    T = x.shape[0]
    q = plain.normed_rotated((x.double() @ base["q"].t()).view(T, 6, 16), base["q.norm"], 1e-5, list(range(T)), sizes["rot"])
    k = plain.normed_rotated((x.double() @ base["k"].t()).view(T, 2, 16), base["k.norm"], 1e-5, list(range(T)), sizes["rot"])
    heads = [plain.windowed_softmax_rows(q[:, a], k[:, a // 3], spec.scale, 9) @ k[:, a // 3] for a in range(6)]
    other = (torch.cat(heads, -1) * plain.logistic(x.double() @ base["g"].t())) @ base["o"].t()
    assert float((other - got).abs().max()) > 3e-3


def _loud_two_map_part(hidden, dim, vdim, window, dtype):
    """A layer in which one marked token decides the output of every later token whose window
    holds it: input element 0 marks the loud token (it alone sets the last key channel of the first
    map and value channel 0); element 1, which every token carries, sets the last query channel of
    the first map and value channel 1. After the norm the marked key and every query have length
    sqrt(dim), all other keys are zero; the rotation leaves the last channel alone (half of the
    vector is rotated). The second map's scores are all equal, lambda is its constant, 0.5. While
    the loud key is seen the normed output points along value channel 0, else along channel 1."""
    spec = _two_map_spec(hidden, 2, 1, dim, vdim, window, dim // 2, scale=1.0, diff=0.5, eps=1e-6)
    part = build_part(spec)
    c = dim - 1

    def change(v):
        for name in ("qkv_weight", "qkv_bias", "lq1", "lk1", "lq2", "lk2", "out_weight", "out_bias"):
            v[name].zero_()
        v["q_norm"].fill_(1.0)
        v["k_norm"].fill_(1.0)
        nq, nk = 2 * 2 * dim, 2 * dim
        v["qkv_weight"][c, 1] = 6.0                 # head 0, map 0, last channel
        v["qkv_weight"][2 * dim + c, 1] = 6.0       # head 1, map 0, last channel
        v["qkv_weight"][nq + c, 0] = 1.0            # key, map 0, last channel
        v["qkv_weight"][nq + nk, 0] = 1.0           # value channel 0
        v["qkv_weight"][nq + nk + 1, 1] = 1.0       # value channel 1
        v["out_weight"][0, 0] = 1.0                 # head 0's channel 0
        v["out_weight"][1, vdim] = 1.0              # head 1's channel 0
        v["out_weight"][2, 1] = 1.0                 # head 0's channel 1

    return spec, part, bind(part, dtype, change=change)


def _loud_gated_part(hidden, dim, window, dtype):
    """The same for the one-map mixer, whose values are the key projections before the norm:
    element 0 of the input sets the marked token's last key channel to 4, element 1 gives every
    token a key of 0.05 in the channel before it (so no norm divides by zero) and every query its
    last channel. The gate is one half everywhere. The output's element 0 (head 0) and 1 (head 1)
    read value channel dim - 1: 4 while the marked key is seen, 0 after."""
    spec = _gated_spec(hidden, 2, 1, dim, window, dim // 2, scale=1.0, eps=1e-6)
    part = build_part(spec)
    c = dim - 1

    def change(v):
        v["in_weight"].zero_()
        v["out_weight"].zero_()
        v["q_norm"].fill_(1.0)
        v["k_norm"].fill_(1.0)
        v["in_weight"][c, 1] = 1.0                  # query head 0, last channel
        v["in_weight"][dim + c, 1] = 1.0            # query head 1, last channel
        v["in_weight"][2 * dim + c, 0] = 1.0        # key, last channel
        v["in_weight"][2 * dim + c - 1, 1] = 0.05   # a small key for every token
        v["out_weight"][0, c] = 2.0                 # head 0's last value channel (the gate halves it)
        v["out_weight"][1, dim + c] = 2.0           # head 1's
        v["out_weight"][2, c - 1] = 2.0

    return spec, part, bind(part, dtype, change=change)


def _loud(kind, hidden, dim, window, dtype, vdim=8):
    if kind == "attention":
        spec, part, w = _loud_two_map_part(hidden, dim, vdim, window, dtype)
        return part, lambda x: plain.two_map_window_attention(x, _two_map_names(w, spec), "", _two_map_sizes(spec), 1e-6)
    spec, part, w = _loud_gated_part(hidden, dim, window, dtype)
    return part, lambda x: plain.keys_as_values_attention(x, _gated_names(w, spec), "", _gated_sizes(spec), 1e-6)


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
@pytest.mark.parametrize("window", [1, 5, 16, 17, 40])
@pytest.mark.parametrize("cuts", ["whole", "portions", "single"])
def test_one_loud_key_just_inside_and_just_outside_the_window(kind, window, cuts):
    """The loud token sits at position 3: every token up to position 3 + window - 1 must show it,
    the next one and all after it must not. Pages of 4 and 8 tokens put the edge at page borders and
    inside pages; pages behind the window are given back and used again."""
    hidden, dim = 32, 16
    part, want_of = _loud(kind, hidden, dim, window, torch.float32)
    T, loud = 70, 3
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    want = want_of(x.double())
    # the plain result itself shows the edge
    last = loud + window - 1
    assert float(want[last, 0]) > 1.0 and abs(float(want[last + 1, 0])) < 1e-5 and abs(float(want[loud - 1, 0])) < 1e-5
    for block_size in (4, 8):
        steps = {"whole": [T], "portions": [2, 7, 3, 16, 5, 2, 31, 4], "single": [loud + 2] + [1] * (T - loud - 2)}[cuts]
        got = _step_through(part, part.cache_need(), x, steps, torch.float32, block_size=block_size, num_blocks=24)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_decides_the_output(kind, dtype):
    """The same loud key behind a window of 400: it is one of 400 keys that the last query that
    sees it has, 399 positions back, and gone at the next. In bfloat16 these head sizes run on the
    matrix cores, and single tokens behind long contexts share their keys among workgroups."""
    hidden, dim, window = 32, 64, 400
    part, want_of = _loud(kind, hidden, dim, window, dtype, vdim=64)
    if dtype == torch.bfloat16:
        assert part.mfma if kind == "attention" else part.plain
    T, loud = 450, 7
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    want = want_of(x.double())
    assert float(want[loud + window - 1, 0]) > 2.5 and abs(float(want[loud + window, 0])) < 1e-5
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for steps in ([T], [2, 300, 7, 64, 29, 33, 15], [390] + [1] * 60):
        got = _step_through(part, part.cache_need(), x, steps, dtype, block_size=16, num_blocks=40)
        torch.testing.assert_close(got, want, **tol)


# ------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def nenodra_dirs(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("nenodra")
    return {name: write_random_model(root / name, cfg, seed) for name, (cfg, seed, _) in NENODRA_CONFIGS.items()}


def _requests(vocab, lengths, seed):
    gen = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=gen).tolist() for i, n in enumerate(lengths)}


def _check(got, ref, dtype):
    if dtype == "float32":
        replay.compare(got, ref, rtol=3e-5, atol=3e-5)
    else:
        replay.compare_to_scale(got, ref, rms_bound=3e-2, worst_bound=1.5e-1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
@pytest.mark.parametrize("name", list(NENODRA_CONFIGS))
def test_models_in_four_batching_modes(nenodra_dirs, name, mode, dtype):
    cfg, _, block_size = NENODRA_CONFIGS[name]
    requests = _requests(cfg["vocab"], [50, 9, 77, 30, 64, 1, 2], seed=11)
    # pages for the four longest requests and two more: freed pages are used again (NaN-poisoned
    # pools: a read outside a request's pages shows)
    runner = replay.make_runner(nenodra_dirs[name], dtype, block_size, replay.pages_needed(requests, 4, block_size) + 2)
    oracle = plain.PlainNenodra(nenodra_dirs[name])
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    assert len(got) == sum(len(t) for t in requests.values())
    _check(got, ref, dtype)
    assert not runner.manager.live_requests()
    assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("seed", range(2000, 2010))
def test_models_drawn_at_random(tmp_path, seed):
    """Ten models whose sizes, layer order and constants are drawn at random, six requests of 1 to
    420 tokens on pages of 64 barely enough for four of them, as mixed batches, in portions and as
    prefill then single tokens. float32 against the plain implementation as the model stands (its
    routers scaled down, so that no logit lies where the logistic function is flat and few choices
    are close calls); bfloat16 with the routed layers made dense, because a rounded router input
    flips close choices, which a comparison of logits cannot tell from a fault."""
    import copy
    import random

    from safetensors.torch import load_file, save_file

    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import random_nenodra_config

    cfg = random_nenodra_config(seed)
    dense = copy.deepcopy(cfg)
    for entry in dense["layers"]:
        if entry["mlp"] is not None and entry["mlp"]["kind"] == "moe":
            entry["mlp"] = {"kind": "dense", "ff": 2 * entry["mlp"]["expert"]["ff"]}
    rng = random.Random(seed)
    lengths = [rng.randint(100, 420), rng.randint(2, 90), rng.randint(200, 330), rng.randint(40, 300), 1, 65]
    for dtype, config in (("float32", cfg), ("bfloat16", dense)):
        model_dir = write_random_model(tmp_path / dtype, config, seed)
        path = str(Path(model_dir) / "model.safetensors")
        tensors = load_file(path)
        for key in tensors:
            if key.endswith("mlp.router"):
                tensors[key] = (tensors[key].float() * 0.05).to(tensors[key].dtype)
        save_file(tensors, path)
        requests = _requests(config["vocab"], lengths, seed)
        oracle = plain.PlainNenodra(model_dir)
        ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
        for mode in ("mixed", "portions", "prefill_then_decode"):
            runner = replay.make_runner(model_dir, dtype, 64, replay.pages_needed(requests, 4, 64) + 1)
            got = replay.run_trace(runner, getattr(replay, mode)(requests))
            assert len(got) == sum(len(t) for t in requests.values())
            _check(got, ref, dtype)
            assert not runner.manager.live_requests()


def test_the_stream_after_every_layer(nenodra_dirs):
    """Float32, one request: the residual stream after every layer against the plain implementation's."""
    cfg, _, block_size = NENODRA_CONFIGS["NA"]
    runner = replay.make_runner(nenodra_dirs["NA"], "float32", block_size, 16)
    tokens = _requests(cfg["vocab"], [40], seed=2)["q0"]
    seen = []
    for layer in runner.model.layers:
        inner = layer.forward

        def forward(resid, delta, ctx, cache, inner=inner):
            out = inner(resid, delta, ctx, cache)
            seen.append(resid.clone().cpu())       # nothing is pending behind a block of this kind
            return out

        layer.forward = forward
    replay.run_trace(runner, replay.whole({"a": tokens}))
    want = plain.PlainNenodra(nenodra_dirs["NA"]).streams(tokens)
    assert len(seen) == want.shape[0] == 4
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_through_layers_of_unlike_sizes(tmp_path, dtype):
    """1400 and 333 tokens through five layers that share no size: windows of 77 to 1500 pass over
    hundreds of tokens of prompts and of decoded tokens, sixteen experts of which a token uses four;
    whole, prefill then single tokens, portions of 2 to 512 tokens, and mixed."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import NENODRA_LONG

    model_dir = write_random_model(tmp_path / "long", NENODRA_LONG, 5)
    requests = _requests(211, [1400, 333], seed=3)
    oracle = plain.PlainNenodra(model_dir)
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    for mode in ("whole", "prefill_then_decode", "portions", "mixed"):
        runner = replay.make_runner(model_dir, dtype, 16, 120, max_model_len=1600)
        if dtype == "bfloat16":
            fast = [getattr(m, "mfma", None) if hasattr(m, "mfma") else m.plain for m in runner.model.mixers()]
            assert fast == [False, True, True, True, False]
        steps = replay.portions(requests, sizes=[2, 300, 7, 64, 129, 33, 512]) if mode == "portions" else getattr(replay, mode)(requests)
        got = replay.run_trace(runner, steps)
        if dtype == "float32":
            _check(got, ref, dtype)
        else:
            # A token whose fourth and fifth expert score alike goes to another expert once its
            # input is rounded to bfloat16, and moves by the size of an expert's output: with
            # sixteen experts and 1700 tokens there are some. So rounding is judged by the median
            # row, which a wrong mask or page would move as well, and the whole by a wider bound;
            # the float32 run of the same trace is exact to the element
            keys = sorted(got)
            want = torch.stack([ref[rid][pos] for rid, pos in keys]).float()
            rows = torch.stack([got[k] for k in keys])
            assert not torch.isnan(rows).any()
            scale = float(want.square().mean().sqrt())
            per_row = (rows - want).square().mean(dim=1).sqrt()
            assert float(per_row.median()) < 3e-2 * scale and float(per_row.square().mean().sqrt()) < 1e-1 * scale, (
                f"{mode}: median row error {float(per_row.median()):.3e}, rms {float(per_row.square().mean().sqrt()):.3e}, "
                f"scale {scale:.3e}")
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("name", ["NA", "NB"])
def test_random_traces_with_forks(nenodra_dirs, name):
    """Random traces (portions of 2 to 200 tokens and single tokens in any mix, requests left out of
    steps, forks cut at any token: shared pages copied on the first write) on pools little larger
    than four requests, in float32."""
    cfg, _, _ = NENODRA_CONFIGS[name]
    oracle = plain.PlainNenodra(nenodra_dirs[name])
    for seed in range(6):
        steps, seqs = replay.random_trace(seed, cfg["vocab"], kinds=("fork",))
        block_size = (4, 8, 16)[seed % 3]
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(nenodra_dirs[name], "float32", block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: oracle.logits(toks) for rid, toks in seqs.items()}
        replay.compare(got, ref, rtol=3e-5, atol=3e-5)
        assert not runner.manager.live_requests()
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_replays_graphs_and_equals_eager_steps(nenodra_dirs, dtype):
    """A prompt, then 150 single tokens (windows of 5 to 33 pass over decoded tokens, pages behind
    them are given back): with captured graphs, against the same steps run eagerly and against the
    plain implementation; two requests decode side by side."""
    cfg, _, block_size = NENODRA_CONFIGS["NA"]
    requests = _requests(cfg["vocab"], [200, 170], seed=12)
    steps = [{"entries": [{"id": rid, "tokens": toks[:20], "want": [19]}], "end": []} for rid, toks in requests.items()]
    for p in range(20, 170):
        steps.append({"entries": [{"id": rid, "tokens": toks[p : p + 1], "want": [0]} for rid, toks in requests.items()], "end": []})
    steps[-1]["end"] = list(requests)
    oracle = plain.PlainNenodra(nenodra_dirs["NA"])
    ref = {rid: oracle.logits(toks[:170]) for rid, toks in requests.items()}
    results = {}
    for graphs in (True, False):
        runner = replay.make_runner(nenodra_dirs["NA"], dtype, block_size, 64, use_graphs=graphs)
        results[graphs] = replay.run_trace(runner, steps)
        if graphs:
            assert any(isinstance(v, tuple) for v in runner._graphs.values()), "no decode step was captured"
        _check(results[graphs], ref, dtype)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=1e-5, atol=1e-5)


def test_greedy_generation_through_the_engine(nenodra_dirs):
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    oracle = plain.PlainNenodra(nenodra_dirs["NA"])
    prompts = [[3, 14, 15, 92, 65], list(range(100, 160)), [7], list(range(40))]
    want = [oracle.greedy(p, 8) for p in prompts]
    cfg = EngineConfig.defaults(str(nenodra_dirs["NA"]), dtype="float32", block_size=8, num_blocks=64, max_num_batched_tokens=24)
    engine = LLMEngine(cfg)
    outs = engine.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    # once more on the same engine: pages of the first round are used again
    outs = engine.generate(prompts[::-1], SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want[::-1]


def test_the_command_line_and_the_trace_program(nenodra_dirs, tmp_path):
    oracle = plain.PlainNenodra(nenodra_dirs["NC"])
    prompt = [5, 17, 3, 60, 1]
    out = subprocess.run([sys.executable, str(REPO / "bin" / "clockwork-generate"), "--model", str(nenodra_dirs["NC"]),
                          "--set", "dtype=float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5"],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert json.loads(out.stdout.splitlines()[-1])["token_ids"] == oracle.greedy(prompt, 5), out.stdout
    tokens = _requests(64, [45], seed=13)["q0"]
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": tokens[30:32], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": tokens[32:], "want": [12]}], "end": ["a"]})]
    run = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(nenodra_dirs["NC"]), "--dtype", "float32",
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
