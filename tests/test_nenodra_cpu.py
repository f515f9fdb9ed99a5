"""Nenodra without a GPU: the configuration reader and what it refuses, the weight plan against
the tensors a checkpoint of the design holds, cache groups whose pages are given back behind a
window, and invariants of the plain implementation that the GPU tests lean on (a window's edge,
both mixers against dense masked matrices written another way, rotation, the routed feed-forward
against a dense sum over all experts)."""

import copy

import pytest
import torch

from clockwork_amd.cache.manager import NO_PAGE, CacheManager, cache_needs_of, plan_groups
from clockwork_amd.parts.model import DecoderModel, model_param_specs
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import check_plan
from clockwork_amd.weights.random_init import write_random_model
from tests.configs import NENODRA_A, NENODRA_B, NENODRA_C, NENODRA_LONG
from tests.plain import nenodra_plain as plain


def _describe(config):
    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    spec = arch.build_spec(cfg)
    return arch, cfg, spec, arch.weight_plan(cfg, spec)


def test_the_design_is_found_and_every_constant_is_read():
    arch, cfg, spec, _ = _describe(NENODRA_A)
    assert arch.name == "Nenodra" and spec.architecture == "Nenodra"
    assert (cfg.vocab, cfg.width, cfg.residual_mult, cfg.logit_scale, cfg.eps) == (300, 96, 0.7, 1.3, 1e-5)
    assert not spec.tie_embeddings and spec.head.scale == 1.3
    n = spec.final_norm
    assert (n.size, n.eps, n.branch_scale, n.weight_offset) == (96, 1e-5, 0.7, 1.0)
    assert [e.layer for e in spec.run] == [0, 1, 2, 3]
    a, b, c, d = spec.layers
    assert all(l.arrangement == "branchnorm" for l in spec.layers)
    m = a.mixer
    assert type(m).__name__ == "GatedAttentionSpec"
    assert (m.num_heads, m.num_kv_heads, m.key_dim, m.value_dim, m.scale, m.window, m.norm_eps) == (6, 2, 16, 16, 0.2, 9, 1e-5)
    assert (m.values, m.output_gate, m.qk_norm, m.qkv_bias, m.position.rotary_dim, m.position.theta) == ("keys", True, True, False, 8, 100.0)
    f = a.feed_forward
    assert (f.intermediate_size, f.num_experts, f.top_k, f.router, f.renormalize, f.weight_on) == (40, 5, 2, "sigmoid", False, "input")
    m = b.mixer
    assert type(m).__name__ == "DifferentialAttentionSpec"
    assert (m.num_heads, m.num_kv_heads, m.key_dim, m.value_dim, m.scale, m.lambda_init, m.window, m.segment) == \
        (4, 2, 8, 24, 0.3, 0.3, 33, None)
    assert (m.qk_norm, m.qkv_bias, m.out_bias, m.position.rotary_dim, m.position.theta) == (True, True, True, 8, 1000.0)
    assert (b.feed_forward.intermediate_size, b.feed_forward.activation) == (72, "relu2")
    assert c.mixer.lambda_init == 0.8 and c.mixer.window == 5 and c.feed_forward.top_k == 3
    assert d.feed_forward is None and d.ffn_norm is None and d.mixer.position.rotary_dim == 40
    # a layer that rotates nothing has no position encoding at all
    assert _describe(NENODRA_B)[2].layers[2].mixer.position is None


@pytest.mark.parametrize("path, value, error", [
    (("layers", 0, "type"), "recurrent", NotImplementedError),
    (("layers", 1, "mlp", "kind"), "gated", NotImplementedError),
    (("layers", 0, "mixer", "kv_heads"), 4, ValueError),
    (("layers", 0, "mixer", "mask"), None, ValueError),
    (("layers", 0, "mixer", "vdim"), 24, ValueError),        # the one-map mixer's values are its keys
    (("layers", 1, "mixer", "diff"), None, ValueError),
    (("layers", 1, "mixer", "rot"), None, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 7, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 10, ValueError),
    (("layers", 0, "mlp", "router", "top"), 6, ValueError),
    (("layers", 0, "mlp", "router", "top"), 0, ValueError),
    (("layers", 0, "mlp", "expert"), None, ValueError),
    (("layers", 1, "mlp", "ff"), 0, ValueError),
    (("norm",), None, ValueError),
    (("residual_mult",), None, ValueError),
    (("logit_scale",), None, ValueError),
    (("layers",), [], ValueError),
    (("width",), 0, ValueError),
])
def test_what_the_configuration_reader_refuses(path, value, error):
    config = copy.deepcopy(NENODRA_A)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(error):
        _describe(config)


def _tensor_names(config):
    """Names and shapes of a checkpoint of the design, written out from the layer list."""
    W = config["width"]
    names = {"embed": (config["vocab"], W), "head": (config["vocab"], W), "final.norm": (W,)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        names.update({p + "norm1": (W,), p + "mix.q.norm": (D,), p + "mix.k.norm": (D,), p + "mix.o": (W, H * V)})
        if layer["type"] == "attention":
            names.update({p + "mix.q": (H * 2 * D, W), p + "mix.q.b": (H * 2 * D,), p + "mix.k": (G * 2 * D, W),
                          p + "mix.k.b": (G * 2 * D,), p + "mix.v": (G * V, W), p + "mix.v.b": (G * V,), p + "mix.o.b": (W,)})
            names.update({p + "mix." + n: (D,) for n in ("lq1", "lk1", "lq2", "lk2")})
        else:
            names.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.g": (H * V, W)})
        mlp = layer["mlp"]
        if mlp is None:
            continue
        names[p + "norm2"] = (W,)
        if mlp["kind"] == "dense":
            names.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            ff = mlp["expert"]["ff"]
            names[p + "mlp.router"] = (mlp["router"]["experts"], W)
            for e in range(mlp["router"]["experts"]):
                names.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
    return names


@pytest.mark.parametrize("config", [NENODRA_A, NENODRA_B, NENODRA_C, NENODRA_LONG])
def test_the_weight_plan_names_every_tensor_of_the_design(config):
    _, _, spec, plan = _describe(config)
    names = _tensor_names(config)
    assert check_plan(names, plan) == ([], [], [])
    specs = model_param_specs(spec)
    assert {t.param for t in plan} == set(specs)
    missing, unexpected, _ = check_plan({k: v for k, v in names.items() if k != "l0.mix.k.norm"} | {"l0.mix.extra": (3,)}, plan)
    assert missing == ["l0.mix.k.norm"] and unexpected == ["l0.mix.extra"]
    # stacked parameters have one row for every row of their sources
    for target in plan:
        assert specs[target.param].shape[0] == sum(shape[0] for shape in target.source_shapes)


def test_the_experts_matrices_are_stacked_expert_by_expert():
    _, _, _, plan = _describe(NENODRA_A)
    by_param = {t.param: t for t in plan}
    assert by_param["layers.0.feed_forward.gate_up_weight"].sources[:4] == ("l0.mlp.e0.gate", "l0.mlp.e0.up", "l0.mlp.e1.gate", "l0.mlp.e1.up")
    assert by_param["layers.0.feed_forward.down_weight"].sources == tuple(f"l0.mlp.e{e}.down" for e in range(5))
    assert by_param["layers.0.mixer.in_weight"].sources == ("l0.mix.q", "l0.mix.k", "l0.mix.g")
    assert by_param["layers.1.mixer.qkv_bias"].sources == ("l1.mix.q.b", "l1.mix.k.b", "l1.mix.v.b")


def test_random_models_hold_what_the_plain_reader_needs(tmp_path):
    for name, config in (("a", NENODRA_A), ("b", NENODRA_B), ("c", NENODRA_C)):
        folder = write_random_model(tmp_path / name, config, 5)
        oracle = plain.PlainNenodra(folder)
        assert set(oracle.w) == set(_tensor_names(config))
        logits = oracle.logits([1, 2, 3, 4, 5])
        assert logits.shape == (5, config["vocab"]) and torch.isfinite(logits).all()
        assert oracle.streams([1, 2, 3]).shape == (len(config["layers"]), 3, config["width"])


def test_cache_groups_and_pages_given_back_behind_the_window():
    model = DecoderModel(_describe(NENODRA_A)[2])
    groups = plan_groups(cache_needs_of(model.spec, model.mixers()))
    assert [(g.window, g.segment, g.entries) for g in groups] == [(9, None, (0,)), (33, None, (1,)), (5, None, (2,)), (17, None, (3,))]
    assert [[name for name, _ in g.need.planes] for g in groups] == [["k", "v"]] * 4
    assert [tuple(shape for _, shape in g.need.planes) for g in groups[:2]] == [((2, 16), (2, 16)), ((2, 16), (2, 24))]
    manager = CacheManager(groups, block_size=4, num_blocks=40, max_num_seqs=4)
    assert not manager.supports_prefix_sharing
    manager.admit("s", 70, portion_end=30)
    manager.extend("s", 0, 30)
    manager.release_behind_window("s", 30)
    rec = manager.record("s")
    # the next token, position 30, sees 22.. in group 0, 26.. in group 2 and everything in group 1
    assert rec.released[0] == 22 // 4 and all(p == NO_PAGE for p in rec.tables[0][: 22 // 4]) and rec.tables[0][22 // 4] != NO_PAGE
    assert rec.released[2] == 26 // 4 and rec.released[1] == 0 and rec.released[3] == 14 // 4
    manager.free("s")
    assert all(p.num_free == 40 for p in manager.pools)


# ------------------------------------------------------------------------------- the plain implementation
def _rand(seed):
    gen = torch.Generator().manual_seed(seed)
    return lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)


def _two_map_weights(H, G, D, V, W, seed):
    r = _rand(seed)
    w = {"q": r(H * 2 * D, W) * 0.3, "q.b": r(H * 2 * D) * 0.1, "k": r(G * 2 * D, W) * 0.3, "k.b": r(G * 2 * D) * 0.1,
         "v": r(G * V, W) * 0.3, "v.b": r(G * V) * 0.1, "o": r(W, H * V) * 0.2, "o.b": r(W) * 0.1,
         "q.norm": 1 + r(D) * 0.2, "k.norm": 1 + r(D) * 0.2}
    w.update({n: r(D) * 0.2 for n in ("lq1", "lk1", "lq2", "lk2")})
    return w


def _gated_weights(H, G, D, W, seed):
    r = _rand(seed)
    return {"q": r(H * D, W) * 0.3, "k": r(G * D, W) * 0.3, "g": r(H * D, W) * 0.3, "o": r(W, H * D) * 0.2,
            "q.norm": 1 + r(D) * 0.2, "k.norm": 1 + r(D) * 0.2}


def _turn(v, pos, base, dims):
    """Rotation written pair by pair with complex numbers."""
    out = v.clone()
    for i in range(dims // 2):
        angle = torch.as_tensor(pos, dtype=torch.float64) * base ** (-2.0 * i / dims)
        z = torch.complex(v[..., i], v[..., i + dims // 2]) * torch.polar(torch.ones_like(angle), angle).reshape(-1, *[1] * (v.dim() - 2))
        out[..., i], out[..., i + dims // 2] = z.real, z.imag
    return out


def test_plain_rotation_against_complex_numbers_and_what_stays():
    v = _rand(1)(6, 3, 10)
    pos = [0, 1, 5, 17, 100, 1000]
    got = plain.rotate_first(v, pos, 50.0, 6)
    torch.testing.assert_close(got, _turn(v, pos, 50.0, 6))
    torch.testing.assert_close(got[..., 6:], v[..., 6:])       # past rot.dims nothing moves
    torch.testing.assert_close(got[0], v[0])                   # position 0 turns nothing
    assert plain.rotate_first(v, pos, 50.0, 0) is v


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_plain_mixers_see_exactly_their_window(kind):
    H, G, D, V, W, S = 2, 1, 8, 6, 16, 7
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.4, "diff": 0.3, "mask": {"size": S}, "rot": {"base": 30.0, "dims": 4}}
    if kind == "attention":
        w, fn = _two_map_weights(H, G, D, V, W, 1), plain.two_map_window_attention
    else:
        m["vdim"] = D
        w, fn = _gated_weights(H, G, D, W, 1), plain.keys_as_values_attention
    x = _rand(2)(30, W)
    base = fn(x, w, "", m, 1e-6)
    moved = x.clone()
    moved[10] += 1.0
    changed = (fn(moved, w, "", m, 1e-6) - base).abs().amax(dim=1) > 1e-9
    assert changed.nonzero().flatten().tolist() == list(range(10, 10 + S))   # position 10 and the S - 1 after it
    # scores depend on differences of positions alone: the same tokens further along give the same
    shifted = fn(x, w, "", m, 1e-6, positions=[p + 11 for p in range(30)])
    torch.testing.assert_close(shifted, base)
    # the rotation matters
    assert float((fn(x, w, "", dict(m, rot={"base": 30.0, "dims": 8}), 1e-6) - base).abs().max()) > 1e-3


def test_plain_two_map_attention_against_dense_matrices():
    H, G, D, V, W, S = 4, 2, 8, 6, 16, 5
    w = _two_map_weights(H, G, D, V, W, 3)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.4, "diff": 0.25, "mask": {"size": S}, "rot": {"base": 100.0, "dims": 6}}
    T = 23
    x = _rand(4)(T, W)
    pos = list(range(T))

    def prepared(name, n):
        v = (x @ w[name].t() + w[name + ".b"]).view(T, n, 2, D)
        v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-6) * w[name + ".norm"]
        return _turn(v.reshape(T, n * 2, D), pos, 100.0, 6).view(T, n, 2, D)

    q, k = prepared("q", H), prepared("k", G).repeat_interleave(H // G, dim=1)
    v = (x @ w["v"].t() + w["v.b"]).view(T, G, V).repeat_interleave(H // G, dim=1)
    at = torch.arange(T)
    seen = (at[None, :] <= at[:, None]) & (at[:, None] - at[None, :] < S)
    probs = torch.softmax((torch.einsum("ihcd,jhcd->hcij", q, k) * 0.4).masked_fill(~seen, float("-inf")), dim=-1)
    lam = torch.exp(w["lq1"] @ w["lk1"]) - torch.exp(w["lq2"] @ w["lk2"]) + 0.25
    o = torch.einsum("hij,jhv->ihv", probs[:, 0] - lam * probs[:, 1], v)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * 0.75
    torch.testing.assert_close(plain.two_map_window_attention(x, w, "", m, 1e-6), o.reshape(T, -1) @ w["o"].t() + w["o.b"])


def test_plain_gated_attention_token_by_token():
    """Every output row made by itself from the keys it sees: the values are the raw key projections."""
    H, G, D, W, S = 4, 2, 6, 12, 4
    w = _gated_weights(H, G, D, W, 5)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": 0.5, "mask": {"size": S}, "rot": {"base": 20.0, "dims": 6}}
    T = 11
    x = _rand(6)(T, W)
    want = plain.keys_as_values_attention(x, w, "", m, 1e-6)
    raw = (x @ w["k"].t()).view(T, G, D)
    unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-6)
    keys = _turn(unit(raw) * w["k.norm"], list(range(T)), 20.0, 6)
    queries = _turn(unit((x @ w["q"].t()).view(T, H, D)) * w["q.norm"], list(range(T)), 20.0, 6)
    for i in range(T):
        lo = max(0, i - S + 1)
        heads = []
        for a in range(H):
            g = a // (H // G)
            p = torch.softmax(keys[lo : i + 1, g] @ queries[i, a] * 0.5, dim=0)
            heads.append(p @ raw[lo : i + 1, g])
        row = torch.cat(heads) * plain.logistic(w["g"] @ x[i])
        torch.testing.assert_close(w["o"] @ row, want[i])
    with pytest.raises(ValueError):
        plain.keys_as_values_attention(x, w, "", dict(m, vdim=D + 1), 1e-6)


def test_plain_feed_forwards():
    r = _rand(7)
    W, ff, E = 10, 6, 5
    w = {"router": r(E, W)}
    for e in range(E):
        w.update({f"e{e}.gate": r(ff, W) * 0.4, f"e{e}.up": r(ff, W) * 0.4, f"e{e}.down": r(W, ff) * 0.4})
    x = r(9, W)
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": 2}}
    got = plain.feed_forward(x, w, "", mlp)
    # the same as a dense sum over all experts with the unchosen ones' weights struck out; the score
    # goes INTO the expert (the expert is not linear: scaling its output instead differs)
    score = plain.logistic(x @ w["router"].t())
    keep = torch.zeros_like(score)
    keep.scatter_(1, score.topk(2, dim=-1).indices, 1.0)
    dense = sum(plain.expert((score[:, e] * keep[:, e])[:, None] * x, w, f"e{e}.") for e in range(E))
    torch.testing.assert_close(got, dense)
    outside = sum((score[:, e] * keep[:, e])[:, None] * plain.expert(x, w, f"e{e}.") for e in range(E))
    assert float((outside - got).abs().max()) > 1e-3
    # all experts chosen: nothing is struck out; the scores are not made to sum to one
    everything = plain.feed_forward(x, w, "", dict(mlp, router={"experts": E, "top": E}))
    torch.testing.assert_close(everything, sum(plain.expert(score[:, e : e + 1] * x, w, f"e{e}.") for e in range(E)))
    # among equal scores the lower index wins
    tie = dict(w, router=torch.zeros(E, W, dtype=torch.float64))
    chosen, s = plain.routed_choice(x, tie, "", 2)
    assert chosen.tolist() == [[0, 1]] * 9 and torch.all(s == 0.5)
    z = torch.tensor([-2.0, -0.0, 0.5, 3.0], dtype=torch.float64)
    torch.testing.assert_close(plain.relu_squared(z), torch.tensor([0.0, 0.0, 0.25, 9.0], dtype=torch.float64))
    torch.testing.assert_close(plain.silu(z), torch.nn.functional.silu(z))
    d = {"up": r(ff, W), "down": r(W, ff)}
    torch.testing.assert_close(plain.dense_feed_forward(x, d, ""), torch.relu(x @ d["up"].t()) ** 2 @ d["down"].t())


def test_plain_layer_norms_the_branch_not_the_input(tmp_path):
    folder = write_random_model(tmp_path / "a", NENODRA_A, 9)
    oracle = plain.PlainNenodra(folder)
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    streams = oracle.streams(tokens)
    w, cfg = oracle.w, oracle.cfg
    x0 = w["embed"][torch.tensor(tokens)]
    # layer 3 has no feed-forward: the stream moves by residual_mult times a vector whose root mean
    # square, before the weight, is one (a little less: eps stands beside a small mean square)
    step = (streams[3] - streams[2]) / cfg["residual_mult"] / (1.0 + w["l3.norm1"])
    mean_square = (step * step).mean(-1)
    assert bool(((mean_square > 0.9) & (mean_square <= 1.0)).all())
    # the first layer reads the embedding itself
    branch = plain.keys_as_values_attention(x0, w, "l0.mix.", cfg["layers"][0]["mixer"], cfg["norm"]["eps"])
    after = x0 + cfg["residual_mult"] * plain.output_norm(branch, w["l0.norm1"], cfg["norm"]["eps"])
    mlp = plain.feed_forward(after, w, "l0.mlp.", cfg["layers"][0]["mlp"])
    torch.testing.assert_close(streams[0], after + cfg["residual_mult"] * plain.output_norm(mlp, w["l0.norm2"], cfg["norm"]["eps"]))
    # the logits carry the constant factor
    oracle.cfg = dict(cfg, logit_scale=2 * cfg["logit_scale"])
    torch.testing.assert_close(oracle.logits(tokens), 2 * plain.PlainNenodra(folder).logits(tokens))
