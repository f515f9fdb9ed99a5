"""Raranex without a GPU: the configuration reader and what it refuses, the order of layer runs and
where the stream is re-entered, the weight plan against the tensors a checkpoint of the design
holds, the decay rank from a checkpoint's shapes, cache groups (pages given back behind a window
but for the kept first ones, a state slot a pass), and the plain implementation against second
ways of writing it (rotation as complex numbers, the masks by hand, the recurrence in closed form,
the router by brute force)."""

import copy
import itertools
import math

import pytest
import torch

from clockwork_amd.cache.manager import NO_PAGE, CacheManager, cache_needs_of, plan_groups
from clockwork_amd.parts.model import DecoderModel, model_param_specs
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import check_plan
from clockwork_amd.weights.random_init import write_random_model
from tests.configs import RARANEX_A, RARANEX_B, RARANEX_C, RARANEX_D, random_raranex_config
from tests.plain import raranex_plain as plain


def _describe(config):
    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    spec = arch.build_spec(cfg)
    return arch, cfg, spec, arch.weight_plan(cfg, spec)


def test_the_design_is_found_and_every_constant_is_read():
    arch, cfg, spec, _ = _describe(RARANEX_A)
    assert arch.name == "Raranex" and spec.architecture == "Raranex"
    assert (cfg.vocab, cfg.width, cfg.eps) == (211, 96, 1e-5)
    assert (spec.final_norm.size, spec.final_norm.eps) == (96, 1e-5) and not spec.tie_embeddings
    assert all(l.arrangement == "twonorm" for l in spec.layers)
    a, b, c = spec.layers
    pair = a.mixer
    assert type(pair).__name__ == "PairMixerSpec" and pair.eps == 1e-5
    l, r = pair.left, pair.right
    assert (l.num_heads, l.num_kv_heads, l.key_dim, l.value_dim, l.scale, l.softcap, l.query_temperature) == (4, 2, 24, 16, 0.2, 8.0, (0.3, 7))
    assert (l.window, l.keep_first, l.position, l.qk_norm, l.qk_norm_weight, l.qk_norm_after_rotation) == (None, 0, None, True, True, False)
    assert l.output_gate and l.gate_per_head and l.values == "projection" and l.norm_eps == 1e-5
    assert (r.num_heads, r.head_dim, r.decay_rank, r.norm_eps) == (3, 16, 6, 1e-5)
    f = a.feed_forward
    assert (f.intermediate_size, f.num_experts, f.top_k, f.router, f.renormalize, f.weight_on) == (40, 6, 2, "sigmoid", True, "output")
    assert (f.choice_correction, f.groups, f.renorm_eps, f.shared_intermediate, f.shared_gate) == (True, (3, 2, 2), 1e-20, 48, True)
    m = b.mixer
    assert type(m).__name__ == "GatedAttentionSpec"
    assert (m.num_heads, m.num_kv_heads, m.key_dim, m.value_dim, m.scale, m.window, m.keep_first) == (4, 4, 32, 24, 0.18, 9, 3)
    assert (type(m.position).__name__, m.position.rotary_dim, m.position.theta) == ("RopePairsSpec", 16, 100.0)
    assert (m.qk_norm, m.qk_norm_weight, m.qk_norm_after_rotation, m.softcap, m.query_temperature) == (True, False, True, None, None)
    assert b.feed_forward is None and b.ffn_norm is None
    assert c.feed_forward.groups is None and c.feed_forward.top_k == 3 and c.feed_forward.shared_intermediate == 20
    # no shared expert: no gate row; no rotated elements: no position encoding; no rank named: the default
    _, _, spec_b, _ = _describe(RARANEX_B)
    assert spec_b.layers[0].feed_forward.shared_intermediate is None and not spec_b.layers[0].feed_forward.shared_gate
    assert spec_b.layers[2].mixer.position is None and spec_b.layers[1].mixer.right.decay_rank == 16


def test_the_order_of_layer_runs_and_where_the_stream_is_re_entered():
    run = lambda config: [(e.layer, e.reenter) for e in _describe(config)[2].run]  # noqa: E731
    assert run(RARANEX_A) == [(0, 0), (1, None), (0, 1), (1, None), (2, None)]
    assert run(RARANEX_C) == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    assert run(RARANEX_D) == [(0, None), (1, 0), (1, 1)]
    spec_a, spec_b = _describe(RARANEX_A)[2], _describe(RARANEX_B)[2]
    assert (spec_a.reentry.hidden_size, spec_a.reentry.passes) == (96, 2)
    assert run(RARANEX_B) == [(0, None), (1, None), (2, None)] and spec_b.reentry is None
    # an empty run repeats nothing and re-enters nothing
    empty = copy.deepcopy(RARANEX_A)
    empty["loop"] = {"start": 1, "stop": 1, "times": 4}
    assert run(empty) == [(0, None), (1, None), (2, None)] and _describe(empty)[2].reentry is None
    # the plain implementation runs in the same order
    for config in (RARANEX_A, RARANEX_B, RARANEX_C, RARANEX_D, empty):
        assert plain.run_order(len(config["layers"]), config.get("loop")) == run(config)


@pytest.mark.parametrize("path, value, error", [
    (("layers", 0, "type"), "recurrent", NotImplementedError),
    (("layers", 0, "mlp", "kind"), "dense", NotImplementedError),
    (("layers", 1, "mixer", "kv_heads"), 3, ValueError),
    (("layers", 1, "mixer", "mask"), None, ValueError),
    (("layers", 1, "mixer", "rot"), None, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 7, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 34, ValueError),
    (("layers", 0, "mixer", "left"), None, ValueError),
    (("layers", 0, "mixer", "right"), None, ValueError),
    (("layers", 0, "mixer", "left", "scale"), None, ValueError),
    (("layers", 0, "mixer", "left", "q_temp", "every"), 0, ValueError),
    (("layers", 0, "mixer", "right", "dim"), 0, ValueError),
    (("layers", 0, "mlp", "router", "top"), 7, ValueError),
    (("layers", 0, "mlp", "router", "top"), 0, ValueError),
    (("layers", 0, "mlp", "router", "groups", "count"), 4, ValueError),     # six experts do not lie in four equal runs
    (("layers", 0, "mlp", "router", "groups", "keep"), 4, ValueError),
    (("layers", 0, "mlp", "expert"), None, ValueError),
    (("loop", "stop"), 4, ValueError),
    (("loop", "times"), 0, ValueError),
    (("norm",), None, ValueError),
    (("layers",), [], ValueError),
    (("width",), 0, ValueError),
])
def test_what_the_configuration_reader_refuses(path, value, error):
    config = copy.deepcopy(RARANEX_A)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(error):
        _describe(config)
    # a run too small for the experts a token takes
    config = copy.deepcopy(RARANEX_A)
    config["layers"][0]["mlp"]["router"].update(top=3, groups={"count": 3, "keep": 1})
    with pytest.raises(ValueError):
        _describe(config)


def _tensor_names(config, rank=16):
    """Names and shapes of a checkpoint of the design, written out from the layer list."""
    W = config["width"]
    names = {"embed": (config["vocab"], W), "head": (config["vocab"], W), "final.norm": (W,)}
    loop = config.get("loop")
    if loop and loop["stop"] > loop["start"]:
        names.update({"loop.in": (W, 2 * W), "loop.step": (loop["times"], W)})

    def attention(p, m, weighted):
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        names.update({p + "q": (H * D, W), p + "k": (G * D, W), p + "v": (G * V, W), p + "g": (H, W), p + "o": (W, H * V)})
        if weighted:
            names.update({p + "q.norm": (D,), p + "k.norm": (D,)})

    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        names[p + "norm1"] = (W,)
        if layer["type"] == "attention":
            attention(p + "mix.", m, False)
        else:
            attention(p + "mix.left.", m["left"], True)
            r, q = m["right"], p + "mix.right."
            inner, rk = r["heads"] * r["dim"], r.get("rank", rank)
            names.update({q + "mu." + s: (W,) for s in ("r", "k", "v", "g", "w")})
            names.update({q + s: (inner, W) for s in ("r", "k", "v", "g")})
            names.update({q + "w1": (rk, W), q + "w2": (inner, rk), q + "w0": (inner,), q + "u": (r["heads"], r["dim"]),
                          q + "norm": (inner,), q + "o": (W, inner), p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
        mlp = layer["mlp"]
        if mlp is None:
            continue
        ff, E = mlp["expert"]["ff"], mlp["router"]["experts"]
        names.update({p + "norm2": (W,), p + "mlp.router": (E, W), p + "mlp.correction": (E,)})
        for e in range(E):
            names.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
        if mlp.get("shared") is not None:
            s = mlp["shared"]["ff"]
            names.update({p + "mlp.shared.gate": (s, W), p + "mlp.shared.up": (s, W), p + "mlp.shared.down": (W, s), p + "mlp.shared.sg": (1, W)})
    return names


@pytest.mark.parametrize("config", [RARANEX_A, RARANEX_B, RARANEX_C, RARANEX_D] + [random_raranex_config(s) for s in range(5)])
def test_the_weight_plan_names_every_tensor_of_the_design(config):
    _, _, spec, plan = _describe(config)
    names = _tensor_names(config)
    assert check_plan(names, plan) == ([], [], [])
    specs = model_param_specs(spec)
    assert {t.param for t in plan} == set(specs)
    gone = next(n for n in names if n.endswith("mix.g") or n.endswith("left.g"))
    missing, unexpected, _ = check_plan({k: v for k, v in names.items() if k != gone} | {"l0.mix.extra": (3,)}, plan)
    assert missing == [gone] and unexpected == ["l0.mix.extra"]
    # stacked parameters have one row for every row of their sources
    for target in plan:
        assert specs[target.param].shape[0] == sum(shape[0] for shape in target.source_shapes)


def test_what_is_stacked_and_the_decay_rank_from_the_checkpoint():
    arch, _, _, plan = _describe(RARANEX_A)
    by_param = {t.param: t for t in plan}
    assert by_param["layers.0.mixer.left.in_weight"].sources == ("l0.mix.left.q", "l0.mix.left.k", "l0.mix.left.v", "l0.mix.left.g")
    assert by_param["layers.1.mixer.in_weight"].sources == ("l1.mix.q", "l1.mix.k", "l1.mix.v", "l1.mix.g")
    assert by_param["layers.0.mixer.right.mix"].sources == tuple(f"l0.mix.right.mu.{s}" for s in "rkvgw")
    assert by_param["layers.0.mixer.right.rkvg_weight"].sources == tuple(f"l0.mix.right.{s}" for s in "rkvg")
    assert by_param["layers.0.feed_forward.router_weight"].sources == ("l0.mlp.router", "l0.mlp.shared.sg")
    assert by_param["layers.0.feed_forward.gate_up_weight"].sources[:4] == ("l0.mlp.e0.gate", "l0.mlp.e0.up", "l0.mlp.e1.gate", "l0.mlp.e1.up")
    assert by_param["reentry.in_weight"].sources == ("loop.in",) and by_param["reentry.step"].sources == ("loop.step",)
    # the rank is the decay projection's first dimension where the configuration does not name it
    config = copy.deepcopy(RARANEX_B)
    filled = arch.sizes_from_checkpoint(config, {"l1.mix.right.w1": (5, 100)})
    assert filled["layers"][1]["mixer"]["right"]["rank"] == 5 and "rank" not in config["layers"][1]["mixer"]["right"]
    assert _describe(filled)[2].layers[1].mixer.right.decay_rank == 5
    named = arch.sizes_from_checkpoint(RARANEX_A, {"l0.mix.right.w1": (9, 96)})
    assert named["layers"][0]["mixer"]["right"]["rank"] == 6


def test_random_models_hold_what_the_plain_reader_needs(tmp_path):
    for name, config in (("a", RARANEX_A), ("b", RARANEX_B), ("c", RARANEX_C), ("d", RARANEX_D)):
        folder = write_random_model(tmp_path / name, config, 5)
        oracle = plain.PlainRaranex(folder)
        assert set(oracle.w) == set(_tensor_names(config))
        logits = oracle.logits([1, 2, 3, 4, 5])
        assert logits.shape == (5, config["vocab"]) and torch.isfinite(logits).all()
        assert oracle.streams([1, 2, 3]).shape == (len(plain.run_order(len(config["layers"]), config.get("loop"))), 3, config["width"])


def test_cache_groups_kept_first_pages_and_a_state_a_pass():
    model = DecoderModel(_describe(RARANEX_A)[2])
    groups = plan_groups(cache_needs_of(model.spec, model.mixers()))
    kv = [g for g in groups if g.is_kv]
    state = [g for g in groups if not g.is_kv]
    # the capped attention keeps everything; the window layers give pages back but for the kept ones;
    # every pass of the repeated layers owns a cache of its own
    assert [(g.window, g.keep_first, g.entries) for g in kv] == [(None, 0, ((0, 0), (2, 0))), (9, 3, (1, 3)), (33, 1, (4,))]
    assert [g.entries for g in state] == [((0, 1), (2, 1))] and state[0].need.shape == (3 * 16 * 16 + 96,)
    manager = CacheManager(groups, block_size=4, num_blocks=40, max_num_seqs=4)
    assert not manager.supports_prefix_sharing
    manager.admit("s", 70, portion_end=30)
    manager.extend("s", 0, 30)
    manager.release_behind_window("s", 30)
    rec = manager.record("s")
    # the next token, position 30, sees 22.. and 0..2 in group 1: page 0 stays, pages 1..4 go
    assert rec.tables[1][0] != NO_PAGE and all(p == NO_PAGE for p in rec.tables[1][1 : 22 // 4]) and rec.tables[1][22 // 4] != NO_PAGE
    assert all(p != NO_PAGE for p in rec.tables[0]) and all(p != NO_PAGE for p in rec.tables[2][:8])
    manager.extend("s", 30, 70)
    manager.release_behind_window("s", 70)
    assert rec.tables[1][0] != NO_PAGE and rec.tables[2][0] != NO_PAGE and rec.tables[2][1] == NO_PAGE
    manager.free("s")
    assert all(p.num_free == 40 for p in manager.pools)
    # more kept tokens than a page holds: every page they touch stays
    from clockwork_amd.config.spec import PagedRowsSpec

    need = PagedRowsSpec((("k", (1, 8)), ("v", (1, 8))), window=2, keep_first=9)
    m2 = CacheManager(plan_groups([need]), block_size=4, num_blocks=20, max_num_seqs=2)
    m2.admit("t", 40, portion_end=40)
    m2.extend("t", 0, 40)
    m2.release_behind_window("t", 40)
    table = m2.record("t").tables[0]
    assert all(p != NO_PAGE for p in table[:3]) and all(p == NO_PAGE for p in table[3:9]) and table[9] != NO_PAGE
    with pytest.raises(ValueError):
        PagedRowsSpec((("k", (1, 8)),), keep_first=3)


# ------------------------------------------------------------------------------- the plain implementation
def _rand(seed):
    gen = torch.Generator().manual_seed(seed)
    return lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)


def test_plain_rotation_against_complex_numbers_and_what_stays():
    v = _rand(1)(6, 3, 10)
    pos = [0, 1, 5, 17, 100, 1000]
    got = plain.rotate_neighbours(v, pos, 50.0, 6)
    for t, p in enumerate(pos):
        for i in range(3):
            z = torch.complex(v[t, :, 2 * i], v[t, :, 2 * i + 1]) * complex(math.cos(p * 50.0 ** (-2 * i / 6)), math.sin(p * 50.0 ** (-2 * i / 6)))
            torch.testing.assert_close(got[t, :, 2 * i], z.real)
            torch.testing.assert_close(got[t, :, 2 * i + 1], z.imag)
    assert torch.equal(got[..., 6:], v[..., 6:]) and torch.equal(got[0], v[0])
    # a rotation keeps the vector's length: the norm after it equals the norm before it
    torch.testing.assert_close(plain.unit_rms(got, 0.0), plain.rotate_neighbours(plain.unit_rms(v, 0.0), pos, 50.0, 6))
    assert torch.equal(plain.rotate_neighbours(v, pos, 50.0, 0), v)


def test_plain_masks_by_hand():
    seen = plain.seen_mask(list(range(12)), size=3, keep_first=2)
    for i in range(12):
        for j in range(12):
            assert bool(seen[i, j]) == (j <= i and (i - j < 3 or j < 2)), (i, j)
    causal = plain.seen_mask(list(range(5)))
    assert torch.equal(causal, torch.tril(torch.ones(5, 5, dtype=torch.bool)))
    # with positions that do not start at 0 the kept tokens are those of the sequence's start
    later = plain.seen_mask([10, 11, 12], size=2, keep_first=11)
    assert later.tolist() == [[True, False, False], [True, True, False], [True, True, True]]


def test_plain_window_attention_sees_exactly_its_window_and_the_kept_tokens():
    r = _rand(2)
    W, H, G, D, V, T = 24, 2, 1, 8, 6, 20
    w = {"q": r(H * D, W) * 0.3, "k": r(G * D, W) * 0.3, "v": r(G * V, W) * 0.3, "g": r(H, W) * 0.3, "o": r(W, H * V) * 0.2}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.4, "mask": {"size": 4, "keep_first": 2}, "rot": {"base": 30.0, "dims": 4}}
    x = r(T, W)
    base = plain.window_attention(x, w, "", m, 1e-6)
    for moved in (0, 1, 2, 7):
        y = x.clone()
        y[moved] += r(W)
        changed = (plain.window_attention(y, w, "", m, 1e-6) - base).abs().max(-1).values > 1e-9
        want = [i >= moved and (i - moved < 4 or moved < 2) for i in range(T)]
        assert changed.tolist() == want, moved
    # the gate is one number a head: closed on head 0, its columns of the output projection see nothing
    shut = torch.cat([torch.full((1, W), -1e4, dtype=torch.float64) * x[:1].sign(), w["g"][1:]])
    gated = plain.window_attention(x[:1], dict(w, g=shut), "", m, 1e-6)
    no_head = plain.window_attention(x[:1], dict(w, g=shut, o=torch.cat([torch.zeros(W, V, dtype=torch.float64), w["o"][:, V:]], 1)), "", m, 1e-6)
    torch.testing.assert_close(gated, no_head)


def test_plain_capped_attention_written_another_way():
    r = _rand(3)
    W, H, G, D, V, T = 20, 4, 2, 6, 5, 15
    w = {"q": r(H * D, W) * 0.5, "k": r(G * D, W) * 0.5, "v": r(G * V, W) * 0.3, "g": r(H, W) * 0.3, "o": r(W, H * V) * 0.2,
         "q.norm": 1 + r(D) * 0.2, "k.norm": 1 + r(D) * 0.2}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.9, "softcap": 1.5, "q_temp": {"coef": 0.7, "every": 4}}
    x = r(T, W)
    got = plain.capped_attention(x, w, "", m, 1e-6)
    out = torch.zeros(T, H * V, dtype=torch.float64)
    for i in range(T):
        factor = 1 + 0.7 * math.log((i + 1) // 4 + 1)
        for a in range(H):
            q = w["q"][a * D : (a + 1) * D] @ x[i]
            q = q / math.sqrt(float((q * q).mean()) + 1e-6) * w["q.norm"] * factor
            scores = []
            for j in range(i + 1):
                k = w["k"][(a // 2) * D : (a // 2 + 1) * D] @ x[j]
                k = k / math.sqrt(float((k * k).mean()) + 1e-6) * w["k.norm"]
                scores.append(1.5 * math.tanh(float(q @ k) * 0.9 / 1.5))
            p = torch.softmax(torch.tensor(scores, dtype=torch.float64), 0)
            vals = torch.stack([w["v"][(a // 2) * V : (a // 2 + 1) * V] @ x[j] for j in range(i + 1)])
            gate = 1 / (1 + math.exp(-float(w["g"][a] @ x[i])))
            out[i, a * V : (a + 1) * V] = (p[:, None] * vals).sum(0) * gate
    torch.testing.assert_close(got, out @ w["o"].t())
    assert plain.query_temperature([0, 2, 3, 7, 63], 0.5, 4, torch.float64).tolist() == \
        [1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3), 1 + 0.5 * math.log(17)]


def test_plain_recurrence_in_closed_form_and_the_shift():
    r = _rand(4)
    T, D = 9, 5
    q, k, v, u = r(T, D), r(T, D), r(T, D), r(D)
    decay = torch.rand(T, D, dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    got = plain.matrix_recurrence(q, k, v, decay, u)
    for t in range(T):
        # o_t = sum over s < t of (r_t . (prod of decays s+1 .. t-1) k_s) v_s  +  (r_t . u k_t) v_t
        o = (q[t] * u * k[t]).sum() * v[t]
        for s in range(t):
            between = torch.ones(D, dtype=torch.float64)
            for j in range(s + 1, t):
                between = between * decay[j]
            o = o + (q[t] * between * k[s]).sum() * v[s]
        torch.testing.assert_close(got[t], o)
    h = r(4, 3)
    mixes = plain.shifted_mixes(h, {"a": torch.zeros(3, dtype=torch.float64), "b": torch.ones(3, dtype=torch.float64)})
    assert torch.equal(mixes["a"], h)                                                 # mu 0: the token itself
    torch.testing.assert_close(mixes["b"], torch.cat([torch.zeros(1, 3, dtype=torch.float64), h[:-1]]))  # mu 1: the one before, zeros first


def test_plain_router_by_brute_force():
    r = _rand(6)
    W, E, T = 10, 8, 50
    w = {"router": r(E, W), "correction": r(E) * 0.8 - 0.5}
    x = r(T, W)
    router = {"experts": E, "top": 3, "groups": {"count": 4, "keep": 2}}
    chosen, weight = plain.routed_choice(x, w, "", router)
    s = 1 / (1 + torch.exp(-(x @ w["router"].t())))
    c = s + w["correction"]
    for t in range(T):
        runs = [c[t, 2 * g : 2 * g + 2].sum() for g in range(4)]   # a run of two: the sum of both
        kept = sorted(range(4), key=lambda g: -float(runs[g]))[:2]
        allowed = [e for e in range(E) if e // 2 in kept]
        best = max(itertools.combinations(allowed, 3), key=lambda combo: sum(float(c[t, e]) for e in combo))
        assert sorted(chosen[t].tolist()) == sorted(best)
        picked = s[t, chosen[t]]
        torch.testing.assert_close(weight[t], picked / (picked.sum() + 1e-20))
        assert float(c[t, chosen[t][0]]) >= float(c[t, chosen[t][1]]) >= float(c[t, chosen[t][2]])
    # negative choice scores: a run that is not kept counts as minus infinity, not as nothing
    w2 = {"router": torch.zeros(4, W, dtype=torch.float64), "correction": torch.tensor([-3.0, -2.0, -0.9, -0.8], dtype=torch.float64)}
    chosen, _ = plain.routed_choice(x[:1], w2, "", {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}})
    assert chosen.tolist() == [[3, 2]]
    chosen, _ = plain.routed_choice(x[:1], w2, "", {"experts": 4, "top": 2})
    assert chosen.tolist() == [[3, 2]]
    # the shared expert joins every token, times its gate
    ws = {"router": r(2, W), "correction": torch.zeros(2, dtype=torch.float64), "shared.sg": r(1, W)}
    for e in ("e0.", "e1.", "shared."):
        ws.update({e + "gate": r(6, W) * 0.3, e + "up": r(6, W) * 0.3, e + "down": r(W, 6) * 0.3})
    mlp = {"kind": "moe", "router": {"experts": 2, "top": 1}, "shared": {"ff": 6}}
    both = plain.routed_feed_forward(x, ws, "", mlp)
    alone = plain.routed_feed_forward(x, ws, "", dict(mlp, shared=None))
    gate = 1 / (1 + torch.exp(-(x @ ws["shared.sg"].t())))
    torch.testing.assert_close(both - alone, plain.gated_expert(x, ws, "shared.") * gate)


def test_plain_layer_reads_one_stream_through_two_norms(tmp_path):
    folder = write_random_model(tmp_path / "d", RARANEX_D, 7)
    oracle = plain.PlainRaranex(folder)
    w, cfg = oracle.w, oracle.cfg
    x = _rand(8)(6, cfg["width"])
    got = plain.layer(x, w, 0, cfg["layers"][0], 1e-5)
    mixed = plain.window_attention(plain.weighted_norm(x, w["l0.norm1"], 1e-5), w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    fed = plain.routed_feed_forward(plain.weighted_norm(x, w["l0.norm2"], 1e-5), w, "l0.mlp.", cfg["layers"][0]["mlp"])
    torch.testing.assert_close(got, x + mixed + fed)
    # the repeated layer runs twice with the same weights, each pass behind a re-entry of its own
    tokens = [3, 1, 4, 1, 5]
    streams = oracle.streams(tokens)
    e = w["embed"][torch.tensor(tokens)]
    first = plain.layer(e, w, 0, cfg["layers"][0], 1e-5)
    torch.testing.assert_close(streams[0], first)
    again = torch.cat([first, e], -1) @ w["loop.in"].t() + w["loop.step"][0]
    torch.testing.assert_close(streams[1], plain.layer(again, w, 1, cfg["layers"][1], 1e-5))
    third = torch.cat([streams[1], e], -1) @ w["loop.in"].t() + w["loop.step"][1]
    torch.testing.assert_close(streams[2], plain.layer(third, w, 1, cfg["layers"][1], 1e-5))
