"""The tiny configurations the tests run: they differ in every size and option.

A and B are the benchmark description's tiny models; C makes num_heads * head_dim
differ from hidden_size (an explicit head_dim key) and uses sizes that are no powers
of two, which neither A nor B pins.
"""

TINY_A = dict(
    model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=512, hidden_size=64,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, intermediate_size=176,
    rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True, hidden_act="silu",
    use_sliding_window=False, max_position_embeddings=256,
)
TINY_B = dict(
    model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=1000, hidden_size=192,
    num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, intermediate_size=384,
    rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False, hidden_act="silu",
    use_sliding_window=False, max_position_embeddings=512,
)
TINY_C = dict(
    model_type="qwen2", vocab_size=777, hidden_size=80, head_dim=48,
    num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=3, intermediate_size=100,
    rms_norm_eps=3e-6, rope_theta=50000.0, tie_word_embeddings=False,
)
# name -> (config, weight seed, cache block size)
TINY_CONFIGS = {"A": (TINY_A, 0, 16), "B": (TINY_B, 1, 8), "C": (TINY_C, 5, 16)}

# Sizes that none of the above pins: groups of 5, 7, 14, 17 and 66 query heads (17 and more: more than one
# workgroup of the decode kernel takes), widths that are multiples of 2 only or odd, a feed-forward of 7,
# pages of 4, 24 and 48 tokens, head sizes 32 to 256. name -> (config, weight seed, block size)
ODD_CONFIGS = {
    "group14": (dict(model_type="qwen2", vocab_size=1001, hidden_size=66, head_dim=96, num_hidden_layers=2,
                     num_attention_heads=42, num_key_value_heads=3, intermediate_size=255, rms_norm_eps=1e-5,
                     rope_theta=50000.0, tie_word_embeddings=False), 11, 16),
    "pages_of_4": (dict(model_type="qwen2", vocab_size=127, hidden_size=130, head_dim=256, num_hidden_layers=3,
                        num_attention_heads=15, num_key_value_heads=3, intermediate_size=33, rms_norm_eps=3e-4,
                        rope_theta=10000.0, tie_word_embeddings=False), 12, 4),
    "narrow": (dict(model_type="qwen2", vocab_size=51, hidden_size=66, head_dim=32, num_hidden_layers=2,
                    num_attention_heads=14, num_key_value_heads=2, intermediate_size=7, rms_norm_eps=1e-6,
                    rope_theta=1000000.0, tie_word_embeddings=True), 13, 24),
    "group17": (dict(model_type="qwen2", vocab_size=2049, hidden_size=1032, head_dim=160, num_hidden_layers=1,
                     num_attention_heads=34, num_key_value_heads=2, intermediate_size=1000, rms_norm_eps=1e-6,
                     rope_theta=1000000.0, tie_word_embeddings=True), 14, 48),
    # odd widths (rows that no 16-byte load fits) and a group of 66 query heads on one key head
    "odd_widths": (dict(model_type="qwen2", vocab_size=33, hidden_size=65, head_dim=16, num_hidden_layers=2,
                        num_attention_heads=3, num_key_value_heads=1, intermediate_size=9, rms_norm_eps=1e-6,
                        rope_theta=10000.0, tie_word_embeddings=False), 15, 8),
    "group66": (dict(model_type="qwen2", vocab_size=300, hidden_size=72, head_dim=32, num_hidden_layers=1,
                     num_attention_heads=66, num_key_value_heads=1, intermediate_size=50, rms_norm_eps=1e-6,
                     rope_theta=10000.0, tie_word_embeddings=False), 16, 16),
}

# Layers wide enough for the decode kernels that only take large shapes (the persistent
# weight-streaming product, the norm fused into the gate/up product): hidden >= 1024 and at least
# 512 row tiles of 8 in the feed-forward. Two layers and a small vocabulary keep it quick.
WIDE = dict(
    model_type="qwen2", vocab_size=1203, hidden_size=1024, num_hidden_layers=2, num_attention_heads=8,
    num_key_value_heads=2, intermediate_size=4360, rms_norm_eps=2e-6, rope_theta=300000.0,
    tie_word_embeddings=False,
)

# One layer each of the larger models the engine is meant for (Qwen2.5-7B and -32B layer sizes, a
# small vocabulary): products whose K does not fit the streaming kernel's registers, groups of 7
# and 5 query heads per key head, 18944 / 27648-wide feed-forwards.
# One layer of exactly the benchmark's model (Qwen2.5-1.5B): its widths, its full vocabulary, its
# tied output head.
LAYER_1P5B = dict(
    model_type="qwen2", vocab_size=151936, hidden_size=1536, num_hidden_layers=1, num_attention_heads=12,
    num_key_value_heads=2, intermediate_size=8960, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=True,
)
LAYER_7B = dict(
    model_type="qwen2", vocab_size=1501, hidden_size=3584, num_hidden_layers=1, num_attention_heads=28,
    num_key_value_heads=4, intermediate_size=18944, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)
LAYER_32B = dict(
    model_type="qwen2", vocab_size=1302, hidden_size=5120, num_hidden_layers=1, num_attention_heads=40,
    num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=False,
)


# ---- Fuvavik: small models that differ in every size and constant; layers of one model differ too.
def _fuvavik_layer(heads, kv_heads, dim, vdim, scale, window, r_heads, r_dim, r_vdim, tau, rank, ff):
    return {
        "type": "parallel",
        "mixer": {
            "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window}},
            "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau, "rank": rank},
        },
        "mlp": None if ff is None else {"kind": "dense", "ff": ff},
    }


# two layers that share nothing: grouped heads with key and value sizes apart and a window of 9
# beside a recurrence of rank 5; then one key/value head per query head, a window of 33, no
# feed-forward
FUVAVIK_A = {
    "architecture": "Fuvavik", "vocab": 300, "width": 96, "max_positions": 640,
    "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
    "layers": [
        _fuvavik_layer(4, 2, 24, 16, 0.2, 9, 2, 12, 20, 4.0, 5, 72),
        _fuvavik_layer(6, 6, 16, 16, 0.25, 33, 3, 20, 8, 16.0, 3, None),
    ],
}
# a width that is no multiple of 8, one key/value head for three query heads, a window longer than
# any request of the tests (every key is seen), a single recurrent head with tau = 1, a window of 1
FUVAVIK_B = {
    "architecture": "Fuvavik", "vocab": 127, "width": 100, "max_positions": 700,
    "embedding": {"scale": 0.5}, "norm": {"eps": 3e-4}, "logit_softcap": 7.5,
    "layers": [
        _fuvavik_layer(3, 1, 40, 24, 0.16, 300, 1, 64, 64, 1.0, 16, 50),
        _fuvavik_layer(2, 1, 8, 32, 0.35, 1, 4, 6, 10, 2.5, 2, 130),
        _fuvavik_layer(3, 1, 40, 24, 0.16, 300, 1, 64, 64, 1.0, 16, 50),
    ],
}
# one head everywhere and sizes of 1 where the design allows them
FUVAVIK_C = {
    "architecture": "Fuvavik", "vocab": 64, "width": 48, "max_positions": 200,
    "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
    "layers": [_fuvavik_layer(1, 1, 32, 8, 0.18, 17, 1, 16, 4, 8.0, 1, 24)],
}
# four layers of unlike sizes for long requests: windows of 77 to 1500, key and value sizes that the
# matrix-core attention kernel takes (layers 1 to 3) and one that it does not, states from 16 x 16 to
# 128 x 256
FUVAVIK_LONG = {
    "architecture": "Fuvavik", "vocab": 211, "width": 192, "max_positions": 1600,
    "embedding": {"scale": 1.7}, "norm": {"eps": 2e-6}, "logit_softcap": 11.0,
    "layers": [
        _fuvavik_layer(6, 3, 32, 48, 0.3, 200, 3, 40, 24, 8.0, 12, 384),
        _fuvavik_layer(4, 4, 64, 64, 0.2, 77, 2, 64, 128, 32.0, 8, None),
        _fuvavik_layer(8, 2, 128, 64, 0.15, 513, 6, 16, 16, 2.0, 4, 100),
        _fuvavik_layer(16, 2, 64, 128, 0.2, 1500, 1, 128, 256, 64.0, 16, 64),
    ],
}
# name -> (config, weight seed, cache block size)
FUVAVIK_CONFIGS = {"FA": (FUVAVIK_A, 21, 8), "FB": (FUVAVIK_B, 22, 16), "FC": (FUVAVIK_C, 23, 4)}


# ---- Pesorax: small models that differ in every size and constant; layers of one model differ too.
def _pesorax_attention(heads, kv_heads, dim, vdim, scale, diff, segment, ff):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
                      "mask": {"size": segment}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _pesorax_latent(heads, dim, rot_dim, rot_dims, vdim, q_rank, kv_rank, scale, base, ff):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale, "rot": {"base": base, "dims": rot_dims}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# four layers that share nothing; the middle two run twice; three query heads a key/value head,
# segments of 9 and 33, a rope part of which only half is rotated, a layer without a feed-forward
PESORAX_A = {
    "architecture": "Pesorax", "vocab": 300, "width": 96, "residual_mult": 0.5, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        _pesorax_attention(6, 2, 16, 24, 0.2, 0.3, 9, 72),
        _pesorax_latent(3, 24, 16, 8, 20, 40, 48, 0.15, 100.0, None),
        _pesorax_attention(2, 2, 8, 8, 0.3, 0.8, 33, 40),
        _pesorax_latent(2, 16, 8, 8, 32, 24, 16, 0.2, 10000.0, 64),
    ],
}
# a width that is no multiple of 8, no repeated layers (no "loop" key at all), one key/value head
# for three query heads, a segment longer than any request of the tests (every earlier key is
# seen) and one of 1 (a token sees itself alone), a residual multiplier of 1
PESORAX_B = {
    "architecture": "Pesorax", "vocab": 127, "width": 100, "residual_mult": 1.0, "norm": {"eps": 3e-4},
    "layers": [
        _pesorax_attention(3, 1, 40, 24, 0.16, 0.5, 300, 50),
        _pesorax_latent(5, 8, 4, 4, 12, 20, 36, 0.3, 50.0, 130),
        _pesorax_attention(2, 1, 8, 32, 0.35, 0.1, 1, None),
    ],
}
# one head everywhere, sizes of 1 and 2 where the design allows them, the whole model repeated
# three times
PESORAX_C = {
    "architecture": "Pesorax", "vocab": 64, "width": 48, "residual_mult": 0.25, "norm": {"eps": 1e-6},
    "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        _pesorax_latent(1, 2, 2, 2, 1, 4, 8, 0.5, 4.0, 24),
        _pesorax_attention(1, 1, 32, 8, 0.18, 0.6, 17, 24),
    ],
}
# layers of unlike sizes for long requests: segments of 77 to 1500, latents of 256 + 64 and 128 + 32
# elements, sizes that the matrix cores take (layers 1 to 4) and one that they do not
PESORAX_LONG = {
    "architecture": "Pesorax", "vocab": 211, "width": 192, "residual_mult": 0.4, "norm": {"eps": 2e-6},
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [
        _pesorax_attention(6, 3, 32, 48, 0.3, 0.4, 200, 384),
        _pesorax_latent(8, 64, 64, 32, 64, 96, 256, 0.2, 10000.0, None),
        _pesorax_attention(8, 2, 64, 128, 0.15, 0.7, 1500, 100),
        _pesorax_latent(16, 32, 32, 32, 32, 64, 128, 0.25, 500.0, 64),
        _pesorax_attention(4, 4, 64, 64, 0.2, 0.2, 77, None),
    ],
}
# name -> (config, weight seed, cache block size)
PESORAX_CONFIGS = {"PA": (PESORAX_A, 31, 8), "PB": (PESORAX_B, 32, 16), "PC": (PESORAX_C, 33, 4)}


# ---- Nenodra: small models that differ in every size and constant; layers of one model differ too.
def _nenodra_mlp(mlp):
    if mlp is None or isinstance(mlp, dict):
        return mlp
    if isinstance(mlp, int):
        return {"kind": "dense", "ff": mlp}
    ff, experts, top = mlp
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _nenodra_two_map(heads, kv_heads, dim, vdim, scale, diff, window, base, rot_dims, mlp):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
                      "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims}},
            "mlp": _nenodra_mlp(mlp)}


def _nenodra_gated(heads, kv_heads, dim, scale, window, base, rot_dims, mlp):
    return {"type": "attention_2",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                      "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims}},
            "mlp": _nenodra_mlp(mlp)}


# four layers that share nothing: three query heads a key/value head, windows of 9, 33, 5 and 17,
# rotations of a part of the vector and of all of it, two and three experts a token (all of three),
# a layer without a feed-forward; the three model-wide constants all differ
NENODRA_A = {
    "architecture": "Nenodra", "vocab": 300, "width": 96, "residual_mult": 0.7, "logit_scale": 1.3, "norm": {"eps": 1e-5},
    "layers": [
        _nenodra_gated(6, 2, 16, 0.2, 9, 100.0, 8, (40, 5, 2)),
        _nenodra_two_map(4, 2, 8, 24, 0.3, 0.3, 33, 1000.0, 8, 72),
        _nenodra_two_map(2, 2, 24, 8, 0.25, 0.8, 5, 50.0, 12, (24, 3, 3)),
        _nenodra_gated(3, 1, 40, 0.16, 17, 10000.0, 40, None),
    ],
}
# a width that is no multiple of 8, a window longer than any request of the tests (every earlier key
# is seen) and one of 1 (a token sees itself alone), no rotation at all in one layer, one expert of
# two, constants of 1
NENODRA_B = {
    "architecture": "Nenodra", "vocab": 127, "width": 100, "residual_mult": 1.0, "logit_scale": 1.0, "norm": {"eps": 3e-4},
    "layers": [
        _nenodra_two_map(3, 1, 40, 24, 0.16, 0.45, 300, 200000.0, 2, (50, 2, 1)),
        _nenodra_gated(5, 5, 12, 0.3, 1, 50.0, 12, 130),
        _nenodra_two_map(2, 1, 8, 32, 0.35, 0.1, 40, 10.0, 0, (36, 7, 4)),
    ],
}
# one head everywhere, sizes of 1 and 2 where the design allows them, a single expert
NENODRA_C = {
    "architecture": "Nenodra", "vocab": 64, "width": 48, "residual_mult": 0.25, "logit_scale": 0.1, "norm": {"eps": 1e-6},
    "layers": [
        _nenodra_gated(1, 1, 2, 0.5, 16, 4.0, 2, (1, 1, 1)),
        _nenodra_two_map(1, 1, 32, 1, 0.18, 0.6, 17, 500.0, 16, 24),
    ],
}
# layers of unlike sizes for long requests: windows of 77 to 1500, head sizes that the matrix cores
# take and ones that they do not, sixteen experts of which a token uses four
NENODRA_LONG = {
    "architecture": "Nenodra", "vocab": 211, "width": 192, "residual_mult": 0.4, "logit_scale": 0.8, "norm": {"eps": 2e-6},
    "layers": [
        _nenodra_two_map(6, 3, 32, 48, 0.3, 0.4, 200, 10000.0, 32, 384),
        _nenodra_gated(8, 2, 64, 0.2, 513, 10000.0, 32, (64, 16, 4)),
        _nenodra_two_map(8, 2, 64, 128, 0.15, 0.7, 1500, 500000.0, 64, 100),
        _nenodra_gated(4, 4, 128, 0.12, 77, 500.0, 128, None),
        _nenodra_gated(6, 2, 24, 0.25, 130, 1000.0, 20, (40, 3, 2)),
    ],
}
# name -> (config, weight seed, cache block size)
NENODRA_CONFIGS = {"NA": (NENODRA_A, 41, 8), "NB": (NENODRA_B, 42, 16), "NC": (NENODRA_C, 43, 4)}


def random_nenodra_config(seed: int) -> dict:
    """A model of the design drawn at random: three to seven layers that share nothing, head sizes
    that the matrix-core kernels take and ones they do not, windows shorter and longer than a
    page, rotation of all, a part and nothing, one to four experts a token, layers without a
    feed-forward."""
    import random

    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(3, 7)):
        kv = rng.choice([1, 2, 4])
        heads = kv * rng.choice([1, 2, 3, 4])
        dim = rng.choice([16, 24, 32, 40, 48, 64, 80, 96, 128])
        rot = rng.choice([dim, dim // 4 * 2, 16, 0, dim])
        scale = dim ** -0.5 * rng.choice([0.5, 1.0, 2.0])
        window = rng.choice([1, 33, 64, 65, 100, 130, 200, 257])
        base = rng.choice([100.0, 10000.0, 5e5])
        kind = rng.choice(["dense", "dense", "moe", "moe", "moe", None])
        if kind == "dense":
            mlp = rng.choice([72, 104, 200, 512])
        elif kind == "moe":
            experts = rng.choice([2, 4, 5, 8, 16])
            mlp = (rng.choice([40, 64, 88, 128, 256]), experts, rng.randint(1, min(4, experts)))
        else:
            mlp = None
        if rng.random() < 0.5:
            layers.append(_nenodra_two_map(heads, kv, dim, rng.choice([16, 32, 48, 64, 96, 128]), scale, rng.choice([0.2, 0.45, 0.8]),
                                           window, base, rot, mlp))
        else:
            layers.append(_nenodra_gated(heads, kv, dim, scale, window, base, rot, mlp))
    return {"architecture": "Nenodra", "vocab": rng.choice([300, 500, 1000]), "width": rng.choice([128, 192, 320, 384, 512]),
            "residual_mult": rng.choice([0.3, 0.6, 1.0]), "logit_scale": rng.choice([0.25, 0.7, 2.0]),
            "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}



# ------------------------------------------------------------------------------- Raranex
def _raranex_window(heads, kv_heads, dim, vdim, scale, window, keep_first, base, rot_dims):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "mask": {"size": window, "keep_first": keep_first}, "rot": {"base": base, "dims": rot_dims}}


def _raranex_pair(heads, kv_heads, dim, vdim, scale, softcap, coef, every, r_heads, r_dim, rank=None):
    right = {"heads": r_heads, "dim": r_dim}
    if rank is not None:
        right["rank"] = rank
    return {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
                     "q_temp": {"coef": coef, "every": every}}, "right": right}


def _raranex_moe(ff, experts, top, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


# three layers of which the first two run twice: grouped heads with keys and values of unlike sizes,
# a window of 9 that keeps 3 first tokens, a partial rotation, six experts in three runs of which two
# are kept, a layer without a feed-forward, a decay projection of rank 6
RARANEX_A = {
    "architecture": "Raranex", "vocab": 211, "width": 96, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        {"type": "parallel", "mixer": _raranex_pair(4, 2, 24, 16, 0.2, 8.0, 0.3, 7, 3, 16, rank=6),
         "mlp": _raranex_moe(40, 6, 2, groups=(3, 2), shared=48)},
        {"type": "attention", "mixer": _raranex_window(4, 4, 32, 24, 0.18, 9, 3, 100.0, 16), "mlp": None},
        {"type": "attention", "mixer": _raranex_window(6, 2, 16, 40, 0.25, 33, 1, 10000.0, 16),
         "mlp": _raranex_moe(24, 3, 3, shared=20)},
    ],
}
# a width that is no multiple of 8, heads of 20 and 12 elements, a recurrence of one head whose size
# is no multiple of 4, no loop, no expert runs, every expert chosen, no shared expert, a window of 1
# (a token sees itself and the kept first ones) and a layer that only sees itself (nothing kept)
RARANEX_B = {
    "architecture": "Raranex", "vocab": 127, "width": 100, "norm": {"eps": 3e-4},
    "layers": [
        {"type": "attention", "mixer": _raranex_window(5, 5, 20, 12, 0.22, 1, 2, 50.0, 10), "mlp": _raranex_moe(36, 4, 4)},
        {"type": "parallel", "mixer": _raranex_pair(3, 1, 40, 24, 0.16, 2.0, 1.5, 1, 1, 18), "mlp": _raranex_moe(50, 2, 1, shared=8)},
        {"type": "attention", "mixer": _raranex_window(2, 1, 8, 32, 0.35, 1, 0, 10.0, 0), "mlp": None},
    ],
}
# the whole model three times over, a window longer than any request of the tests, more first tokens
# kept than the window holds, runs of one expert each, one expert a token, sizes of 1 and 2
RARANEX_C = {
    "architecture": "Raranex", "vocab": 64, "width": 48, "norm": {"eps": 1e-6},
    "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        {"type": "attention", "mixer": _raranex_window(1, 1, 2, 1, 0.5, 300, 0, 4.0, 2), "mlp": _raranex_moe(1, 4, 1, groups=(4, 2), shared=1)},
        {"type": "parallel", "mixer": _raranex_pair(1, 1, 32, 1, 0.18, 50.0, 0.0, 64, 2, 4, rank=1),
         "mlp": _raranex_moe(16, 8, 3, groups=(2, 1), shared=24)},
    ],
}
RARANEX_D = {
    "architecture": "Raranex", "vocab": 90, "width": 64, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 2, "times": 2},
    "layers": [
        {"type": "attention", "mixer": _raranex_window(2, 2, 16, 16, 0.3, 4, 6, 1000.0, 16), "mlp": _raranex_moe(24, 4, 2, groups=(2, 1), shared=16)},
        {"type": "parallel", "mixer": _raranex_pair(2, 2, 16, 8, 0.25, 5.0, 0.5, 3, 2, 8), "mlp": None},
    ],
}
# name -> (config, weight seed, cache block size)
RARANEX_CONFIGS = {"RA": (RARANEX_A, 51, 8), "RB": (RARANEX_B, 52, 16), "RC": (RARANEX_C, 53, 4), "RD": (RARANEX_D, 54, 8)}


def random_raranex_config(seed: int) -> dict:
    """A model of the design drawn at random: two to six layers that share nothing, a repeated run
    anywhere among them (or none), head sizes that the matrix-core kernels take and ones they do
    not, windows shorter and longer than a page with none to many first tokens kept, rotation of
    all, a part and nothing, expert runs or none, a shared expert or none."""
    import random

    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(2, 6)):
        kv = rng.choice([1, 2, 4])
        heads = kv * rng.choice([1, 2, 3, 4])
        dim = rng.choice([16, 24, 32, 40, 48, 64, 80, 96, 128])
        vdim = rng.choice([16, 24, 32, 48, 64, 96, 128])
        scale = dim ** -0.5 * rng.choice([0.5, 1.0, 2.0])
        experts = rng.choice([2, 4, 6, 8, 16])
        top = rng.randint(1, min(4, experts))
        groups = None
        if rng.random() < 0.6:
            count = rng.choice([c for c in (1, 2, 4, 8) if experts % c == 0])
            keep = rng.randint(1, count)
            if (experts // count) * keep >= top:
                groups = (count, keep)
        mlp = None if rng.random() < 0.15 else _raranex_moe(rng.choice([40, 64, 88, 128]), experts, top, groups,
                                                               rng.choice([None, 32, 72, 128]))
        if rng.random() < 0.5:
            rot = rng.choice([dim, dim // 4 * 2, 16, 0, dim])
            mixer = _raranex_window(heads, kv, dim, vdim, scale, rng.choice([1, 33, 64, 65, 100, 130, 200, 257]),
                                    rng.choice([0, 1, 5, 64, 70, 150]), rng.choice([100.0, 10000.0, 5e5]), rot)
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        else:
            mixer = _raranex_pair(heads, kv, dim, vdim, scale, rng.choice([3.0, 20.0, 50.0]), rng.choice([0.0, 0.25, 1.0]),
                                  rng.choice([1, 16, 64, 100]), rng.choice([1, 2, 4, 6]), rng.choice([8, 16, 20, 32, 64]),
                                  rank=rng.choice([None, 4, 12, 32]))
            layers.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Raranex", "vocab": rng.choice([300, 500, 1000]), "width": rng.choice([128, 192, 320, 384]),
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        start = rng.randint(0, len(layers) - 1)
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return cfg

