"""Raranex: config.json keys -> typed config -> parts -> weight names.

A decoder whose layers run mixer and feed-forward side by side, each behind an RMS norm of its own
of the same stream: x <- x + M(N1(x)) + F(N2(x)). A run of layers is repeated with the same
weights and a cache per pass; right before every pass (the first too) the stream is re-entered from
itself and the embedding output e, x <- R [x; e] + s_n.

A layer's mixer is one of two kinds. "attention": grouped softmax attention whose queries and keys
are rotated over neighbouring element pairs and then divided by their root mean square (no
weights), behind a sliding window that keeps the request's first tokens visible, with a logistic
gate a head. "parallel": two mixers on the same input, their outputs RMS-normed over the width and
averaged: grouped attention with weighted per-head query/key norms, no rotation, a query factor
that grows with the logarithm of the position, tanh-capped scores, all earlier tokens visible and
the same gate a head; beside a recurrence over a matrix state a head whose inputs are mixes of a
token with the one before it. The feed-forward is routed: a logistic router whose choice (not its
weights) takes a learned correction and is confined to the best runs of neighbouring experts,
weights renormalised over the chosen, and a gated shared expert. The output is the model's RMS
norm and an untied head.

Every size and every constant that can differ between models of the design is read from
config.json: ``vocab``, ``width``, ``norm.eps``, ``loop`` (``start``, ``stop``, ``times``; absent:
every layer once, no re-entry) and, per entry of ``layers``, ``type``, ``mixer`` ("attention":
``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size``, ``mask.keep_first``,
``rot.base``, ``rot.dims``; "parallel": ``left`` with ``heads``, ``kv_heads``, ``dim``, ``vdim``,
``scale``, ``softcap``, ``q_temp.coef``, ``q_temp.every`` and ``right`` with ``heads``, ``dim``) and
``mlp`` (``kind`` "moe": ``expert.ff``, ``router.experts``, ``router.top``, ``router.groups.count``,
``router.groups.keep``, ``shared.ff``; null: no feed-forward). The rank of the recurrence's decay
projection is the first dimension of its checkpoint tensor (``mixer.right.rank`` may name it).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry, WeightTarget
from clockwork_amd.parts.specs import (GatedAttentionSpec, LinearHeadSpec, PairMixerSpec, RMSNormSpec, RopePairsSpec,
                                       RoutedExpertsSpec, ShiftedRecurrenceSpec, StreamReentrySpec, TokenEmbeddingSpec)
from clockwork_amd.registry import Architecture, register_architecture

NAME = "Raranex"
MIXER_KINDS = ("attention", "parallel")
DEFAULT_DECAY_RANK = 16
# a run of experts is scored by the sum of this many of its largest choice scores; the sum that the
# chosen weights are divided by carries this term
GROUP_SCORE_TOP = 2
RENORM_EPS = 1e-20
SHIFT_MIXES = ("r", "k", "v", "g", "w")


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ValueError(f"config.json lacks {where}{key}")
    return d[key]


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None       # None: every earlier token
    keep_first: int = 0
    rot_base: float = 10000.0
    rot_dims: int = 0
    softcap: Optional[float] = None
    q_temp: Optional[tuple] = None     # (coef, every)


@dataclass(frozen=True)
class RecurrenceConfig:
    heads: int
    dim: int
    rank: Optional[int]  # None: as the checkpoint's tensor has it


@dataclass(frozen=True)
class RoutedConfig:
    ff: int
    experts: int
    top: int
    groups: Optional[tuple]       # (count, keep) or None
    shared_ff: Optional[int]


@dataclass(frozen=True)
class RaranexLayerConfig:
    kind: str                               # "attention" or "parallel"
    attention: AttentionConfig              # the mixer, or its left half
    recurrence: Optional[RecurrenceConfig]  # the right half of "parallel"
    mlp: Optional[RoutedConfig]             # None: no feed-forward


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


def _attention(m: dict, where: str, windowed: bool) -> AttentionConfig:
    kw = dict(heads=int(_need(m, "heads", where)), kv_heads=int(_need(m, "kv_heads", where)), dim=int(_need(m, "dim", where)),
              vdim=int(_need(m, "vdim", where)), scale=float(_need(m, "scale", where)))
    if windowed:
        mask, rot = _need(m, "mask", where), _need(m, "rot", where)
        kw.update(window=int(_need(mask, "size", where + "mask.")), keep_first=int(mask.get("keep_first") or 0),
                  rot_base=float(_need(rot, "base", where + "rot.")), rot_dims=int(_need(rot, "dims", where + "rot.")))
    else:
        if m.get("softcap") is not None:
            kw["softcap"] = float(m["softcap"])
        if m.get("q_temp") is not None:
            qt = m["q_temp"]
            kw["q_temp"] = (float(_need(qt, "coef", where + "q_temp.")), int(_need(qt, "every", where + "q_temp.")))
    return AttentionConfig(**kw)


@dataclass(frozen=True)
class RaranexConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    loop: Optional[LoopConfig]

    @classmethod
    def from_dict(cls, d: dict) -> "RaranexConfig":
        if d.get("architecture", NAME) != NAME and NAME not in (d.get("architectures") or []):
            raise ValueError(f"expected a {NAME} model, got architecture={d.get('architecture')!r}")
        entries = _need(d, "layers", "")
        if not isinstance(entries, list) or not entries:
            raise ValueError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            if kind not in MIXER_KINDS:
                raise NotImplementedError(f"{where}type {kind!r} is not a layer of this design {MIXER_KINDS}")
            m, mw = _need(entry, "mixer", where), where + "mixer."
            recurrence = None
            if kind == "attention":
                attention = _attention(m, mw, windowed=True)
            else:
                attention = _attention(_need(m, "left", mw), mw + "left.", windowed=False)
                r, rw = _need(m, "right", mw), mw + "right."
                recurrence = RecurrenceConfig(heads=int(_need(r, "heads", rw)), dim=int(_need(r, "dim", rw)),
                                              rank=int(r["rank"]) if r.get("rank") is not None else None)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                fw = where + "mlp."
                ff_kind = _need(mlp, "kind", fw)
                if ff_kind != "moe":
                    raise NotImplementedError(f"{fw}kind {ff_kind!r} is not a feed-forward of this design ('moe')")
                router = _need(mlp, "router", fw)
                groups = router.get("groups")
                shared = mlp.get("shared")
                ff = RoutedConfig(ff=int(_need(_need(mlp, "expert", fw), "ff", fw + "expert.")),
                                  experts=int(_need(router, "experts", fw + "router.")), top=int(_need(router, "top", fw + "router.")),
                                  groups=None if groups is None else (int(_need(groups, "count", fw + "router.groups.")),
                                                                      int(_need(groups, "keep", fw + "router.groups."))),
                                  shared_ff=None if shared is None else int(_need(shared, "ff", fw + "shared.")))
            layers.append(RaranexLayerConfig(kind, attention, recurrence, ff))
        loop = d.get("loop")
        if loop is not None:
            loop = LoopConfig(int(_need(loop, "start", "loop.")), int(_need(loop, "stop", "loop.")), int(_need(loop, "times", "loop.")))
        cfg = cls(vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
                  eps=float(_need(_need(d, "norm", ""), "eps", "norm.")), layers=tuple(layers), loop=loop)
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab", "width"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if not self.eps > 0:
            raise ValueError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            a = layer.attention
            if min(a.heads, a.kv_heads, a.dim, a.vdim) <= 0 or (a.window is not None and a.window <= 0) or a.keep_first < 0:
                raise ValueError(f"layers[{i}]: sizes must be positive")
            if a.heads % a.kv_heads:
                raise ValueError(f"layers[{i}]: {a.heads} heads are not a multiple of {a.kv_heads} kv_heads")
            if a.rot_dims % 2 or not 0 <= a.rot_dims <= a.dim:
                raise ValueError(f"layers[{i}]: rot.dims {a.rot_dims} must be even and at most dim {a.dim}")
            if a.q_temp is not None and a.q_temp[1] < 1:
                raise ValueError(f"layers[{i}]: q_temp.every must be positive")
            r = layer.recurrence
            if r is not None and (min(r.heads, r.dim) <= 0 or (r.rank is not None and r.rank <= 0)):
                raise ValueError(f"layers[{i}]: the recurrence's sizes must be positive")
            f = layer.mlp
            if f is not None:
                if f.ff <= 0 or not 1 <= f.top <= f.experts or (f.shared_ff is not None and f.shared_ff <= 0):
                    raise ValueError(f"layers[{i}]: router.top {f.top} of {f.experts} experts of inner width {f.ff}")
                if f.groups is not None:
                    count, keep = f.groups
                    if count < 1 or f.experts % count or not 1 <= keep <= count or (f.experts // count) * keep < f.top:
                        raise ValueError(f"layers[{i}]: {f.experts} experts in {count} groups of which {keep} are kept "
                                         f"cannot give {f.top} experts a token")
        if self.loop is not None:
            lp = self.loop
            if not 0 <= lp.start <= lp.stop <= len(self.layers) or lp.times < 1:
                raise ValueError(f"loop {lp.start}..{lp.stop} x {lp.times} does not fit {len(self.layers)} layers")

    def run_order(self) -> list:
        """[(layer, number of the pass that begins with it or None)], in the order the layers run."""
        n = len(self.layers)
        lp = self.loop
        if lp is None or lp.stop <= lp.start:
            return [(i, None) for i in range(n)]
        order = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t if i == lp.start else None) for i in range(lp.start, lp.stop)]
        return order + [(i, None) for i in range(lp.stop, n)]


def with_checkpoint_shapes(config: dict, shapes: dict) -> dict:
    """``config`` with the decay rank of every recurrence set from the checkpoint's tensor shapes
    (``shapes``: name -> shape) where the configuration does not give it."""
    out = dict(config)
    out["layers"] = []
    for i, entry in enumerate(config.get("layers") or []):
        entry = dict(entry)
        name = f"l{i}.mix.right.w1"
        right = (entry.get("mixer") or {}).get("right") if isinstance(entry.get("mixer"), dict) else None
        if isinstance(right, dict) and right.get("rank") is None and name in shapes:
            entry["mixer"] = dict(entry["mixer"], right=dict(right, rank=int(shapes[name][0])))
        out["layers"].append(entry)
    return out


def _attention_spec(W: int, a: AttentionConfig, eps: float, windowed: bool) -> GatedAttentionSpec:
    common = dict(hidden_size=W, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim, scale=a.scale,
                  norm_eps=eps, qk_norm=True, values="projection", output_gate=True, gate_per_head=True)
    if windowed:
        return GatedAttentionSpec(window=a.window, keep_first=a.keep_first, qk_norm_weight=False, qk_norm_after_rotation=True,
                                  position=RopePairsSpec(rotary_dim=a.rot_dims, theta=a.rot_base) if a.rot_dims else None, **common)
    return GatedAttentionSpec(qk_norm_weight=True, softcap=a.softcap, query_temperature=a.q_temp, **common)


def build_spec(cfg: RaranexConfig) -> ModelSpec:
    W = cfg.width
    norm = RMSNormSpec(size=W, eps=cfg.eps)
    layers = []
    for layer in cfg.layers:
        if layer.kind == "attention":
            mixer = _attention_spec(W, layer.attention, cfg.eps, windowed=True)
        else:
            r = layer.recurrence
            right = ShiftedRecurrenceSpec(hidden_size=W, num_heads=r.heads, head_dim=r.dim,
                                          decay_rank=r.rank if r.rank is not None else DEFAULT_DECAY_RANK, norm_eps=cfg.eps)
            mixer = PairMixerSpec(hidden_size=W, left=_attention_spec(W, layer.attention, cfg.eps, windowed=False), right=right,
                                  eps=cfg.eps)
        f = layer.mlp
        feed_forward = None
        if f is not None:
            feed_forward = RoutedExpertsSpec(
                hidden_size=W, intermediate_size=f.ff, num_experts=f.experts, top_k=f.top, router="sigmoid", renormalize=True,
                weight_on="output", choice_correction=True, groups=None if f.groups is None else (*f.groups, GROUP_SCORE_TOP),
                renorm_eps=RENORM_EPS, shared_intermediate=f.shared_ff, shared_gate=f.shared_ff is not None)
        layers.append(LayerSpec(arrangement="twonorm", mixer=mixer, mixer_norm=norm, feed_forward=feed_forward,
                                ffn_norm=norm if feed_forward is not None else None))
    order = cfg.run_order()
    reenters = any(t is not None for _, t in order)
    spec = ModelSpec(
        architecture=NAME, vocab_size=cfg.vocab, hidden_size=W, layers=layers,
        run=[RunEntry(layer=i, reenter=t) for i, t in order],
        final_norm=norm, tie_embeddings=False,
        embedding=TokenEmbeddingSpec(cfg.vocab, W), head=LinearHeadSpec(cfg.vocab, W),
        reentry=StreamReentrySpec(W, cfg.loop.times) if reenters else None,
        info={"layers": len(layers), "layer_runs": len(order), "hidden": W, "vocab": cfg.vocab,
              "kinds": [l.kind for l in cfg.layers], "tied": False},
    )
    spec.validate()
    return spec


def _attention_plan(dst: str, mix: str, W: int, a: AttentionConfig, weighted_norm: bool) -> list:
    """q, k, v and the gates read the same input: one product, stacked along the output dimension."""
    nq, nk, nv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
    plan = [WeightTarget(f"{dst}.in_weight", (f"{mix}.q", f"{mix}.k", f"{mix}.v", f"{mix}.g"), ((nq, W), (nk, W), (nv, W), (a.heads, W))),
            WeightTarget(f"{dst}.out_weight", (f"{mix}.o",), ((W, a.heads * a.vdim),))]
    if weighted_norm:
        plan += [WeightTarget(f"{dst}.q_norm", (f"{mix}.q.norm",), ((a.dim,),)),
                 WeightTarget(f"{dst}.k_norm", (f"{mix}.k.norm",), ((a.dim,),))]
    return plan


def weight_plan(cfg: RaranexConfig, spec: ModelSpec) -> list[WeightTarget]:
    """Checkpoint names -> the model's parameters. What reads the same input is stacked into one
    parameter: q, k, v and the gates of an attention mixer; the recurrence's five mixing vectors,
    and its r, k, v and gate matrices; the router's rows with the shared expert's gate row; the
    experts' gate and up matrices, expert by expert, and their down matrices; the shared expert's
    gate and up."""
    W = cfg.width
    plan = [WeightTarget("embed.weight", ("embed",), ((cfg.vocab, W),))]
    if spec.reentry is not None:
        plan += [WeightTarget("reentry.in_weight", ("loop.in",), ((W, 2 * W),)),
                 WeightTarget("reentry.step", ("loop.step",), ((cfg.loop.times, W),))]
    for i, layer in enumerate(cfg.layers):
        src, dst, mix = f"l{i}", f"layers.{i}", f"l{i}.mix"
        plan.append(WeightTarget(f"{dst}.mixer_norm.weight", (f"{src}.norm1",), ((W,),)))
        if layer.kind == "attention":
            plan += _attention_plan(f"{dst}.mixer", mix, W, layer.attention, weighted_norm=False)
        else:
            plan += _attention_plan(f"{dst}.mixer.left", f"{mix}.left", W, layer.attention, weighted_norm=True)
            r = layer.recurrence
            inner, rank = r.heads * r.dim, spec.layers[i].mixer.right.decay_rank
            right, rd = f"{mix}.right", f"{dst}.mixer.right"
            plan += [
                WeightTarget(f"{rd}.mix", tuple(f"{right}.mu.{s}" for s in SHIFT_MIXES), ((W,),) * len(SHIFT_MIXES)),
                WeightTarget(f"{rd}.rkvg_weight", tuple(f"{right}.{s}" for s in ("r", "k", "v", "g")), ((inner, W),) * 4),
                WeightTarget(f"{rd}.decay_in_weight", (f"{right}.w1",), ((rank, W),)),
                WeightTarget(f"{rd}.decay_weight", (f"{right}.w2",), ((inner, rank),)),
                WeightTarget(f"{rd}.decay_bias", (f"{right}.w0",), ((inner,),)),
                WeightTarget(f"{rd}.bonus", (f"{right}.u",), ((r.heads, r.dim),)),
                WeightTarget(f"{rd}.norm_weight", (f"{right}.norm",), ((inner,),)),
                WeightTarget(f"{rd}.out_weight", (f"{right}.o",), ((W, inner),)),
                WeightTarget(f"{dst}.mixer.left_out_norm", (f"{mix}.left.out",), ((W,),)),
                WeightTarget(f"{dst}.mixer.right_out_norm", (f"{mix}.right.out",), ((W,),)),
            ]
        f = layer.mlp
        if f is None:
            continue
        ff, mlp = f"{dst}.feed_forward", f"{src}.mlp"
        plan.append(WeightTarget(f"{dst}.ffn_norm.weight", (f"{src}.norm2",), ((W,),)))
        gate_up = tuple(f"{mlp}.e{e}.{n}" for e in range(f.experts) for n in ("gate", "up"))
        down = tuple(f"{mlp}.e{e}.down" for e in range(f.experts))
        router = (f"{mlp}.router",) + ((f"{mlp}.shared.sg",) if f.shared_ff is not None else ())
        plan += [WeightTarget(f"{ff}.router_weight", router, ((f.experts, W),) + (((1, W),) if f.shared_ff is not None else ())),
                 WeightTarget(f"{ff}.correction", (f"{mlp}.correction",), ((f.experts,),)),
                 WeightTarget(f"{ff}.gate_up_weight", gate_up, ((f.ff, W),) * len(gate_up)),
                 WeightTarget(f"{ff}.down_weight", down, ((W, f.ff),) * len(down))]
        if f.shared_ff is not None:
            plan += [WeightTarget(f"{ff}.shared_gate_up_weight", (f"{mlp}.shared.gate", f"{mlp}.shared.up"), ((f.shared_ff, W),) * 2),
                     WeightTarget(f"{ff}.shared_down_weight", (f"{mlp}.shared.down",), ((W, f.shared_ff),))]
    plan.append(WeightTarget("final_norm.weight", ("final.norm",), ((W,),)))
    plan.append(WeightTarget("lm_head.weight", ("head",), ((cfg.vocab, W),)))
    return plan


ARCHITECTURE = Architecture(name=NAME, parse_config=RaranexConfig.from_dict, build_spec=build_spec, weight_plan=weight_plan,
                            sizes_from_checkpoint=with_checkpoint_shapes)
register_architecture([NAME], ARCHITECTURE)
