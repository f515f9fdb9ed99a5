"""Nenodra: config.json keys -> typed config -> parts -> weight names.

A decoder whose sublayers read the float32 residual stream itself and whose norms sit on their
OUTPUT: x <- x + residual_mult * N(mixer(x)), then x <- x + residual_mult * N(ff(x)), with
N(y) = y / sqrt(mean(y^2) + eps) * (1 + w). A layer's mixer is one of two kinds, both grouped
attention behind a sliding window with every query and key vector RMS-normed (a weight of ``dim``
elements for all query vectors of the layer, one for all key vectors) and then partly rotated by
position: "attention" has two score maps a head over shared values, biased projections, and the
head's output map 1 - lambda * map 2 divided by its root mean square and multiplied by 1 - diff;
"attention_2" has one map, no biases, the raw key projections as its values and a logistic gate on
the concatenated heads. The feed-forward is dense, down(relu(up x)^2), routed (a logistic router,
the ``top`` largest scores, each expert fed its score times x, experts gated with silu), or absent.
The output is N(x) with the model's norm, an untied head and a constant factor on the logits.

Every size and every constant that can differ between models of the design is read from
config.json: ``vocab``, ``width``, ``residual_mult``, ``logit_scale``, ``norm.eps`` and, per entry
of ``layers``, ``type``, ``mixer`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``,
``mask.size``, ``rot.base``, ``rot.dims``, and ``diff`` for "attention") and ``mlp`` (``kind``
"dense": ``ff``; "moe": ``expert.ff``, ``router.experts``, ``router.top``; null: no feed-forward).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry, WeightTarget
from clockwork_amd.parts.specs import (BranchRMSNormSpec, DenseMLPSpec, DifferentialAttentionSpec, GatedAttentionSpec,
                                       LinearHeadSpec, RopeNeoxSpec, RoutedExpertsSpec, TokenEmbeddingSpec)
from clockwork_amd.registry import Architecture, register_architecture

NAME = "Nenodra"
MIXER_KINDS = ("attention", "attention_2")


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ValueError(f"config.json lacks {where}{key}")
    return d[key]


@dataclass(frozen=True)
class WindowMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    rot_base: float
    rot_dims: int
    diff: Optional[float] = None   # the two-map mixer's constant; None for the one-map mixer


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str          # "dense" or "moe"
    ff: int            # dense: the inner width; moe: one expert's
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class NenodraLayerConfig:
    kind: str                          # "attention" or "attention_2"
    mixer: WindowMixerConfig
    mlp: Optional[FeedForwardConfig]   # None: no feed-forward


@dataclass(frozen=True)
class NenodraConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_scale: float
    layers: tuple

    @classmethod
    def from_dict(cls, d: dict) -> "NenodraConfig":
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
            rot = _need(m, "rot", mw)
            mixer = WindowMixerConfig(
                heads=int(_need(m, "heads", mw)), kv_heads=int(_need(m, "kv_heads", mw)), dim=int(_need(m, "dim", mw)),
                vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)),
                window=int(_need(_need(m, "mask", mw), "size", mw + "mask.")),
                rot_base=float(_need(rot, "base", mw + "rot.")), rot_dims=int(_need(rot, "dims", mw + "rot.")),
                diff=float(_need(m, "diff", mw)) if kind == "attention" else None)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                fw = where + "mlp."
                ff_kind = _need(mlp, "kind", fw)
                if ff_kind == "dense":
                    ff = FeedForwardConfig("dense", int(_need(mlp, "ff", fw)))
                elif ff_kind == "moe":
                    router = _need(mlp, "router", fw)
                    ff = FeedForwardConfig("moe", int(_need(_need(mlp, "expert", fw), "ff", fw + "expert.")),
                                           experts=int(_need(router, "experts", fw + "router.")),
                                           top=int(_need(router, "top", fw + "router.")))
                else:
                    raise NotImplementedError(f"{fw}kind {ff_kind!r} is not a feed-forward of this design ('dense', 'moe')")
            layers.append(NenodraLayerConfig(kind, mixer, ff))
        cfg = cls(vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
                  eps=float(_need(_need(d, "norm", ""), "eps", "norm.")), residual_mult=float(_need(d, "residual_mult", "")),
                  logit_scale=float(_need(d, "logit_scale", "")), layers=tuple(layers))
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab", "width"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if not self.eps > 0:
            raise ValueError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.kv_heads, m.dim, m.vdim, m.window) <= 0:
                raise ValueError(f"layers[{i}]: sizes must be positive")
            if m.heads % m.kv_heads:
                raise ValueError(f"layers[{i}]: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
            if m.rot_dims % 2 or not 0 <= m.rot_dims <= m.dim:
                raise ValueError(f"layers[{i}]: rot.dims {m.rot_dims} must be even and at most dim {m.dim}")
            if layer.kind == "attention_2" and m.vdim != m.dim:
                raise ValueError(f"layers[{i}]: the values of 'attention_2' are its keys: vdim {m.vdim} must equal dim {m.dim}")
            f = layer.mlp
            if f is not None:
                if f.ff <= 0:
                    raise ValueError(f"layers[{i}]: the feed-forward's inner width must be positive")
                if f.kind == "moe" and not 1 <= f.top <= f.experts:
                    raise ValueError(f"layers[{i}]: router.top {f.top} must be between 1 and router.experts {f.experts}")


def build_spec(cfg: NenodraConfig) -> ModelSpec:
    W = cfg.width
    norm = BranchRMSNormSpec(size=W, eps=cfg.eps, branch_scale=cfg.residual_mult, weight_offset=1.0)
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        rope = RopeNeoxSpec(rotary_dim=m.rot_dims, theta=m.rot_base) if m.rot_dims else None
        if layer.kind == "attention":
            mixer = DifferentialAttentionSpec(hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim,
                                              value_dim=m.vdim, scale=m.scale, lambda_init=m.diff, norm_eps=cfg.eps,
                                              window=m.window, qkv_bias=True, qk_norm=True, position=rope, out_bias=True)
        else:
            mixer = GatedAttentionSpec(hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim,
                                       value_dim=m.vdim, scale=m.scale, norm_eps=cfg.eps, window=m.window, qk_norm=True,
                                       position=rope, values="keys", output_gate=True)
        f = layer.mlp
        if f is None:
            feed_forward = None
        elif f.kind == "dense":
            feed_forward = DenseMLPSpec(W, f.ff, activation="relu2")
        else:
            feed_forward = RoutedExpertsSpec(hidden_size=W, intermediate_size=f.ff, num_experts=f.experts, top_k=f.top,
                                             router="sigmoid", renormalize=False, weight_on="input")
        layers.append(LayerSpec(arrangement="branchnorm", mixer=mixer, mixer_norm=norm, feed_forward=feed_forward,
                                ffn_norm=norm if feed_forward is not None else None))
    spec = ModelSpec(
        architecture=NAME, vocab_size=cfg.vocab, hidden_size=W, layers=layers,
        run=[RunEntry(layer=i) for i in range(len(layers))],
        final_norm=norm, tie_embeddings=False,
        embedding=TokenEmbeddingSpec(cfg.vocab, W), head=LinearHeadSpec(cfg.vocab, W, scale=cfg.logit_scale),
        info={"layers": len(layers), "hidden": W, "vocab": cfg.vocab, "kinds": [l.kind for l in cfg.layers],
              "ff": [None if l.mlp is None else (l.mlp.kind, l.mlp.ff, l.mlp.experts, l.mlp.top) for l in cfg.layers],
              "tied": False},
    )
    spec.validate()
    return spec


def weight_plan(cfg: NenodraConfig, spec: ModelSpec) -> list[WeightTarget]:
    """Checkpoint names -> the model's parameters. Projections that read the same input are run as
    one product, so they are stacked along the output dimension: q, k, v (and their biases) of the
    two-map mixer; q, k and the gate of the one-map mixer; the experts' gate and up matrices, expert
    by expert, and their down matrices."""
    W = cfg.width
    plan = [WeightTarget("embed.weight", ("embed",), ((cfg.vocab, W),))]
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}", f"layers.{i}"
        m, mix = layer.mixer, f"l{i}.mix"
        plan.append(WeightTarget(f"{dst}.mixer_norm.weight", (f"{src}.norm1",), ((W,),)))
        plan += [WeightTarget(f"{dst}.mixer.q_norm", (f"{mix}.q.norm",), ((m.dim,),)),
                 WeightTarget(f"{dst}.mixer.k_norm", (f"{mix}.k.norm",), ((m.dim,),)),
                 WeightTarget(f"{dst}.mixer.out_weight", (f"{mix}.o",), ((W, m.heads * m.vdim),))]
        if layer.kind == "attention":
            nq, nk, nv = m.heads * 2 * m.dim, m.kv_heads * 2 * m.dim, m.kv_heads * m.vdim
            plan += [
                WeightTarget(f"{dst}.mixer.qkv_weight", (f"{mix}.q", f"{mix}.k", f"{mix}.v"), ((nq, W), (nk, W), (nv, W))),
                WeightTarget(f"{dst}.mixer.qkv_bias", (f"{mix}.q.b", f"{mix}.k.b", f"{mix}.v.b"), ((nq,), (nk,), (nv,))),
                WeightTarget(f"{dst}.mixer.out_bias", (f"{mix}.o.b",), ((W,),)),
            ]
            plan += [WeightTarget(f"{dst}.mixer.{n}", (f"{mix}.{n}",), ((m.dim,),)) for n in ("lq1", "lk1", "lq2", "lk2")]
        else:
            nq, nk, no = m.heads * m.dim, m.kv_heads * m.dim, m.heads * m.vdim
            plan.append(WeightTarget(f"{dst}.mixer.in_weight", (f"{mix}.q", f"{mix}.k", f"{mix}.g"), ((nq, W), (nk, W), (no, W))))
        f = layer.mlp
        if f is None:
            continue
        plan.append(WeightTarget(f"{dst}.ffn_norm.weight", (f"{src}.norm2",), ((W,),)))
        if f.kind == "dense":
            plan += [WeightTarget(f"{dst}.feed_forward.up_weight", (f"{src}.mlp.up",), ((f.ff, W),)),
                     WeightTarget(f"{dst}.feed_forward.down_weight", (f"{src}.mlp.down",), ((W, f.ff),))]
        else:
            gate_up = tuple(f"{src}.mlp.e{e}.{n}" for e in range(f.experts) for n in ("gate", "up"))
            down = tuple(f"{src}.mlp.e{e}.down" for e in range(f.experts))
            plan += [WeightTarget(f"{dst}.feed_forward.router_weight", (f"{src}.mlp.router",), ((f.experts, W),)),
                     WeightTarget(f"{dst}.feed_forward.gate_up_weight", gate_up, ((f.ff, W),) * len(gate_up)),
                     WeightTarget(f"{dst}.feed_forward.down_weight", down, ((W, f.ff),) * len(down))]
    plan.append(WeightTarget("final_norm.weight", ("final.norm",), ((W,),)))
    plan.append(WeightTarget("lm_head.weight", ("head",), ((cfg.vocab, W),)))
    return plan


ARCHITECTURE = Architecture(name=NAME, parse_config=NenodraConfig.from_dict, build_spec=build_spec, weight_plan=weight_plan)
register_architecture([NAME], ARCHITECTURE)
