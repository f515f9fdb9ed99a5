"""A plain, slow Nenodra: whole sequences, no cache, one function per mechanism.

Shares no code with ``clockwork_amd``: it reads config.json and the safetensors file itself and
runs on the CPU in ``dtype`` (float64 by default, so that all of an error is the engine's).

The design in this file's notation. Tokens t at positions p = 0, 1, ...; the stream x_p has
``width`` elements; c = ``residual_mult``.

* input: x_p = embed[t_p].
* a layer: x <- x + c * N1(M(x)); x <- x + c * N2(F(x)) (F absent where the layer has none). Mixer
  and feed-forward read the stream as it is; what is normed is their OUTPUT, with
  N(y) = y / sqrt(mean(y^2) + eps) * (1 + w).
* shared by both mixers: H query heads over G key/value heads (head a reads key/value head
  a // (H / G)); every query and key vector of ``dim`` elements is divided by its root mean square
  and multiplied by a weight of ``dim`` elements (one for all query vectors, one for all key
  vectors of the layer), then its first ``rot.dims`` elements are rotated by position: element i
  with element i + rot.dims / 2, angle p * rot.base^(-2 i / rot.dims). Position i sees the keys
  j with 0 <= i - j < mask.size; softmax of scale * q . k over them.
* M "attention": two score maps a head. Queries [H, 2, dim] and keys [G, 2, dim] (each of the
  vectors normed and rotated by itself) and values [G, vdim] come from biased projections. With
  lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff the head's output is o = A_1 - lam * A_2 (both maps
  applied to the same values), divided by its root mean square over vdim and multiplied by
  (1 - diff); the heads are concatenated and projected with a bias.
* M "attention_2": one map, no biases; the values are the key projections as they come out of the
  product, before norm and rotation. The concatenated heads are multiplied by
  logistic(g x) and projected.
* F "dense": down(relu(up x)^2).
* F "moe": r = logistic(router x); the ``top`` experts with the largest r are taken (the lower
  index first among equals); the result is the sum over them of E_e(r_e * x) with
  E(u) = down(silu(gate u) * (up u)).
* output: N(x) with the final norm's weight, times ``head``, times ``logit_scale``.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import load_file


# ------------------------------------------------------------------------------- small pieces
def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def output_norm(y, weight, eps):
    """The design's norm: the weight is kept as its distance from one."""
    return unit_rms(y, eps) * (1.0 + weight)


def logistic(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * logistic(z)


def relu_squared(z):
    r = torch.clamp(z, min=0.0)
    return r * r


def rotate_first(v, positions, base, dims):
    """v [T, ..., n >= dims]: among the first ``dims`` elements, element i turns with element
    i + dims / 2 by the angle position * base^(-2 i / dims); the rest stay."""
    half = dims // 2
    if half == 0:
        return v
    freq = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=v.dtype)
    angle = torch.as_tensor(positions, dtype=v.dtype)[:, None] * freq[None, :]
    while angle.dim() < v.dim():
        angle = angle.unsqueeze(1)
    cos, sin = torch.cos(angle), torch.sin(angle)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


def normed_rotated(v, weight, eps, positions, rot):
    """Every vector of the last dimension: unit root mean square, weight, rotation."""
    return rotate_first(unit_rms(v, eps) * weight, positions, float(rot["base"]), int(rot["dims"]))


def windowed_softmax_rows(q, k, scale, window):
    """q [T, dim], k [T, dim] -> weights [T, T]: row i holds the softmax over the keys
    max(0, i - window + 1) .. i, zeros elsewhere."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) & (i - j < window)
    s = torch.where(seen, s, torch.full_like(s, float("-inf")))
    return torch.softmax(s, dim=-1)


# ------------------------------------------------------------------------------- the two mixers
def two_map_window_attention(x, w, pre, m, eps, positions=None):
    """x [T, width]; ``w`` the tensors, ``pre`` the prefix of this mixer's names, ``m`` its sizes."""
    T = x.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    window, diff, scale = int(m["mask"]["size"]), float(m["diff"]), float(m["scale"])
    positions = list(range(T)) if positions is None else positions
    q = (x @ w[pre + "q"].t() + w[pre + "q.b"]).view(T, H, 2, D)
    k = (x @ w[pre + "k"].t() + w[pre + "k.b"]).view(T, G, 2, D)
    v = (x @ w[pre + "v"].t() + w[pre + "v.b"]).view(T, G, V)
    q = normed_rotated(q, w[pre + "q.norm"], eps, positions, m["rot"])
    k = normed_rotated(k, w[pre + "k.norm"], eps, positions, m["rot"])
    lam = torch.exp((w[pre + "lq1"] * w[pre + "lk1"]).sum()) - torch.exp((w[pre + "lq2"] * w[pre + "lk2"]).sum()) + diff
    heads = []
    for a in range(H):
        g = a // (H // G)
        first = windowed_softmax_rows(q[:, a, 0], k[:, g, 0], scale, window) @ v[:, g]
        second = windowed_softmax_rows(q[:, a, 1], k[:, g, 1], scale, window) @ v[:, g]
        heads.append(unit_rms(first - lam * second, eps) * (1.0 - diff))
    return torch.cat(heads, dim=-1) @ w[pre + "o"].t() + w[pre + "o.b"]


def keys_as_values_attention(x, w, pre, m, eps, positions=None):
    T = x.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    if V != D:
        raise ValueError("the values are the key projections: vdim must equal dim")
    window, scale = int(m["mask"]["size"]), float(m["scale"])
    positions = list(range(T)) if positions is None else positions
    q = (x @ w[pre + "q"].t()).view(T, H, D)
    raw = (x @ w[pre + "k"].t()).view(T, G, D)
    q = normed_rotated(q, w[pre + "q.norm"], eps, positions, m["rot"])
    k = normed_rotated(raw, w[pre + "k.norm"], eps, positions, m["rot"])
    heads = [windowed_softmax_rows(q[:, a], k[:, a // (H // G)], scale, window) @ raw[:, a // (H // G)] for a in range(H)]
    gate = logistic(x @ w[pre + "g"].t())
    return (torch.cat(heads, dim=-1) * gate) @ w[pre + "o"].t()


MIXERS = {"attention": two_map_window_attention, "attention_2": keys_as_values_attention}


# ------------------------------------------------------------------------------- feed-forwards
def dense_feed_forward(x, w, pre):
    return relu_squared(x @ w[pre + "up"].t()) @ w[pre + "down"].t()


def routed_choice(x, w, pre, top):
    """(chosen experts [T, top], their scores [T, top]): the largest logistic(router x), the lower
    index first among equals."""
    r = logistic(x @ w[pre + "router"].t())
    order = torch.sort(r, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(r, 1, order)


def expert(u, w, pre):
    return (silu(u @ w[pre + "gate"].t()) * (u @ w[pre + "up"].t())) @ w[pre + "down"].t()


def routed_feed_forward(x, w, pre, mlp):
    top = int(mlp["router"]["top"])
    chosen, score = routed_choice(x, w, pre, top)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e, r in zip(chosen[t].tolist(), score[t]):
            out[t] = out[t] + expert(r * x[t], w, f"{pre}e{e}.")
    return out


def feed_forward(x, w, pre, mlp):
    if mlp["kind"] == "dense":
        return dense_feed_forward(x, w, pre)
    if mlp["kind"] == "moe":
        return routed_feed_forward(x, w, pre, mlp)
    raise ValueError(f"feed-forward kind {mlp['kind']!r}")


def layer(x, w, i, entry, eps, mult, positions=None):
    if entry["type"] not in MIXERS:
        raise ValueError(f"layer type {entry['type']!r}")
    p = f"l{i}."
    x = x + mult * output_norm(MIXERS[entry["type"]](x, w, p + "mix.", entry["mixer"], eps, positions), w[p + "norm1"], eps)
    if entry.get("mlp") is not None:
        x = x + mult * output_norm(feed_forward(x, w, p + "mlp.", entry["mlp"]), w[p + "norm2"], eps)
    return x


class PlainNenodra:
    def __init__(self, model_dir, dtype=torch.float64):
        model_dir = Path(model_dir)
        self.cfg = json.loads((model_dir / "config.json").read_text())
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
        self.dtype = dtype

    def streams(self, tokens):
        """The stream after every layer, [layers, T, width]."""
        cfg, w = self.cfg, self.w
        x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        out = []
        for i, entry in enumerate(cfg["layers"]):
            x = layer(x, w, i, entry, cfg["norm"]["eps"], cfg["residual_mult"])
            out.append(x)
        return torch.stack(out)

    def logits(self, tokens):
        x = self.streams(tokens)[-1]
        return (output_norm(x, self.w["final.norm"], self.cfg["norm"]["eps"]) @ self.w["head"].t() * self.cfg["logit_scale"]).float()

    def greedy(self, prompt, n):
        tokens = list(prompt)
        for _ in range(n):
            tokens.append(int(self.logits(tokens)[-1].argmax()))
        return tokens[len(prompt):]
