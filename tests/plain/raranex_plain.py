"""A plain, slow Raranex: whole sequences, no cache, one function per mechanism.

Shares no code with ``clockwork_amd``: it reads config.json and the safetensors file itself and
runs on the CPU in ``dtype`` (float64 by default, so that all of an error is the engine's).

The design in this file's notation. Tokens t at positions p = 0, 1, ...; the stream x_p has
``width`` elements; N(x; w) = x / sqrt(mean(x^2) + eps) * w, U(x) the same without a weight.

* input: e_p = embed[t_p]; the stream starts as e.
* order: the layers before ``loop.start`` once, then the layers ``loop.start .. loop.stop - 1``
  ``loop.times`` times over with the same weights, then the others once. Right before pass n of
  the repeated run (n = 0 too) the stream is re-entered: x <- R [x; e] + s_n with R = 'loop.in'
  [width, 2 width] and s = 'loop.step' [times, width].
* a layer: x <- x + M(N(x; norm1)) + F(N(x; norm2)); F absent where the layer has none.
* M "attention": H query heads over G key/value heads (head a reads key/value head a // (H / G)).
  Queries and keys are rotated over their first ``rot.dims`` elements, neighbours in pairs:
  (v_2i, v_2i+1) turns by p * rot.base^(-2 i / rot.dims); then each vector is divided by its root
  mean square. Position i sees j <= i with i - j < mask.size or j < mask.keep_first. Softmax of
  scale * q . k; head a's result times logistic(g x)_a; output projection.
* M "parallel": (N(L(h); left.out) + N(T(h); right.out)) / 2 with
  L: attention without rotation. Queries and keys N-normed per head with weights of ``dim``
  elements; the query at position p times 1 + coef * ln(floor((p + 1) / every) + 1);
  scores c * tanh(scale * q . k / c) with c = softcap; every j <= i seen; softmax; the same
  per-head gate and output projection.
  T: a recurrence over a matrix a head. With h_-1 = 0, m^s_p = h_p + (h_(p-1) - h_p) * mu_s for s
  in r, k, v, g, w; r, k, v = W_s m^s cut into heads of ``dim``; gate = silu(W_g m^g);
  decay d = exp(-exp(w2 tanh(w1 m^w) + w0)), one number a head and key channel. A head with
  state S [dim, dim] (S = 0 before position 0): o_p = (S + diag(u) k_p v_p^T)^T r_p, then
  S <- diag(d_p) S + k_p v_p^T. Result: concat_a U(o_a) * norm * gate, projected with W_o.
* F: logistic router z = router x, s = logistic(z), choice score c = s + correction. Experts lie
  in ``groups.count`` equal runs; a run's score is the sum of its two largest c; only experts of
  the ``groups.keep`` best runs can be chosen. The ``top`` largest c among those are taken (the
  lower index first among equals), each weighted s_e / (sum of the chosen s + 1e-20). Expert:
  down(silu(gate h) * (up h)). A shared expert of the same form runs for every token, times
  logistic(sg h).
* output: N(x; final.norm), times ``head``.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


# ------------------------------------------------------------------------------- small pieces
def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def weighted_norm(y, weight, eps):
    return unit_rms(y, eps) * weight


def logistic(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * logistic(z)


def rotate_neighbours(v, positions, base, dims):
    """v [T, heads, n >= dims]: elements 2i and 2i + 1 (2i + 1 < dims) turn together by the angle
    position * base^(-2 i / dims); the rest stay."""
    out = v.clone()
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        angle = torch.as_tensor([p * f for p in positions], dtype=v.dtype)[:, None]
        c, s = torch.cos(angle), torch.sin(angle)
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def seen_mask(positions, size=None, keep_first=0):
    """[T, T] booleans: row i sees column j when j is not later and either within ``size``
    positions (None: any distance) or among the first ``keep_first`` positions."""
    p = torch.as_tensor(positions)
    i, j = p[:, None], p[None, :]
    near = (i - j < size) if size is not None else torch.ones_like(i - j, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def masked_softmax(scores, seen):
    return torch.softmax(torch.where(seen, scores, torch.full_like(scores, float("-inf"))), dim=-1)


def head_gate(h, w_g):
    """[T, heads]: one logistic gate a head, from the mixer's input."""
    return logistic(h @ w_g.t())


# ------------------------------------------------------------------------------- mixers
def window_attention(h, w, pre, m, eps, positions=None):
    """The "attention" mixer. h [T, width]."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = list(range(T)) if positions is None else positions
    q = (h @ w[pre + "q"].t()).view(T, H, D)
    k = (h @ w[pre + "k"].t()).view(T, G, D)
    v = (h @ w[pre + "v"].t()).view(T, G, V)
    q = unit_rms(rotate_neighbours(q, positions, m["rot"]["base"], int(m["rot"]["dims"])), eps)
    k = unit_rms(rotate_neighbours(k, positions, m["rot"]["base"], int(m["rot"]["dims"])), eps)
    seen = seen_mask(positions, int(m["mask"]["size"]), int(m["mask"]["keep_first"]))
    gate = head_gate(h, w[pre + "g"])
    heads = []
    for a in range(H):
        g = a // (H // G)
        p = masked_softmax((q[:, a] @ k[:, g].t()) * float(m["scale"]), seen)
        heads.append((p @ v[:, g]) * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ w[pre + "o"].t()


def query_temperature(positions, coef, every, dtype):
    return torch.as_tensor([1.0 + coef * math.log(((p + 1) // every) + 1) for p in positions], dtype=dtype)


def capped_attention(h, w, pre, m, eps, positions=None):
    """The left half of the "parallel" mixer."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = list(range(T)) if positions is None else positions
    q = weighted_norm((h @ w[pre + "q"].t()).view(T, H, D), w[pre + "q.norm"], eps)
    k = weighted_norm((h @ w[pre + "k"].t()).view(T, G, D), w[pre + "k.norm"], eps)
    v = (h @ w[pre + "v"].t()).view(T, G, V)
    q = q * query_temperature(positions, float(m["q_temp"]["coef"]), int(m["q_temp"]["every"]), h.dtype)[:, None, None]
    seen = seen_mask(positions)
    cap = float(m["softcap"])
    gate = head_gate(h, w[pre + "g"])
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = cap * torch.tanh((q[:, a] @ k[:, g].t()) * float(m["scale"]) / cap)
        heads.append((masked_softmax(s, seen) @ v[:, g]) * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ w[pre + "o"].t()


def shifted_mixes(h, mus):
    """h [T, width] -> one mix a name: h_p + (h_(p-1) - h_p) * mu, with zeros before position 0."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return {name: h + (before - h) * mu for name, mu in mus.items()}


def matrix_recurrence(r, k, v, decay, bonus):
    """One head. r, k, v, decay [T, D], bonus [D] -> outputs [T, D]; the state is [key, value]."""
    T, D = r.shape
    S = torch.zeros(D, D, dtype=r.dtype)
    out = []
    for p in range(T):
        kv = k[p][:, None] * v[p][None, :]
        out.append((S + bonus[:, None] * kv).t() @ r[p])
        S = decay[p][:, None] * S + kv
    return torch.stack(out)


def time_mixing(h, w, pre, m, eps):
    """The right half of the "parallel" mixer."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    mix = shifted_mixes(h, {s: w[pre + "mu." + s] for s in ("r", "k", "v", "g", "w")})
    r = (mix["r"] @ w[pre + "r"].t()).view(T, H, D)
    k = (mix["k"] @ w[pre + "k"].t()).view(T, H, D)
    v = (mix["v"] @ w[pre + "v"].t()).view(T, H, D)
    gate = silu(mix["g"] @ w[pre + "g"].t())
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[pre + "w1"].t()) @ w[pre + "w2"].t() + w[pre + "w0"])).view(T, H, D)
    heads = [unit_rms(matrix_recurrence(r[:, a], k[:, a], v[:, a], decay[:, a], w[pre + "u"][a]), eps) for a in range(H)]
    return (torch.cat(heads, dim=-1) * w[pre + "norm"] * gate) @ w[pre + "o"].t()


def side_by_side(h, w, pre, m, eps, positions=None):
    """The "parallel" mixer."""
    left = capped_attention(h, w, pre + "left.", m["left"], eps, positions)
    right = time_mixing(h, w, pre + "right.", m["right"], eps)
    return 0.5 * (weighted_norm(left, w[pre + "left.out"], eps) + weighted_norm(right, w[pre + "right.out"], eps))


MIXERS = {"attention": window_attention, "parallel": side_by_side}


# ------------------------------------------------------------------------------- feed-forward
def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].t()) * (h @ w[pre + "up"].t())) @ w[pre + "down"].t()


def routed_choice(h, w, pre, router):
    """(chosen experts [T, top], their weights [T, top])."""
    E, top = int(router["experts"]), int(router["top"])
    s = logistic(h @ w[pre + "router"].t())
    c = s + w[pre + "correction"]
    groups = router.get("groups")
    if groups is not None:
        n, keep = int(groups["count"]), int(groups["keep"])
        per = E // n
        runs = c.view(-1, n, per)
        run_score = torch.sort(runs, dim=-1, descending=True).values[..., :2].sum(-1)
        best = torch.sort(run_score, dim=-1, descending=True, stable=True).indices[:, :keep]
        allowed = torch.zeros(c.shape[0], n, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        c = torch.where(allowed[:, :, None].expand(-1, -1, per).reshape(-1, E), c, torch.full_like(c, float("-inf")))
    chosen = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top]
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def routed_feed_forward(h, w, pre, mlp):
    chosen, weight = routed_choice(h, w, pre, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, r in zip(chosen[t].tolist(), weight[t]):
            out[t] = out[t] + r * gated_expert(h[t], w, f"{pre}e{e}.")
    if mlp.get("shared") is not None:
        out = out + gated_expert(h, w, pre + "shared.") * logistic(h @ w[pre + "shared.sg"].t())
    return out


def feed_forward(h, w, pre, mlp):
    if mlp["kind"] == "moe":
        return routed_feed_forward(h, w, pre, mlp)
    raise ValueError(f"feed-forward kind {mlp['kind']!r}")


def layer(x, w, i, entry, eps, positions=None):
    if entry["type"] not in MIXERS:
        raise ValueError(f"layer type {entry['type']!r}")
    p = f"l{i}."
    out = x + MIXERS[entry["type"]](weighted_norm(x, w[p + "norm1"], eps), w, p + "mix.", entry["mixer"], eps, positions)
    if entry.get("mlp") is not None:
        out = out + feed_forward(weighted_norm(x, w[p + "norm2"], eps), w, p + "mlp.", entry["mlp"])
    return out


def run_order(n_layers, loop):
    """[(layer, pass number or None)]: the pass number stands at the first layer of each pass."""
    if not loop or int(loop["stop"]) <= int(loop["start"]):
        return [(i, None) for i in range(n_layers)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None) for i in range(start)]
    for n in range(times):
        order += [(i, n if i == start else None) for i in range(start, stop)]
    return order + [(i, None) for i in range(stop, n_layers)]


class PlainRaranex:
    def __init__(self, model_dir, dtype=torch.float64):
        model_dir = Path(model_dir)
        self.cfg = json.loads((model_dir / "config.json").read_text())
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
        self.dtype = dtype

    def streams(self, tokens):
        """The stream after every layer run, [layer runs, T, width]."""
        cfg, w = self.cfg, self.w
        eps = cfg["norm"]["eps"]
        e = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        x = e
        out = []
        for i, n in run_order(len(cfg["layers"]), cfg.get("loop")):
            if n is not None:
                x = torch.cat([x, e], dim=-1) @ w["loop.in"].t() + w["loop.step"][n]
            x = layer(x, w, i, cfg["layers"][i], eps)
            out.append(x)
        return torch.stack(out)

    def logits(self, tokens):
        x = self.streams(tokens)[-1]
        return (weighted_norm(x, self.w["final.norm"], self.cfg["norm"]["eps"]) @ self.w["head"].t()).float()

    def greedy(self, prompt, n):
        tokens = list(prompt)
        for _ in range(n):
            tokens.append(int(self.logits(tokens)[-1].argmax()))
        return tokens[len(prompt):]
