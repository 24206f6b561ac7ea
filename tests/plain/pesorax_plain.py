"""A plain, slow Pesorax: whole sequences, no cache, one function per mechanism.

Shares no code with ``clockwork_amd``: it reads config.json and the safetensors file itself and
runs on the CPU in ``dtype`` (float64 by default, so that all of an error is the engine's).

The design in this file's notation. Tokens t at positions p = 0, 1, ...; the stream x_p has
``width`` elements; m = ``residual_mult``.

* input: e_p = embed[t_p]; x_p = e_p.
* order: the layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row with the same
  weights, then the others; before every pass but the first, x <- x + e.
* a layer: x <- x + m * M(N1(x)); x <- x + m * F(N2(x)) (F absent where the layer has none), with
  N(x) = tanh(alpha * x) * w + b (a scalar alpha, no statistics).
* M "attention": H query heads over G key/value heads, each head with TWO score maps. Queries
  [H, 2, dim] and keys [G, 2, dim] come from biased projections, values [G, vdim] too. Map c of
  head a is softmax_j(scale * q[a, c] . k_j[g, c]) over the keys j <= i of i's block of
  ``mask.size`` positions (blocks counted from position 0), applied to the values of g. With
  lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff the head's output is o = A_1 - lam * A_2, divided
  by its root mean square over vdim and multiplied by (1 - diff); heads are concatenated and projected.
* M "latent_attention": queries through a low-rank step, cq = RMS(dq n) * w_dq, q = uq cq, laid out
  [H, dim + rot_dim]; dkv n gives kv_rank elements, RMS-normed with a weight into the latent c, and
  rot_dim more, one rotated key part for all heads. Keys of head a: [uk_a c, rotated part], values
  uv_a c. The rot_dim parts of q and k are rotated by position (pairs (i, i + rot_dim / 2), angle
  p * base^(-2 i / rot_dim)). Causal softmax of scale * q . k whose denominator has one more term
  exp(sink_a); the concatenated heads are multiplied by logistic(g n) and projected.
* F: down(gelu(up n)), the erf gelu.
* output: N(x) with the final norm's tensors, times ``head``.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


# ------------------------------------------------------------------------------- small pieces
def dynamic_tanh(x, weight, bias, alpha):
    return torch.tanh(alpha * x) * weight + bias


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def logistic(z):
    return 1.0 / (1.0 + torch.exp(-z))


def rotate_half_pairs(v, positions, base, dims):
    """v [T, ..., dims]: element i is paired with element i + dims / 2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=v.dtype)
    angle = torch.as_tensor(positions, dtype=v.dtype)[:, None] * freq[None, :]
    while angle.dim() < v.dim():
        angle = angle.unsqueeze(1)
    cos, sin = torch.cos(angle), torch.sin(angle)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------- the two mixers
def two_map_block_attention(n, w, pre, m, eps):
    """n [T, width]; ``w`` the tensors, ``pre`` the prefix of this mixer's names, ``m`` its sizes."""
    T = n.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    block, diff, scale = int(m["mask"]["size"]), float(m["diff"]), float(m["scale"])
    q = (n @ w[pre + "q"].t() + w[pre + "q.b"]).view(T, H, 2, D)
    k = (n @ w[pre + "k"].t() + w[pre + "k.b"]).view(T, G, 2, D)
    v = (n @ w[pre + "v"].t() + w[pre + "v.b"]).view(T, G, V)
    lam = torch.exp((w[pre + "lq1"] * w[pre + "lk1"]).sum()) - torch.exp((w[pre + "lq2"] * w[pre + "lk2"]).sum()) + diff
    out = torch.zeros(T, H, V, dtype=n.dtype)
    for i in range(T):
        lo = (i // block) * block
        for a in range(H):
            g = a // (H // G)
            maps = []
            for c in range(2):
                s = (k[lo : i + 1, g, c] @ q[i, a, c]) * scale
                maps.append(torch.softmax(s, dim=0) @ v[lo : i + 1, g])
            o = maps[0] - lam * maps[1]
            out[i, a] = rms(o, eps) * (1.0 - diff)
    return out.reshape(T, H * V) @ w[pre + "o"].t()


def latent_attention(n, w, pre, m, eps, positions=None):
    T = n.shape[0]
    H, D, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims, scale = float(m["rot"]["base"]), int(m["rot"]["dims"]), float(m["scale"])
    positions = list(range(T)) if positions is None else positions
    cq = rms(n @ w[pre + "dq"].t(), eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].t()).view(T, H, D + R)
    down = n @ w[pre + "dkv"].t()
    c = rms(down[:, :rank], eps) * w[pre + "dkv.norm"]
    k_rot = rotate_half_pairs(down[:, rank:], positions, base, dims)                   # [T, R], shared by the heads
    q_rot = rotate_half_pairs(q[..., D:], positions, base, dims)                       # [T, H, R]
    k_plain = (c @ w[pre + "uk"].t()).view(T, H, D)
    v = (c @ w[pre + "uv"].t()).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=n.dtype)
    for i in range(T):
        for a in range(H):
            s = (k_plain[: i + 1, a] @ q[i, a, :D] + k_rot[: i + 1] @ q_rot[i, a]) * scale
            top = torch.maximum(s.max(), w[pre + "sink"][a])
            e = torch.exp(s - top)
            out[i, a] = (e @ v[: i + 1, a]) / (e.sum() + torch.exp(w[pre + "sink"][a] - top))
    gate = logistic(n @ w[pre + "g"].t())
    return (out.reshape(T, H * V) * gate) @ w[pre + "o"].t()


MIXERS = {"attention": two_map_block_attention, "latent_attention": latent_attention}


def dense_feed_forward(n, w, pre):
    return gelu_erf(n @ w[pre + "up"].t()) @ w[pre + "down"].t()


def norm_of(x, w, name):
    return dynamic_tanh(x, w[name], w[name + ".b"], w[name + ".alpha"])


def layer(x, w, i, entry, eps, mult):
    if entry["type"] not in MIXERS:
        raise ValueError(f"layer type {entry['type']!r}")
    p = f"l{i}."
    x = x + mult * MIXERS[entry["type"]](norm_of(x, w, p + "norm1"), w, p + "mix.", entry["mixer"], eps)
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "dense":
            raise ValueError(f"feed-forward kind {entry['mlp']['kind']!r}")
        x = x + mult * dense_feed_forward(norm_of(x, w, p + "norm2"), w, p + "mlp.")
    return x


def layer_order(cfg):
    """(layer index, does a new pass begin here after the first) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for rep in range(times if stop > start else 0):
        order += [(i, rep > 0 and i == start) for i in range(start, stop)]
    order += [(i, False) for i in range(max(stop, start), n)]
    return order


class PlainPesorax:
    def __init__(self, model_dir, dtype=torch.float64):
        model_dir = Path(model_dir)
        self.cfg = json.loads((model_dir / "config.json").read_text())
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
        self.dtype = dtype

    def streams(self, tokens):
        """The stream after every layer run, [runs, T, width]."""
        cfg, w = self.cfg, self.w
        e = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        x = e
        out = []
        for i, new_pass in layer_order(cfg):
            if new_pass:
                x = x + e
            x = layer(x, w, i, cfg["layers"][i], cfg["norm"]["eps"], cfg["residual_mult"])
            out.append(x)
        return torch.stack(out)

    def logits(self, tokens):
        x = self.streams(tokens)[-1]
        return (norm_of(x, self.w, "final.norm") @ self.w["head"].t()).float()

    def greedy(self, prompt, n):
        tokens = list(prompt)
        for _ in range(n):
            tokens.append(int(self.logits(tokens)[-1].argmax()))
        return tokens[len(prompt):]
