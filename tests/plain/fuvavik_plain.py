"""A plain, slow Fuvavik: whole sequences, no cache, one function per mechanism.

Shares no code with ``clockwork_amd``: it reads config.json and the safetensors file itself and
runs on the CPU in ``dtype`` (float64 by default, so that all of an error is the engine's).

The design in this file's notation. Tokens t at positions p = 0, 1, ...; the stream x_p has
``width`` elements.

* input: x_p = embedding.scale * embed[t_p] + pos[p].
* a layer ("parallel"): n = LN(x) with weight and bias; x <- x + s(rg1 n + c1) * M(n) + s(rg2 n + c2) * F(n),
  s the logistic function, M the mixer, F the feed-forward (absent where the layer has none).
* the mixer is two mixers on the same input, M(n) = (RMS(L(n)) * w_left + RMS(R(n)) * w_right) / 2.
* L: attention over a window of ``mask.size`` positions with grouped key/value heads. Queries and
  keys are RMS-normed as whole projections (all heads at once). The score of query i and key j of
  head a is scale * q_i.k_j - r1_a * log(1 + r2_a * (i - j)); the softmax denominator has one extra
  term exp(sink_a); the normalised weights of all heads are then mixed by the matrix ``talk``
  (new_a = sum_b talk[a, b] * old_b) and applied to the values of head a's key/value head.
* R: a linear recurrence with a decay per key channel. Per head S_p = diag(d_p) S_(p-1) + k_p v_p^T,
  o_p = S_p^T (q_p / sqrt(dim)), d_p = logistic(a2 (a1 n_p) + c)^(1/tau); o_p is RMS-normed per head,
  gated by silu(g n_p) and projected.
* F: down(gelu_tanh(gate n) * up n).
* output: LN(x) with the final weight and bias, times the embedding table, capped:
  cap * tanh(logits / cap).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


# ------------------------------------------------------------------------------- small pieces
def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def logistic(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * logistic(z)


def embed(tokens, table, positions_table, scale):
    ids = torch.as_tensor(tokens, dtype=torch.long)
    return table[ids] * scale + positions_table[: len(ids)]


# ------------------------------------------------------------------------------- the left mixer
def sink_window_attention(n, w, pre, m, eps):
    """n [T, width]; ``w`` the tensors, ``pre`` the prefix of this mixer's names, ``m`` its sizes."""
    T = n.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(n @ w[pre + "q"].t(), w[pre + "q.norm"], eps).view(T, H, D)
    k = rms_norm(n @ w[pre + "k"].t(), w[pre + "k.norm"], eps).view(T, G, D)
    v = (n @ w[pre + "v"].t()).view(T, G, V)
    r1, r2, sink, talk = w[pre + "r1"], w[pre + "r2"], w[pre + "sink"], w[pre + "talk"]
    window = int(m["mask"]["size"])
    out = torch.zeros(T, H, V, dtype=n.dtype)
    for i in range(T):
        lo = max(0, i - window + 1)
        dist = torch.arange(i - lo, -1, -1, dtype=n.dtype)                      # i - j for j = lo .. i
        probs = torch.zeros(H, i - lo + 1, dtype=n.dtype)
        for a in range(H):
            g = a // (H // G)
            s = (k[lo : i + 1, g] @ q[i, a]) * m["scale"] - r1[a] * torch.log(1.0 + r2[a] * dist)
            top = torch.maximum(s.max(), sink[a])
            e = torch.exp(s - top)
            probs[a] = e / (e.sum() + torch.exp(sink[a] - top))
        mixed = talk @ probs
        for a in range(H):
            out[i, a] = mixed[a] @ v[lo : i + 1, a // (H // G)]
    return out.reshape(T, H * V) @ w[pre + "o"].t()


# ------------------------------------------------------------------------------- the right mixer
def decayed_recurrence(n, w, pre, m, eps):
    T = n.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (n @ w[pre + "q"].t()).view(T, H, D) * D ** -0.5
    k = (n @ w[pre + "k"].t()).view(T, H, D)
    v = (n @ w[pre + "v"].t()).view(T, H, V)
    z = (n @ w[pre + "a1"].t()) @ w[pre + "a2"].t() + w[pre + "a2.b"]
    decay = (logistic(z) ** (1.0 / m["tau"])).view(T, H, D)
    state = torch.zeros(H, D, V, dtype=n.dtype)
    o = torch.zeros(T, H, V, dtype=n.dtype)
    for t in range(T):
        state = decay[t][:, :, None] * state + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", state, q[t])
    o = rms_norm(o, w[pre + "norm"], eps).reshape(T, H * V)
    return (o * silu(n @ w[pre + "g"].t())) @ w[pre + "o"].t()


def pair_mixer(n, w, pre, m, eps):
    left = rms_norm(sink_window_attention(n, w, pre + "left.", m["left"], eps), w[pre + "left.out"], eps)
    right = rms_norm(decayed_recurrence(n, w, pre + "right.", m["right"], eps), w[pre + "right.out"], eps)
    return 0.5 * (left + right)


# ------------------------------------------------------------------------------- the rest
def dense_feed_forward(n, w, pre):
    return (gelu_tanh(n @ w[pre + "gate"].t()) * (n @ w[pre + "up"].t())) @ w[pre + "down"].t()


def layer(x, w, i, entry, eps):
    if entry["type"] != "parallel":
        raise ValueError(f"layer type {entry['type']!r}")
    p = f"l{i}."
    n = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
    y = logistic(n @ w[p + "rg1"].t() + w[p + "rg1.b"]) * pair_mixer(n, w, p + "mix.", entry["mixer"], eps)
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "dense":
            raise ValueError(f"feed-forward kind {entry['mlp']['kind']!r}")
        y = y + logistic(n @ w[p + "rg2"].t() + w[p + "rg2.b"]) * dense_feed_forward(n, w, p + "mlp.")
    return x + y


def head(x, w, cfg):
    n = layer_norm(x, w["final.norm"], w["final.norm.b"], cfg["norm"]["eps"])
    logits = n @ w["embed"].t()
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(logits / cap)


class PlainFuvavik:
    def __init__(self, model_dir, dtype=torch.float64):
        model_dir = Path(model_dir)
        self.cfg = json.loads((model_dir / "config.json").read_text())
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
        self.dtype = dtype

    def streams(self, tokens):
        """The stream after the input and after every layer, [layers + 1, T, width]."""
        cfg, w = self.cfg, self.w
        x = embed(tokens, w["embed"], w["pos"], cfg["embedding"]["scale"])
        out = [x]
        for i, entry in enumerate(cfg["layers"]):
            x = layer(x, w, i, entry, cfg["norm"]["eps"])
            out.append(x)
        return torch.stack(out)

    def logits(self, tokens):
        return head(self.streams(tokens)[-1], self.w, self.cfg).float()

    def greedy(self, prompt, n):
        tokens = list(prompt)
        for _ in range(n):
            tokens.append(int(self.logits(tokens)[-1].argmax()))
        return tokens[len(prompt):]
