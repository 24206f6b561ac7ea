"""Linear attention with a matrix state per head and a decay per key channel
(``DecayedLinearAttentionSpec``): S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.

One product makes q, k, v, the output gate and the low-rank input of the decay for every token
of the step; one kernel walks each request's tokens in order from the request's state slot
(float32 [heads, key_dim, value_dim], zero at a request's start), makes the decays
(sigmoid(z)^(1/tau) through log-sigmoid, float32), norms and gates the outputs; output product.
A step with a portion of more than 64 tokens cuts every request's tokens into segments of 32 that
are walked side by side: each from a zero state, then the start states are carried from segment
to segment, then each segment is walked again for its outputs (the same sums, other parentheses).
The state is all the mixer keeps: a ``StateSpec``.
"""

from __future__ import annotations

import numpy as np
import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec, StateSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.specs import DecayedLinearAttentionSpec


# tokens of a segment, and the longest portion that is still walked token by token in one piece
SEGMENT_TOKENS = 32
SEGMENT_MIN_TOKENS = 64


class DecayedLinearAttention(Part):
    graph_safe = True

    def __init__(self, spec: DecayedLinearAttentionSpec) -> None:
        self.spec = spec
        qk, v = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        # columns of the input product: q, k, v, gate, decay input
        self.q_off, self.k_off, self.v_off, self.g_off, self.u_off = 0, qk, 2 * qk, 2 * qk + v, 2 * qk + 2 * v
        self.in_width = 2 * qk + 2 * v + spec.decay_rank

    def param_specs(self):
        s = self.spec
        return {
            "in_weight": ParamSpec((self.in_width, s.hidden_size)),
            "decay_weight": ParamSpec((s.num_heads * s.key_dim, s.decay_rank), init=("normal", 0.5)),
            "decay_bias": ParamSpec((s.num_heads * s.key_dim,), precision="float32", init=("normal", 1.0)),
            "norm_weight": ParamSpec((s.value_dim,), precision="float32", init=("one_plus_uniform", 0.1)),
            "out_weight": ParamSpec((s.hidden_size, s.num_heads * s.value_dim)),
        }

    def cache_need(self):
        s = self.spec
        return StateSpec((s.num_heads, s.key_dim, s.value_dim), "float32")

    def kernel_libraries(self) -> list:
        return [("linear_recurrence", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        if not ops.linear_recurrence_supported(s.key_dim, s.value_dim):
            raise ValueError(f"a state of {s.key_dim} x {s.value_dim} a head is beyond the recurrence kernel "
                             "(value_dim up to 256, key_dim up to 128 rows a thread)")
        self.segments_ok = ops.linear_recurrence_segments_supported(s.key_dim, s.value_dim)
        self.in_weight = params["in_weight"]
        self.decay_weight = params["decay_weight"]
        self.decay_bias = params["decay_bias"]
        self.norm_weight = params["norm_weight"]
        self.out_weight = params["out_weight"]

    def _segments(self, ctx):
        """The step's segments when it holds a long portion and the state fits the kernel that
        walks segments side by side, else None (every request is then walked token by token by
        one workgroup a head). Made once a step, kept in ``ctx.plans``."""
        if max(ctx.h_q_lens, default=0) <= SEGMENT_MIN_TOKENS or not self.segments_ok:
            return None
        key = ("recurrence segments", SEGMENT_TOKENS)
        plan = ctx.plans.get(key)
        if plan is None:
            items, first = [], [0]
            for r, q_len in enumerate(ctx.h_q_lens):
                tok0 = np.arange(0, q_len, SEGMENT_TOKENS, dtype=np.int32)
                rows = np.zeros((tok0.size, 4), dtype=np.int32)
                rows[:, 0] = r
                rows[:, 1] = tok0
                rows[:, 2] = np.minimum(SEGMENT_TOKENS, q_len - tok0)
                rows[:, 3] = np.arange(tok0.size)
                items.append(rows.reshape(-1))
                first.append(first[-1] + tok0.size)
            device_items, device_first = ctx.upload([np.concatenate(items), first])
            plan = ctx.plans[key] = (device_items, first[-1], device_first)
        return plan

    def prepare(self, ctx) -> None:
        self._segments(ctx)

    def shape_class(self, q_lens, ctx_lens):
        return "segments" if max(q_lens, default=0) > SEGMENT_MIN_TOKENS and self.segments_ok else "token by token"

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        proj = ops.linear(x, self.in_weight, policy=policy)
        common = (proj, self.q_off, self.k_off, self.v_off, self.g_off, self.u_off, self.decay_weight, self.decay_bias,
                  self.norm_weight, cache.state, ctx.state_slots, ctx.cu_q)
        sizes = (ctx.num_requests, s.num_heads, s.key_dim, s.value_dim, s.key_dim ** -0.5, s.tau, s.norm_eps)
        plan = self._segments(ctx)
        if plan is not None:
            items, n_segments, first = plan
            out = ops.linear_recurrence_segments(*common, items, n_segments, SEGMENT_TOKENS, first, *sizes)
        else:
            out = ops.linear_recurrence(*common, *sizes)
        return ops.linear(out, self.out_weight, policy=policy)
