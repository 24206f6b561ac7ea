"""Windowed softmax attention with whole-projection query/key norms, a bias on the distance, a
sink in the softmax denominator and a mixing of the weights across heads (``SinkAttentionSpec``).

Steps: one fused q/k/v product; one kernel norms the query and key projections (float32
statistics) and writes keys and values to their pages, so every token of the step is in the
cache before any query reads it; the attention kernels read the pages through the block table:
one launch for the step's prompt portions (a workgroup takes a run of a request's tokens with all
heads), three small ones for its single tokens (a request's keys are shared among workgroups);
output product. Keys and values have
widths of their own, so the cache is two planes of a ``PagedRowsSpec``.
"""

from __future__ import annotations

import numpy as np
import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import PagedRowsSpec, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.specs import SinkAttentionSpec


def query_runs(ctx, run: int, skip_single: bool = False):
    """The step's work items for a kernel whose workgroups take up to ``run`` consecutive tokens
    of one request with all heads: (request, first token, tokens, 0) each, uploaded once a step
    and kept in ``ctx.plans``; ``skip_single``: requests of one token have a kernel of their own.
    Returns (device int32 array, number of items)."""
    key = ("query runs", run, skip_single)
    plan = ctx.plans.get(key)
    if plan is None:
        items = []
        for r, q_len in enumerate(ctx.h_q_lens):
            if skip_single and q_len == 1:
                continue
            tok0 = np.arange(0, q_len, run, dtype=np.int32)
            rows = np.zeros((tok0.size, 4), dtype=np.int32)
            rows[:, 0] = r
            rows[:, 1] = tok0
            rows[:, 2] = np.minimum(run, q_len - tok0)
            items.append(rows.reshape(-1))
        flat = np.concatenate(items) if items else np.zeros(0, dtype=np.int32)
        (device_items,) = ctx.upload([flat])
        plan = ctx.plans[key] = (device_items, len(flat) // 4)
    return plan


def longest_key_range(ctx, window=None, segment=None) -> int:
    """The most keys that a token of this step reads: its request's length, capped by a window;
    with segments, what the request's last token sees of its own segment (a single token) or at
    most a whole segment (a portion)."""
    longest = 0
    for q_len, ctx_len in zip(ctx.h_q_lens, ctx.h_ctx_lens):
        keys = ctx_len
        if window is not None:
            keys = min(keys, window)
        if segment is not None:
            keys = min(keys, segment) if q_len > 1 else (ctx_len - 1) % segment + 1
        longest = max(longest, keys)
    return longest


class SinkAttention(Part):
    graph_safe = True

    def __init__(self, spec: SinkAttentionSpec) -> None:
        self.spec = spec
        self.q_width = spec.num_heads * spec.key_dim
        self.k_width = spec.num_kv_heads * spec.key_dim
        self.v_width = spec.num_kv_heads * spec.value_dim

    def param_specs(self):
        s = self.spec
        specs = {
            "qkv_weight": ParamSpec((self.q_width + self.k_width + self.v_width, s.hidden_size)),
            "out_weight": ParamSpec((s.hidden_size, s.num_heads * s.value_dim)),
        }
        if s.qk_norm == "projection":
            specs["q_norm"] = ParamSpec((self.q_width,), precision="float32", init=("one_plus_uniform", 0.1))
            specs["k_norm"] = ParamSpec((self.k_width,), precision="float32", init=("one_plus_uniform", 0.1))
        if s.distance_bias:
            specs["r1"] = ParamSpec((s.num_heads,), precision="float32", init=("uniform", 0.0, 1.0))
            specs["r2"] = ParamSpec((s.num_heads,), precision="float32", init=("uniform", 0.0, 1.0))
        if s.sink:
            specs["sink"] = ParamSpec((s.num_heads,), precision="float32", init=("normal", 1.0))
        if s.talking_heads:
            specs["talk"] = ParamSpec((s.num_heads, s.num_heads), precision="float32", init=("eye_plus_normal", 0.2))
        return specs

    def cache_need(self):
        s = self.spec
        return PagedRowsSpec((("k", (s.num_kv_heads, s.key_dim)), ("v", (s.num_kv_heads, s.value_dim))), window=s.window)

    def kernel_libraries(self) -> list:
        return [("rowwise", None), ("sink_attention", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        self.qkv_weight = params["qkv_weight"]
        self.out_weight = params["out_weight"]
        self.q_norm, self.k_norm = params.get("q_norm"), params.get("k_norm")
        self.r1, self.r2 = params.get("r1"), params.get("r2")
        self.sink, self.talk = params.get("sink"), params.get("talk")
        self.dtype = dtype
        self.run = ops.sink_attention_max_run(s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim)
        # bfloat16 portions of the common head sizes run on the matrix cores; the kernel reads 16 bytes at a time
        self.mfma_ok = (ops.sink_prefill_mfma_supported(s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, dtype)
                        and (self.q_width + self.k_width + self.v_width) % 8 == 0)
        self.decode_ok = ops.sink_decode_supported(s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim)
        if self.run < 1:
            raise ValueError(
                f"attention with {s.num_heads} heads of {s.key_dim} / {s.value_dim} elements over {s.num_kv_heads} "
                "key/value heads is beyond the sink-attention kernel (heads * value_dim up to 8192, 150 KB of LDS)")

    def _plan(self, ctx):
        """(items of the kernel for portions, their number, keys a run and runs of the kernels for
        single tokens; 0 runs: the step has no single tokens, or they go with the portions)."""
        key = ("sink attention", self.spec.window, self.decode_ok, self.run, self.mfma_ok)
        plan = ctx.plans.get(key)
        if plan is None:
            singles = [c for q, c in zip(ctx.h_q_lens, ctx.h_ctx_lens) if q == 1] if self.decode_ok else []
            run_keys = n_runs = 0
            if singles:
                # the most keys a single token of this step sees, cut so that the workgroups about
                # fill the card: runs of 32 to 128 keys
                most = min(max(singles), self.spec.window or max(singles))
                run_keys = 128
                while run_keys > 32 and len(singles) * -(-most // run_keys) < ctx.num_compute_units:
                    run_keys //= 2
                n_runs = -(-most // run_keys)
            items, n_items = query_runs(ctx, 16 if self.mfma_ok else self.run, skip_single=bool(singles))
            plan = ctx.plans[key] = (items, n_items, run_keys, n_runs)
        return plan

    def prepare(self, ctx) -> None:
        self._plan(ctx)

    def shape_class(self, q_lens, ctx_lens):
        return "single tokens" if all(q == 1 for q in q_lens) else "portions"

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        if not cache.writes:
            raise NotImplementedError("this mixer writes its own keys and values: it cannot borrow another entry's cache")
        k_plane, v_plane = cache.planes["k"], cache.planes["v"]
        qkv = ops.linear(x, self.qkv_weight, policy=policy)
        ops.qk_rownorm_store(qkv, 0, self.q_width, self.q_width + self.k_width, self.q_width, self.k_width, self.v_width,
                             self.q_norm, self.k_norm, s.qk_norm_eps, ctx.slots[cache.group], k_plane, v_plane)
        out = torch.empty((x.shape[0], s.num_heads * s.value_dim), dtype=x.dtype, device=x.device)
        items, n_items, run_keys, n_runs = self._plan(ctx)
        options = (self.r1, self.r2, self.sink, self.talk, s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim,
                   cache.block_size, s.window or 0, s.scale)
        if n_items and self.mfma_ok:
            ops.sink_attention_prefill(qkv, qkv.shape[1], out, k_plane, v_plane, ctx.block_tables[cache.group], ctx.ctx_lens,
                                       ctx.cu_q, items, n_items, *options, compute_units=ctx.num_compute_units)
        elif n_items:
            ops.sink_attention(qkv, qkv.shape[1], out, k_plane, v_plane, ctx.block_tables[cache.group], ctx.ctx_lens,
                               ctx.cu_q, items, n_items, self.run, *options)
        if n_runs:
            ops.sink_attention_decode(qkv, qkv.shape[1], out, k_plane, v_plane, ctx.block_tables[cache.group], ctx.ctx_lens,
                                      ctx.cu_q, ctx.num_requests, run_keys, n_runs, *options)
        return ops.linear(out, self.out_weight, policy=policy)
