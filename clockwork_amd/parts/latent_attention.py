"""Attention over one cached latent a token (``LatentAttentionSpec``).

A token's cache row is its latent c (kv_rank elements, RMS-normed) followed by the rotated key
part that all heads share (rope_dim elements): nothing per head is kept. Head a's score against
key j is q_a . (uk_a c_j) + qr_a . kr_j = (uk_a^T q_a) . c_j + qr_a . kr_j, and its output
sum_j w_j (uv_a c_j) = uv_a (sum_j w_j c_j): the up-projections are applied to the queries and to
the attention's result instead of to every cached token, so the attention itself is one
key/value head of kv_rank + rope_dim elements whose values are the row's first kv_rank ones.

Steps: one product for everything that reads the mixer's input (low-rank query step, low-rank
key/value step, gate); one kernel norms the query step, norms the latent, rotates the shared key
part and writes the cache row; the query up-projection; per head uk_a^T q_a (a batched product)
beside the rotation of the queries' rope part; attention with the sink; per head uv_a; the
sigmoid gate; the output product.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import PagedRowsSpec, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.sink_attention import longest_key_range, query_runs
from clockwork_amd.parts.specs import LatentAttentionSpec


class LatentAttention(Part):
    graph_safe = True

    def __init__(self, spec: LatentAttentionSpec) -> None:
        self.spec = spec
        self.row = spec.kv_rank + spec.rope_dim            # elements of a cache row, and of an absorbed query
        self.q_head = spec.key_dim + spec.rope_dim
        self.o_width = spec.num_heads * spec.value_dim
        self.in_width = spec.q_rank + self.row + (self.o_width if spec.output_gate else 0)

    def param_specs(self):
        s = self.spec
        specs = {
            "in_weight": ParamSpec((self.in_width, s.hidden_size)),          # query step, key/value step, gate
            "q_norm": ParamSpec((s.q_rank,), precision="stored", init=("one_plus_uniform", 0.1)),
            "kv_norm": ParamSpec((s.kv_rank,), precision="stored", init=("one_plus_uniform", 0.1)),
            "q_up_weight": ParamSpec((s.num_heads * self.q_head, s.q_rank)),
            "k_up_weight": ParamSpec((s.num_heads * s.key_dim, s.kv_rank)),
            "v_up_weight": ParamSpec((s.num_heads * s.value_dim, s.kv_rank)),
            "out_weight": ParamSpec((s.hidden_size, self.o_width)),
        }
        if s.sink:
            specs["sink"] = ParamSpec((s.num_heads,), precision="float32", init=("normal", 1.0))
        return specs

    def cache_need(self):
        return PagedRowsSpec((("latent", (self.row,)),), window=self.spec.window)

    def kernel_libraries(self) -> list:
        return [("rowwise", None), ("rows_attention", None)]

    def bind(self, params, device, dtype) -> None:
        s = self.spec
        self.in_weight, self.q_up, self.out_weight = params["in_weight"], params["q_up_weight"], params["out_weight"]
        self.q_norm, self.kv_norm = params["q_norm"], params["kv_norm"]
        if self.kv_norm.dtype != self.q_norm.dtype:
            self.kv_norm = self.kv_norm.to(self.q_norm.dtype)
        # per head: the key up-projection transposed ([kv_rank, key_dim]: it is applied to queries) and
        # the value up-projection as it is ([value_dim, kv_rank]: it is applied to the attention's result)
        self.k_up_t = params["k_up_weight"].view(s.num_heads, s.key_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.v_up = params["v_up_weight"].view(s.num_heads, s.value_dim, s.kv_rank)
        self.sink = params.get("sink")
        half = s.rotary_dims // 2
        freq = torch.tensor([float(s.rope_base) ** (-2.0 * i / s.rotary_dims) for i in range(half)], dtype=torch.float64)
        self.freq = freq.to(torch.float32).to(device) if half else None
        self.dtype = dtype
        if not ops.rows_attention_supported(s.num_heads, 1, self.row, s.kv_rank, alias=True):
            raise ValueError(f"latent attention with rows of {self.row} elements is beyond the attention kernel for paged rows "
                             "(a latent of up to 512 elements, tiles of 150 KB of LDS)")
        # bfloat16 with the common latent sizes runs on the matrix cores
        self.mfma = ops.rows_mfma_supported(self.row, s.kv_rank, 1, dtype, alias=True)
        self.run = ops.ROWS_MFMA_TOKENS if self.mfma else ops.rows_attention_tokens_per_item(s.num_heads, 1, 1)

    def _plan(self, ctx):
        """(work items, their number, runs that every item's keys are cut into)."""
        s = self.spec
        key = ("latent attention", s.num_heads, self.row, s.kv_rank, s.window, self.mfma)
        plan = ctx.plans.get(key)
        if plan is None:
            items, n_items = query_runs(ctx, self.run)
            runs = 1
            if self.mfma:
                runs = ops.rows_mfma_key_runs(n_items, longest_key_range(ctx, s.window), s.num_heads, 1, self.row, s.kv_rank, 1,
                                              ctx.num_compute_units, alias=True)
            plan = ctx.plans[key] = (items, n_items, runs)
        return plan

    def prepare(self, ctx) -> None:
        self._plan(ctx)

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        policy = getattr(ctx, "products", None)
        if not cache.writes:
            raise NotImplementedError("this mixer writes its own latents: it cannot borrow another entry's cache")
        T, H = x.shape[0], s.num_heads
        plane = cache.planes["latent"]
        proj = ops.linear(x, self.in_weight, policy=policy)
        cq = torch.empty((T, s.q_rank), dtype=x.dtype, device=x.device)
        ops.latent_store(proj, 0, s.q_rank, s.q_rank, s.kv_rank, s.rope_dim, s.rotary_dims, self.q_norm, self.kv_norm, s.norm_eps,
                         ctx.positions, self.freq, ctx.slots[cache.group], cq, plane)
        q = ops.linear(cq, self.q_up, policy=policy)                                   # [T, H * (key_dim + rope_dim)]
        # absorbed queries, head-major [H, T, kv_rank + rope_dim]: uk_a^T q_a, then the rotated rope part
        qa = torch.empty((H, T, self.row), dtype=x.dtype, device=x.device)
        ops.heads_linear(q.view(T, H, self.q_head)[:, :, : s.key_dim].transpose(0, 1), self.k_up_t, qa[:, :, : s.kv_rank])
        if s.rope_dim:
            ops.rotate_part(q, (q.shape[1], self.q_head), s.key_dim, qa, (self.row, T * self.row), s.kv_rank, H, s.rope_dim,
                            s.rotary_dims, ctx.positions, self.freq)
        ol = torch.empty((H, T, s.kv_rank), dtype=x.dtype, device=x.device)
        items, n_items, runs = self._plan(ctx)
        kind, size = ("window", s.window) if s.window is not None else ("causal", 0)
        ops.rows_attention(qa, (self.row, T * self.row), ol, (s.kv_rank, T * s.kv_rank), plane, None,
                           ctx.block_tables[cache.group], ctx.ctx_lens, ctx.cu_q, items, n_items, H, 1, self.row, s.kv_rank,
                           cache.block_size, s.scale, mask=kind, mask_size=size, sink=self.sink, mfma=self.mfma, key_runs=runs)
        out = torch.empty((T, self.o_width), dtype=x.dtype, device=x.device)
        ops.heads_linear(ol, self.v_up, out.view(T, H, s.value_dim).transpose(0, 1))
        if s.output_gate:
            ops.sigmoid_mul_(out, proj, s.q_rank + self.row)
        return ops.linear(out, self.out_weight, policy=policy)
