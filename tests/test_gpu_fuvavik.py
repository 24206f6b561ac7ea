"""Fuvavik on the GPU against the plain implementation (tests/plain/fuvavik_plain.py): each new
kernel and part alone, then whole models of three small configurations replayed whole, as prefill
then single tokens, in portions down to two tokens and as mixed batches on tight page pools, in
both dtypes; windows' edges and far keys with weights made so that one key decides the output;
long decoding; forks; greedy generation through the engine's entry point, the command line and
the trace program."""

import json
import math
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from clockwork_amd.registry import build_part
from clockwork_amd.parts.specs import (BranchGateSpec, DecayedLinearAttentionSpec, GatedMLPSpec, LayerNormSpec,
                                       LinearHeadSpec, PairMixerSpec, PositionTableEmbeddingSpec, SinkAttentionSpec)
from tests import replay
from tests.configs import FUVAVIK_CONFIGS
from tests.plain import fuvavik_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPO = Path(__file__).resolve().parents[1]
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {torch.float32: dict(rtol=2e-5, atol=2e-5), torch.bfloat16: dict(rtol=4e-2, atol=4e-2)}


def close(got, want, dtype):
    """float32: element by element. bfloat16, whose every activation is rounded to 8 bits: the
    largest error against the values' own scale (an element that is small by cancellation carries
    the rounding of the large terms it came from)."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)
        return
    assert not torch.isnan(got).any()
    scale = float(want.square().mean().sqrt())
    rms, worst = float((got - want).square().mean().sqrt()), float((got - want).abs().max())
    assert rms < 2e-2 * scale and worst < 1e-1 * scale, (
        f"rms error {rms:.3e}, largest error {worst:.3e} against a scale of {scale:.3e}")


def draw(spec, gen):
    kind = spec.init[0]
    if kind == "normal":
        return torch.randn(spec.shape, generator=gen) * spec.init[1]
    if kind == "one_plus_uniform":
        return 1 + (torch.rand(spec.shape, generator=gen) * 2 - 1) * spec.init[1]
    if kind == "uniform":
        return spec.init[1] + torch.rand(spec.shape, generator=gen) * (spec.init[2] - spec.init[1])
    if kind == "eye_plus_normal":
        return torch.eye(*spec.shape) + torch.randn(spec.shape, generator=gen) * spec.init[1]
    return torch.zeros(spec.shape)


def bind(part, dtype, seed=0, matrix_std=None, change=None):
    """Random parameters for ``part`` (bfloat16-representable values, so both dtypes see the same
    model); returns them as float64 CPU tensors by the part's own names."""
    gen = torch.Generator().manual_seed(seed)
    values = {}
    for name, spec in part.param_specs().items():
        t = draw(spec, gen)
        if matrix_std is not None and spec.init[0] == "normal" and len(spec.shape) == 2:
            t = t / spec.init[1] * matrix_std
        values[name] = t.to(torch.bfloat16).float()
    if change is not None:
        change(values)
    params = {}
    for name, spec in part.param_specs().items():
        params[name] = values[name].to(torch.float32 if spec.precision == "float32" else dtype).to(DEV)
    part.bind(params, torch.device(DEV), dtype)
    return {k: v.double() for k, v in values.items()}


# ------------------------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [100, 257, 1024])
def test_layernorm_alone_and_with_gated_branches(dtype, width):
    from clockwork_amd import ops

    part = build_part(LayerNormSpec(size=width, eps=3e-5))
    w = bind(part, dtype)
    T = 7
    gen = torch.Generator().manual_seed(1)
    resid = (torch.randn(T, width, generator=gen) * 3 + 0.7).to(DEV)
    want = plain.layer_norm(resid.double().cpu(), w["weight"], w["bias"], 3e-5)
    before = resid.clone()
    close(part.forward(resid, None).double().cpu(), want, dtype)
    assert torch.equal(resid, before)
    # some rows only: the residual stays as it is
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEV)
    close(part.forward(resid, None, rows=rows).double().cpu(), want[[5, 0, 3]], dtype)
    # two gated branches are added first, in float32
    a, b = (torch.randn(T, width, generator=gen).to(dtype).to(DEV) for _ in range(2))
    z = (torch.randn(T, 2 * width, generator=gen) * 2).to(dtype).to(DEV)
    zb = torch.randn(2 * width, generator=gen).to(DEV)
    g = plain.logistic(z.double().cpu() + zb.double().cpu())
    total = before.double().cpu() + g[:, :width] * a.double().cpu() + g[:, width:] * b.double().cpu()
    out = part.forward(resid, ops.GatedBranches(z, zb, a, b))
    torch.testing.assert_close(resid.double().cpu(), total, rtol=1e-6, atol=1e-6)
    close(out.double().cpu(), plain.layer_norm(total, w["weight"], w["bias"], 3e-5), dtype)
    # the same through the adding kernel, one branch, no gates
    resid2 = before.clone()
    ops.gated_residual_add(resid2, ops.GatedBranches(None, None, a))
    torch.testing.assert_close(resid2.double().cpu(), before.double().cpu() + a.double().cpu(), rtol=1e-6, atol=1e-6)
    resid3 = before.clone()
    ops.gated_residual_add(resid3, ops.GatedBranches(z[:, :width].contiguous(), zb[:width].contiguous(), a))
    torch.testing.assert_close(resid3.double().cpu(), before.double().cpu() + g[:, :width] * a.double().cpu(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_scale_and_positions(dtype):
    part = build_part(PositionTableEmbeddingSpec(vocab_size=50, hidden_size=36, scale=2.5, max_positions=40))
    w = bind(part, dtype, matrix_std=1.0)

    class Ctx:
        num_tokens = 6
        token_ids = torch.tensor([3, 49, 0, 7, 7, 20], dtype=torch.int32, device=DEV)
        positions = torch.tensor([0, 1, 39, 5, 6, 7], dtype=torch.int32, device=DEV)

    got = part.forward(Ctx)
    want = w["weight"][Ctx.token_ids.long().cpu()] * 2.5 + w["positions"][Ctx.positions.long().cpu()]
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double().cpu(), want, rtol=1e-6, atol=1e-6)
    assert part.table() is part.weight  # a tied head multiplies with the table itself


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_feed_forward_and_the_capped_head(dtype):
    ffn = build_part(GatedMLPSpec(hidden_size=72, intermediate_size=50, activation="gelu_tanh"))
    w = bind(ffn, dtype, matrix_std=0.3)
    x = (torch.randn(9, 72, generator=torch.Generator().manual_seed(2)) * 2).to(dtype)
    names = {"gate": w["gate_up_weight"][:50], "up": w["gate_up_weight"][50:], "down": w["down_weight"]}
    want = plain.dense_feed_forward(x.double(), names, "")
    close(ffn.forward(x.to(DEV), None).double().cpu(), want, dtype)
    # gelu_tanh itself at values where its two halves differ most
    z = torch.linspace(-6, 6, 25, dtype=torch.float64)
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12
    from clockwork_amd import ops

    gu = torch.stack([torch.cat([z, torch.ones(25, dtype=torch.float64)])]).float().to(DEV)
    out = ops.gelu_tanh_mul(gu, torch.empty(1, 25, device=DEV))
    torch.testing.assert_close(out[0].double().cpu(), plain.gelu_tanh(z), rtol=1e-6, atol=1e-6)
    # the cap: logits far beyond it saturate
    head = build_part(LinearHeadSpec(vocab_size=40, hidden_size=72, tied=False, softcap=3.0))
    hw = bind(head, dtype, matrix_std=0.5)
    rows = (torch.randn(4, 72, generator=torch.Generator().manual_seed(3)) * 2).to(dtype)
    want = 3.0 * torch.tanh(rows.double() @ hw["weight"].t() / 3.0)
    got = head.forward(rows.to(DEV), None)
    assert got.dtype == torch.float32 and float(got.abs().max()) <= 3.0 and float(want.abs().max()) > 2.9
    close(got.double().cpu(), want, dtype)


def _step_through(part, need, x, cuts, dtype, block_size=8, num_blocks=16, release=True, compute_units=None):
    """Run ``x`` [T, hidden] through a mixer in steps of ``cuts`` tokens with a cache manager and
    NaN-poisoned pools of its own; returns the outputs, concatenated."""
    from clockwork_amd.cache import CacheManager, plan_groups
    from clockwork_amd.cache.pools import CachePools
    from clockwork_amd.engine.batch import StepEntry, build_context

    groups = plan_groups([need])
    manager = CacheManager(groups, block_size, num_blocks, max_num_seqs=4)
    pools = CachePools(groups, block_size, num_blocks, 4, dtype, torch.device(DEV), fill=float("nan"))
    cache = pools.entry_cache(0)
    got, at = [], 0
    for n in cuts:
        if at == 0:
            manager.admit("s", n)
        manager.extend("s", at, at + n)
        ctx = build_context([StepEntry("s", at, [0] * n)], manager, torch.device(DEV), 10)
        if compute_units is not None:
            ctx.num_compute_units = compute_units  # what the parts size their launches by
        if pools.state:
            pools.set_fresh_states(ctx.state_slots, ctx.starts, ctx.num_requests)
        got.append(part.forward(x[at : at + n].to(dtype).to(DEV), ctx, cache))
        at += n
        if release:
            manager.release_behind_window("s", at)
    return torch.cat(got).double().cpu()


def _left_names(w, spec):
    q, k = spec.num_heads * spec.key_dim, spec.num_kv_heads * spec.key_dim
    return {"q": w["qkv_weight"][:q], "k": w["qkv_weight"][q : q + k], "v": w["qkv_weight"][q + k :], "q.norm": w["q_norm"],
            "k.norm": w["k_norm"], "r1": w["r1"], "r2": w["r2"], "sink": w["sink"], "talk": w["talk"], "o": w["out_weight"]}


def _left_sizes(spec):
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim,
            "scale": spec.scale, "mask": {"size": spec.window}}


LEFT_SHAPES = [
    # heads, kv_heads, dim, vdim, window, hidden
    (4, 2, 24, 16, 9, 64),
    (6, 6, 16, 16, 33, 72),
    (3, 1, 40, 24, 300, 50),
    (1, 1, 8, 72, 1, 40),
    (16, 4, 64, 32, 20, 96),
    (5, 5, 20, 12, 11, 40),   # rows that are no multiple of 16 bytes: the kernels' element-by-element loads
    # the sizes that the matrix-core kernel for bfloat16 portions takes
    (12, 2, 128, 128, 40, 64),
    (6, 3, 64, 128, 23, 48),
    (16, 16, 128, 64, 300, 32),
    (1, 1, 64, 64, 7, 40),
    (14, 2, 64, 64, 50, 56),    # heads that the four waves do not share evenly
    (6, 2, 128, 64, 19, 48),
    (8, 4, 64, 64, 30, 64),     # more than two key/value heads: the keys are walked twice
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", LEFT_SHAPES)
def test_sink_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, vdim, window, hidden = shape
    spec = SinkAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim,
                             scale=0.21, window=window, qk_norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, dtype, seed=shape[0], matrix_std=0.15)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.sink_window_attention(x.double(), _left_names(w, spec), "", _left_sizes(spec), 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 32], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)
    if part.mfma_ok:
        # the matrix-core kernel against the plain-arithmetic one on the very same bfloat16 queries,
        # keys and values: they differ by the order of their sums and the rounding of the output
        # alone, a tenth of what separates either from the float64 result
        assert dtype == torch.bfloat16
        fast = _step_through(part, part.cache_need(), x, [T], dtype)
        # on a card of one compute unit a run's value columns are not shared between two workgroups
        whole = _step_through(part, part.cache_need(), x, [T], dtype, compute_units=1)
        assert float((fast - whole).abs().max()) < 1e-6 * max(1.0, float(fast.abs().max()))
        part.mfma_ok = False
        slow = _step_through(part, part.cache_need(), x, [T], dtype)
        scale = float(want.square().mean().sqrt())
        assert float((fast - slow).abs().max()) < 1.5e-2 * scale and float((fast - slow).square().mean().sqrt()) < 3e-3 * scale


def test_the_matrix_core_kernel_is_the_one_that_runs_for_bfloat16_portions():
    spec = SinkAttentionSpec(hidden_size=64, num_heads=12, num_kv_heads=2, key_dim=128, value_dim=128, scale=0.1, window=40)
    for dtype, expected in ((torch.bfloat16, True), (torch.float32, False)):
        part = build_part(spec)
        bind(part, dtype)
        assert part.mfma_ok is expected and part.decode_ok
    odd = build_part(SinkAttentionSpec(hidden_size=64, num_heads=4, num_kv_heads=2, key_dim=24, value_dim=16, scale=0.1, window=9))
    bind(odd, torch.bfloat16)
    assert not odd.mfma_ok and odd.run >= 1


def test_sink_attention_options_each_matter():
    """The sink, the distance bias and the mixing across heads each change the result by much more
    than the tolerance, so the comparison above would not pass without any of them."""
    spec = SinkAttentionSpec(hidden_size=64, num_heads=4, num_kv_heads=2, key_dim=24, value_dim=16, scale=0.21, window=9,
                             qk_norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=7, matrix_std=0.15)
    x = torch.randn(30, 64, generator=torch.Generator().manual_seed(5))
    got = _step_through(part, part.cache_need(), x, [30], torch.float32)
    base = _left_names(w, spec)
    for name, value in (("sink", base["sink"] - 30.0), ("r1", torch.zeros(4, dtype=torch.float64)),
                        ("talk", torch.eye(4, dtype=torch.float64))):
        other = plain.sink_window_attention(x.double(), dict(base, **{name: value}), "", _left_sizes(spec), 1e-5)
        assert float((other - got).abs().max()) > 1e-2, name


@pytest.mark.parametrize("window", [5, 16, 17, 40])
@pytest.mark.parametrize("cuts", ["whole", "portions", "single"])
def test_one_loud_key_just_inside_and_just_outside_the_window(window, cuts):
    """One early token gets a key that every later query scores far above all others, and a value
    of its own. While it is inside the window it decides the output; from the first position
    whose window has passed it, it must be gone. Pages of 4 and 8 tokens put the edge at page
    borders and inside pages; pages behind the window are given back and used again."""
    hidden, heads, dim, vdim = 32, 2, 16, 8
    spec = SinkAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=1, key_dim=dim, value_dim=vdim, scale=1.0,
                             window=window, qk_norm_eps=1e-6, distance_bias=False, talking_heads=False)
    part = build_part(spec)

    def change(v):
        # input element 0 marks the loud token: it alone sets key channel 0 and value channel 0;
        # element 1, which every token carries, sets query channel 0 of both heads
        v["qkv_weight"].zero_()
        v["qkv_weight"][0, 1] = 1.0           # query head 0, channel 0
        v["qkv_weight"][dim, 1] = 1.0         # query head 1, channel 0
        v["qkv_weight"][2 * dim, 0] = 1.0     # key channel 0
        v["qkv_weight"][2 * dim + 1, 1] = 0.05  # a small key for every token, so no norm divides by zero
        v["qkv_weight"][3 * dim, 0] = 1.0     # value channel 0
        v["q_norm"].fill_(6.0)
        v["k_norm"].fill_(6.0)
        v["sink"].fill_(-2.0)
        v["out_weight"].zero_()
        v["out_weight"][0, 0] = 1.0
        v["out_weight"][1, vdim] = 1.0

    w = bind(part, torch.float32, change=change)
    T, loud = 70, 3
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    want = plain.sink_window_attention(x.double(), _left_names({**w, "r1": torch.zeros(2, dtype=torch.float64), "r2": torch.zeros(2, dtype=torch.float64), "talk": torch.eye(2, dtype=torch.float64)}, spec), "", _left_sizes(spec), 1e-6)
    # the plain result itself shows the edge: the loud value fills the output while seen, then nothing is left
    assert float(want[loud + window - 1, 0]) > 0.5 and abs(float(want[loud + window, 0])) < 1e-6
    for block_size in (4, 8):
        steps = {"whole": [T], "portions": [2, 7, 3, 16, 5, 2, 31, 4], "single": [loud + 2] + [1] * (T - loud - 2)}[cuts]
        got = _step_through(part, part.cache_need(), x, steps, torch.float32, block_size=block_size, num_blocks=24)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_decides_the_output(dtype):
    """The same loud key behind a window of 400: it is one of up to 400 keys that a query sees, 399
    positions back at the last one that sees it, and gone at the next. In bfloat16 the portions
    run on the matrix cores and the single tokens share their keys among several workgroups."""
    hidden, heads, dim, vdim, window = 32, 2, 64, 64, 400
    spec = SinkAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=1, key_dim=dim, value_dim=vdim, scale=1.0,
                             window=window, qk_norm_eps=1e-6, distance_bias=False, talking_heads=False)
    part = build_part(spec)

    def change(v):
        v["qkv_weight"].zero_()
        v["qkv_weight"][0, 1] = 1.0
        v["qkv_weight"][dim, 1] = 1.0
        v["qkv_weight"][2 * dim, 0] = 1.0
        v["qkv_weight"][2 * dim + 1, 1] = 0.05
        v["qkv_weight"][3 * dim, 0] = 1.0
        v["q_norm"].fill_(6.0)
        v["k_norm"].fill_(6.0)
        v["sink"].fill_(-2.0)
        v["out_weight"].zero_()
        v["out_weight"][0, 0] = 1.0
        v["out_weight"][1, vdim] = 1.0

    w = bind(part, dtype, change=change)
    assert part.mfma_ok == (dtype == torch.bfloat16)
    T, loud = 450, 7
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    names = _left_names({**w, "r1": torch.zeros(2, dtype=torch.float64), "r2": torch.zeros(2, dtype=torch.float64),
                         "talk": torch.eye(2, dtype=torch.float64)}, spec)
    want = plain.sink_window_attention(x.double(), names, "", _left_sizes(spec), 1e-6)
    assert float(want[loud + window - 1, 0]) > 3.9 and abs(float(want[loud + window, 0])) < 1e-6
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    for steps in ([T], [2, 300, 7, 64, 29, 33, 15], [390] + [1] * 60):
        got = _step_through(part, part.cache_need(), x, steps, dtype, block_size=16, num_blocks=40)
        torch.testing.assert_close(got, want, **tol)


def _right_names(w, spec):
    qk, v = spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
    iw = w["in_weight"]
    return {"q": iw[:qk], "k": iw[qk : 2 * qk], "v": iw[2 * qk : 2 * qk + v], "g": iw[2 * qk + v : 2 * qk + 2 * v],
            "a1": iw[2 * qk + 2 * v :], "a2": w["decay_weight"], "a2.b": w["decay_bias"], "norm": w["norm_weight"],
            "o": w["out_weight"]}


RIGHT_SHAPES = [
    # heads, dim, vdim, rank, tau, hidden
    (2, 12, 20, 5, 4.0, 64),
    (3, 20, 8, 3, 16.0, 72),
    (1, 64, 64, 16, 1.0, 50),
    (4, 6, 10, 2, 2.5, 40),
    (1, 16, 4, 1, 8.0, 48),
    (2, 128, 256, 8, 32.0, 64),
    (1, 100, 3, 4, 2.0, 32),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", RIGHT_SHAPES)
def test_decayed_linear_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, dim, vdim, rank, tau, hidden = shape
    spec = DecayedLinearAttentionSpec(hidden_size=hidden, num_heads=heads, key_dim=dim, value_dim=vdim, decay_rank=rank,
                                      tau=tau, norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, dtype, seed=shape[1], matrix_std=0.2)
    T = 75
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(6)).to(dtype)
    sizes = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    want = plain.decayed_recurrence(x.double(), _right_names(w, spec), "", sizes, 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 16, 30], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)


def test_the_state_carries_a_far_token_and_a_lost_state_shows():
    """Decays close to one: a token 150 positions back still weighs in the output, so a state that
    was dropped between two steps (or begun anew) moves the result by far more than the tolerance."""
    spec = DecayedLinearAttentionSpec(hidden_size=32, num_heads=2, key_dim=8, value_dim=8, decay_rank=2, tau=64.0, norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=9, matrix_std=0.3, change=lambda v: v["decay_bias"].fill_(4.0))
    T = 160
    x = torch.randn(T, 32, generator=torch.Generator().manual_seed(7))
    sizes = {"heads": 2, "dim": 8, "vdim": 8, "tau": 64.0}
    want = plain.decayed_recurrence(x.double(), _right_names(w, spec), "", sizes, 1e-5)
    got = _step_through(part, part.cache_need(), x, [3, 100] + [1] * 57, torch.float32)
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)
    fresh = plain.decayed_recurrence(x[103:].double(), _right_names(w, spec), "", sizes, 1e-5)
    assert float((fresh[-1] - want[-1]).abs().max()) > 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_mixer_and_gated_parallel_block(dtype):
    """The pair of mixers with two caches of one run entry, then the whole block: one norm, gated
    branches, with and without a feed-forward, the branches added by the block's own kernel."""
    from clockwork_amd.cache import CacheManager, plan_groups
    from clockwork_amd.cache.pools import CachePools
    from clockwork_amd.config.spec import CacheNeeds
    from clockwork_amd.engine.batch import StepEntry, build_context
    from clockwork_amd.registry import build_arrangement

    H = 64
    left = SinkAttentionSpec(hidden_size=H, num_heads=4, num_kv_heads=2, key_dim=24, value_dim=16, scale=0.2, window=9, qk_norm_eps=1e-5)
    right = DecayedLinearAttentionSpec(hidden_size=H, num_heads=2, key_dim=12, value_dim=20, decay_rank=5, tau=4.0, norm_eps=1e-5)
    sizes = {"left": _left_sizes(left), "right": {"heads": 2, "dim": 12, "vdim": 20, "tau": 4.0}}
    for ff in (40, None):
        mixer = build_part(PairMixerSpec(hidden_size=H, left=left, right=right, eps=1e-5))
        norm = build_part(LayerNormSpec(size=H, eps=1e-5))
        gate = build_part(BranchGateSpec(hidden_size=H, branches=2 if ff else 1))
        ffn = build_part(GatedMLPSpec(H, ff)) if ff else None
        block = build_arrangement("parallel", mixer=mixer, mixer_norm=norm, feed_forward=ffn, gate=gate)
        need = mixer.cache_need()
        assert isinstance(need, CacheNeeds) and len(need.needs) == 2
        wm, wn, wg = bind(mixer, dtype, seed=1, matrix_std=0.15), bind(norm, dtype, seed=2), bind(gate, dtype, seed=3, matrix_std=0.2)
        names = {"l0.norm1": wn["weight"], "l0.norm1.b": wn["bias"], "l0.rg1": wg["weight"][:H], "l0.rg1.b": wg["bias"][:H],
                 "l0.mix.left.out": wm["left_out_norm"], "l0.mix.right.out": wm["right_out_norm"]}
        names.update({"l0.mix.left." + k: v for k, v in _left_names({k[5:]: v for k, v in wm.items() if k.startswith("left.")}, left).items()})
        names.update({"l0.mix.right." + k: v for k, v in _right_names({k[6:]: v for k, v in wm.items() if k.startswith("right.")}, right).items()})
        entry = {"type": "parallel", "mixer": sizes, "mlp": None}
        if ff:
            wf = bind(ffn, dtype, seed=4, matrix_std=0.2)
            names.update({"l0.rg2": wg["weight"][H:], "l0.rg2.b": wg["bias"][H:], "l0.mlp.gate": wf["gate_up_weight"][:ff],
                          "l0.mlp.up": wf["gate_up_weight"][ff:], "l0.mlp.down": wf["down_weight"]})
            entry["mlp"] = {"kind": "dense", "ff": ff}
        T = 40
        x0 = torch.randn(T, H, generator=torch.Generator().manual_seed(8)) * 2
        want = plain.layer(x0.double(), names, 0, entry, 1e-5)
        groups = plan_groups([need])
        assert [(g.is_kv, g.entries) for g in groups] == [(True, ((0, 0),)), (False, ((0, 1),))]
        manager = CacheManager(groups, 8, 8, max_num_seqs=2)
        pools = CachePools(groups, 8, 8, 2, dtype, torch.device(DEV), fill=float("nan"))
        cache = pools.entry_cache(0)
        assert len(cache.members) == 2 and cache.members[0].planes is not None and cache.members[1].state is not None
        got, at = [], 0
        for n in (9, 1, 2, 28):
            if at == 0:
                manager.admit("s", n)
            manager.extend("s", at, at + n)
            ctx = build_context([StepEntry("s", at, [0] * n)], manager, torch.device(DEV), 10)
            pools.set_fresh_states(ctx.state_slots, ctx.starts, ctx.num_requests)
            resid = x0[at : at + n].clone().to(DEV)
            assert block.forward(resid, None, ctx, cache) is None  # nobody said the next norm adds the branches
            got.append(resid)
            at += n
            manager.release_behind_window("s", at)
        close(torch.cat(got).double().cpu(), want, dtype)


# ------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def fuvavik_dirs(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("fuvavik")
    return {name: write_random_model(root / name, cfg, seed) for name, (cfg, seed, _) in FUVAVIK_CONFIGS.items()}


def _requests(vocab, lengths, seed):
    gen = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=gen).tolist() for i, n in enumerate(lengths)}


def _check(got, ref, dtype):
    if dtype == "float32":
        replay.compare(got, ref, rtol=3e-5, atol=3e-5)
    else:
        replay.compare_to_scale(got, ref, rms_bound=3e-2, worst_bound=1.5e-1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
@pytest.mark.parametrize("name", list(FUVAVIK_CONFIGS))
def test_models_in_four_batching_modes(fuvavik_dirs, name, mode, dtype):
    cfg, _, block_size = FUVAVIK_CONFIGS[name]
    requests = _requests(cfg["vocab"], [50, 9, 77, 30, 64, 1, 2], seed=11)
    # pages for the four longest requests and two more: freed pages and slots are used again
    # (NaN-poisoned pools: a read outside a request's pages shows)
    runner = replay.make_runner(fuvavik_dirs[name], dtype, block_size, replay.pages_needed(requests, 4, block_size) + 2)
    assert runner.manager.max_num_seqs >= 4
    oracle = plain.PlainFuvavik(fuvavik_dirs[name])
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    assert len(got) == sum(len(t) for t in requests.values())
    _check(got, ref, dtype)
    assert not runner.manager.live_requests()
    assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_through_layers_of_unlike_sizes(tmp_path, dtype):
    """1400 and 333 tokens through four layers that share no size: windows of 77 to 1500 pass over
    hundreds of tokens, keys far back are inside the longest and outside the others, the
    matrix-core kernel serves three of the four layers in bfloat16, the recurrence runs in
    segments; whole, prefill then single tokens, portions of 2 to 512 tokens, and mixed."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import FUVAVIK_LONG

    model_dir = write_random_model(tmp_path / "long", FUVAVIK_LONG, 5)
    requests = _requests(211, [1400, 333], seed=3)
    oracle = plain.PlainFuvavik(model_dir)
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    for mode in ("whole", "prefill_then_decode", "portions", "mixed"):
        runner = replay.make_runner(model_dir, dtype, 16, 120, max_model_len=1600)
        if dtype == "bfloat16":
            assert [m.left.mfma_ok for m in runner.model.mixers()] == [False, True, True, True]
        steps = replay.portions(requests, sizes=[2, 300, 7, 64, 129, 33, 512]) if mode == "portions" else getattr(replay, mode)(requests)
        _check(replay.run_trace(runner, steps), ref, dtype)
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


def test_cache_groups_of_a_model_whose_layers_differ(fuvavik_dirs):
    runner = replay.make_runner(fuvavik_dirs["FB"], "float32", 16, 40)
    groups = [(g.is_kv, g.window, g.entries) for g in runner.manager.groups]
    # layers 0 and 2 are alike and share their groups; layer 1 has groups of its own
    assert groups == [(True, 300, ((0, 0), (2, 0))), (False, None, ((0, 1), (2, 1))),
                      (True, 1, ((1, 0),)), (False, None, ((1, 1),))]
    assert not runner.manager.supports_prefix_sharing


@pytest.mark.parametrize("name", ["FA", "FB"])
def test_random_traces_with_forks(fuvavik_dirs, name):
    """Random traces (portions of 2 to 200 tokens and single tokens in any mix, requests left out of
    steps, forks cut at any token: shared pages copied on the first write, the state copied at the
    fork) on pools little larger than four requests, in float32."""
    cfg, _, _ = FUVAVIK_CONFIGS[name]
    oracle = plain.PlainFuvavik(fuvavik_dirs[name])
    for seed in range(6):
        steps, seqs = replay.random_trace(seed, cfg["vocab"], kinds=("fork",))
        seqs = {rid: toks for rid, toks in seqs.items()}
        if max(len(t) for t in seqs.values()) > cfg["max_positions"]:
            continue
        block_size = (4, 8, 16)[seed % 3]
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(fuvavik_dirs[name], "float32", block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: oracle.logits(toks) for rid, toks in seqs.items()}
        replay.compare(got, ref, rtol=3e-5, atol=3e-5)
        assert not runner.manager.live_requests()
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_replays_graphs_and_equals_eager_steps(fuvavik_dirs, dtype):
    """A prompt, then 150 single tokens (the window passes over decoded tokens, pages behind it are
    given back): with captured graphs, against the same steps run eagerly and against the plain
    implementation; two requests decode side by side, so slots and pages of both are in play."""
    cfg, _, block_size = FUVAVIK_CONFIGS["FA"]
    requests = _requests(cfg["vocab"], [200, 170], seed=12)
    steps = [{"entries": [{"id": rid, "tokens": toks[:20], "want": [19]}], "end": []} for rid, toks in requests.items()]
    for p in range(20, 170):
        steps.append({"entries": [{"id": rid, "tokens": toks[p : p + 1], "want": [0]} for rid, toks in requests.items()], "end": []})
    steps[-1]["end"] = list(requests)
    oracle = plain.PlainFuvavik(fuvavik_dirs["FA"])
    ref = {rid: oracle.logits(toks[:170]) for rid, toks in requests.items()}
    results = {}
    for graphs in (True, False):
        runner = replay.make_runner(fuvavik_dirs["FA"], dtype, block_size, 24, use_graphs=graphs)
        results[graphs] = replay.run_trace(runner, steps)
        if graphs:
            assert any(isinstance(v, tuple) for v in runner._graphs.values()), "no decode step was captured"
        _check(results[graphs], ref, dtype)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=1e-5, atol=1e-5)


def test_greedy_generation_through_the_engine(fuvavik_dirs):
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    oracle = plain.PlainFuvavik(fuvavik_dirs["FA"])
    prompts = [[3, 14, 15, 92, 65], list(range(100, 160)), [7], list(range(40))]
    want = [oracle.greedy(p, 8) for p in prompts]
    cfg = EngineConfig.defaults(str(fuvavik_dirs["FA"]), dtype="float32", block_size=8, num_blocks=48, max_num_batched_tokens=24)
    engine = LLMEngine(cfg)
    assert cfg.model.max_model_len == 640  # the model's position table ends there
    outs = engine.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    # once more on the same engine: slots and pages of the first round are used again
    outs = engine.generate(prompts[::-1], SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want[::-1]
    with pytest.raises(ValueError):
        engine.generate([[1] * 640], SamplingParams(max_tokens=4))


def test_the_command_line_and_the_trace_program(fuvavik_dirs, tmp_path):
    oracle = plain.PlainFuvavik(fuvavik_dirs["FC"])
    prompt = [5, 17, 3, 60, 1]
    out = subprocess.run([sys.executable, str(REPO / "bin" / "clockwork-generate"), "--model", str(fuvavik_dirs["FC"]),
                          "--set", "dtype=float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5"],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert json.loads(out.stdout.splitlines()[-1])["token_ids"] == oracle.greedy(prompt, 5), out.stdout
    tokens = _requests(64, [45], seed=13)["q0"]
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": tokens[30:32], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": tokens[32:], "want": [12]}], "end": ["a"]})]
    run = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(fuvavik_dirs["FC"]), "--dtype", "float32",
                          "--out", str(tmp_path / "out"), "--max-tokens", "64"], input="\n".join(lines) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np

    ref = oracle.logits(tokens)
    first = torch.from_numpy(np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(2, -1))
    last = torch.from_numpy(np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (tmp_path / "out" / "1.f32").exists()
    torch.testing.assert_close(first, ref[[0, 29]], rtol=3e-5, atol=3e-5)
    torch.testing.assert_close(last, ref[[44]], rtol=3e-5, atol=3e-5)
