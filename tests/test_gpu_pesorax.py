"""Pesorax on the GPU against the plain implementation (tests/plain/pesorax_plain.py): each new
kernel and part alone, then whole models of three small configurations replayed whole, as prefill
then single tokens, in portions down to two tokens and as mixed batches on tight page pools, in
both dtypes; segments' edges and far keys with weights made so that one key decides the output;
long decoding; forks; greedy generation through the engine's entry point, the command line and
the trace program."""

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from clockwork_amd import ops
from clockwork_amd.parts.specs import DenseMLPSpec, DifferentialAttentionSpec, DynamicTanhSpec, LatentAttentionSpec
from clockwork_amd.registry import build_part
from tests import replay
from tests.configs import PESORAX_CONFIGS
from tests.plain import pesorax_plain as plain
from tests.test_gpu_fuvavik import _step_through, bind, close

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPO = Path(__file__).resolve().parents[1]


# ------------------------------------------------------------------------------- norm and feed-forward
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [100, 257, 1024])
def test_dynamic_tanh_alone_with_a_scaled_branch_and_with_the_input_again(dtype, width):
    part = build_part(DynamicTanhSpec(size=width, delta_scale=0.3))
    w = bind(part, dtype, seed=width)
    gen = torch.Generator().manual_seed(1)
    T = 37
    resid0 = torch.randn(T, width, generator=gen) * 2
    delta = (torch.randn(T, width, generator=gen)).to(dtype)
    extra = torch.randn(T, width, generator=gen)
    alpha = w["alpha"].reshape(())

    def want(x):
        return plain.dynamic_tanh(x, w["weight"], w["bias"], alpha)

    resid = resid0.clone().to(DEV)
    close(part.forward(resid, None).double().cpu(), want(resid0.double()), dtype)
    torch.testing.assert_close(resid.cpu(), resid0)                      # nothing pending: the stream stays
    got = part.forward(resid, delta.to(DEV)).double().cpu()
    summed = resid0.double() + 0.3 * delta.double()
    close(got, want(summed), dtype)
    torch.testing.assert_close(resid.cpu().double(), summed, rtol=1e-6, atol=1e-6)   # the float32 stream took the branch
    resid = resid0.clone().to(DEV)
    got = part.forward(resid, ops.WithStreamInput(delta.to(DEV), extra.to(DEV))).double().cpu()
    close(got, want(summed + extra.double()), dtype)
    torch.testing.assert_close(resid.cpu().double(), summed + extra.double(), rtol=1e-6, atol=1e-6)
    # chosen rows only (the final norm): the stream is left alone
    resid = resid0.clone().to(DEV)
    rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)
    got = part.forward(resid, delta.to(DEV), rows=rows).double().cpu()
    close(got, want(summed[[5, 0, 36]]), dtype)
    torch.testing.assert_close(resid.cpu(), resid0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, rows", [(100, 41), (128, 8), (128, 41), (1024, 3), (128, 200)])
def test_dense_gelu_feed_forward(dtype, hidden, rows):
    """Few bfloat16 rows of a width that is a multiple of 8 take the product with the activation
    in its epilogue, the others the product and the activation kernel."""
    from types import SimpleNamespace

    part = build_part(DenseMLPSpec(hidden_size=hidden, intermediate_size=72))
    w = bind(part, dtype, seed=2, matrix_std=0.2)
    x = torch.randn(rows, hidden, generator=torch.Generator().manual_seed(3)).to(dtype)
    got = part.forward(x.to(DEV), SimpleNamespace()).double().cpu()
    close(got, plain.dense_feed_forward(x.double(), {"up": w["up_weight"], "down": w["down_weight"]}, ""), dtype)
    if dtype == torch.bfloat16:
        inner = ops.linear_gelu(x.to(DEV), part.up).double().cpu()
        want = plain.gelu_erf(x.double() @ w["up_weight"].t())
        close(inner, want, dtype)


# ------------------------------------------------------------------------------- two-map attention
def _two_map_names(w, spec):
    nq = spec.num_heads * 2 * spec.key_dim
    nk = spec.num_kv_heads * 2 * spec.key_dim
    qkv, b = w["qkv_weight"], w["qkv_bias"]
    out = {"q": qkv[:nq], "k": qkv[nq : nq + nk], "v": qkv[nq + nk :], "q.b": b[:nq], "k.b": b[nq : nq + nk], "v.b": b[nq + nk :],
           "o": w["out_weight"]}
    out.update({n: w[n] for n in ("lq1", "lk1", "lq2", "lk2")})
    return out


def _two_map_sizes(spec):
    return {"heads": spec.num_heads, "kv_heads": spec.num_kv_heads, "dim": spec.key_dim, "vdim": spec.value_dim,
            "scale": spec.scale, "diff": spec.lambda_init, "mask": {"size": spec.segment}}


# heads, kv_heads, dim, vdim, segment, hidden: grouped heads, a group larger than a workgroup takes
# at once, sizes of 1, value sizes that are no multiple of 16, a segment longer than the sequence
TWO_MAP_SHAPES = [(4, 2, 24, 16, 9, 64), (6, 6, 16, 16, 33, 96), (3, 1, 40, 24, 300, 100), (2, 1, 8, 32, 1, 48),
                  (1, 1, 32, 8, 17, 48), (20, 2, 8, 20, 12, 64), (2, 2, 64, 130, 16, 64), (8, 2, 64, 128, 40, 128),
                  # the other sizes that the matrix-core kernel is built for
                  (4, 2, 128, 128, 40, 64), (3, 1, 128, 64, 16, 64), (2, 1, 64, 256, 25, 64), (2, 2, 128, 256, 30, 64),
                  (10, 2, 64, 64, 21, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", TWO_MAP_SHAPES)
def test_two_map_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, kv_heads, dim, vdim, segment, hidden = shape
    spec = DifferentialAttentionSpec(hidden_size=hidden, num_heads=heads, num_kv_heads=kv_heads, key_dim=dim, value_dim=vdim,
                                     scale=0.21, lambda_init=0.35, norm_eps=1e-5, segment=segment)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.15)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.two_map_block_attention(x.double(), _two_map_names(w, spec), "", _two_map_sizes(spec), 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 32], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)
    _matrix_cores_against_plain_arithmetic(part, x, want, dtype)


def _matrix_cores_against_plain_arithmetic(part, x, want, dtype):
    """Where the matrix-core kernel runs: against the plain-arithmetic kernel on the very same
    bfloat16 queries, keys and values. They differ by the order of their sums, by the weights'
    rounding to bfloat16 before the value product and by the rounding of the output, a fraction of
    what separates either from the float64 result."""
    if not part.mfma:
        return
    assert dtype == torch.bfloat16
    T = x.shape[0]
    fast = _step_through(part, part.cache_need(), x, [T], dtype)
    s = part.spec
    part.mfma = False
    part.run = (ops.rows_attention_tokens_per_item(s.num_heads, s.num_kv_heads, 2) if hasattr(s, "num_kv_heads")
                else ops.rows_attention_tokens_per_item(s.num_heads, 1, 1))
    slow = _step_through(part, part.cache_need(), x, [T], dtype)
    scale = float(want.square().mean().sqrt())
    assert float((fast - slow).abs().max()) < 3e-2 * scale and float((fast - slow).square().mean().sqrt()) < 6e-3 * scale


def test_the_matrix_core_kernel_is_the_one_that_runs_for_bfloat16():
    two = DifferentialAttentionSpec(hidden_size=64, num_heads=8, num_kv_heads=2, key_dim=64, value_dim=128, scale=0.1,
                                    lambda_init=0.5, norm_eps=1e-6, segment=40)
    latent = LatentAttentionSpec(hidden_size=64, num_heads=4, key_dim=32, rope_dim=64, value_dim=32, q_rank=48, kv_rank=256,
                                 scale=0.1, rope_base=100.0, rotary_dims=64, norm_eps=1e-6)
    for spec in (two, latent):
        for dtype, expected in ((torch.bfloat16, True), (torch.float32, False)):
            part = build_part(spec)
            bind(part, dtype)
            assert part.mfma is expected and part.run == (16 if expected else part.run)
    odd = build_part(DifferentialAttentionSpec(hidden_size=64, num_heads=4, num_kv_heads=2, key_dim=24, value_dim=16, scale=0.1,
                                               lambda_init=0.5, norm_eps=1e-6, segment=9))
    bind(odd, torch.bfloat16)
    assert not odd.mfma and odd.run >= 1


def test_two_map_attention_options_each_matter():
    """lambda, the biases, the head norm's constant and the segment each change the result by much
    more than the tolerance, so the comparison above would not pass without any of them."""
    spec = DifferentialAttentionSpec(hidden_size=64, num_heads=4, num_kv_heads=2, key_dim=24, value_dim=16, scale=0.21,
                                     lambda_init=0.35, norm_eps=1e-5, segment=9)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=7, matrix_std=0.15)
    x = torch.randn(30, 64, generator=torch.Generator().manual_seed(5))
    got = _step_through(part, part.cache_need(), x, [30], torch.float32)
    base, sizes = _two_map_names(w, spec), _two_map_sizes(spec)
    torch.testing.assert_close(got, plain.two_map_block_attention(x.double(), base, "", sizes, 1e-5), rtol=2e-5, atol=2e-5)
    # (a key bias alone would not show: it moves all scores of a query by the same amount)
    for change in ({"lq1": base["lq1"] + 1.0}, {"q.b": base["q.b"] + 1.5 * (torch.arange(base["q.b"].numel()) % 3 - 1)},
                   {"v.b": base["v.b"] + 0.5}):
        other = plain.two_map_block_attention(x.double(), dict(base, **change), "", sizes, 1e-5)
        assert float((other - got).abs().max()) > 1e-2, list(change)
    for change in ({"diff": 0.6}, {"mask": {"size": 10}}, {"scale": 0.4}):
        other = plain.two_map_block_attention(x.double(), base, "", dict(sizes, **change), 1e-5)
        assert float((other - got).abs().max()) > 1e-2, list(change)


def _loud_two_map_part(hidden, dim, vdim, segment, dtype):
    """A layer in which one marked token decides the output of every later token of its segment:
    input element 0 marks the loud token (it alone sets key channel 0 of the first map and value
    channel 0); element 1, which every token carries, sets query channel 0 of the first map and
    value channel 1. The second map's scores are all equal, lambda is lambda_init = 0.5. While the
    loud key is seen the normed output points along value channel 0, else along channel 1."""
    spec = DifferentialAttentionSpec(hidden_size=hidden, num_heads=2, num_kv_heads=1, key_dim=dim, value_dim=vdim, scale=1.0,
                                     lambda_init=0.5, norm_eps=1e-6, segment=segment)
    part = build_part(spec)

    def change(v):
        for name in ("qkv_weight", "qkv_bias", "lq1", "lk1", "lq2", "lk2", "out_weight"):
            v[name].zero_()
        nq, nk = 2 * 2 * dim, 2 * dim
        v["qkv_weight"][0, 1] = 6.0                 # head 0, map 0, channel 0
        v["qkv_weight"][2 * dim, 1] = 6.0           # head 1, map 0, channel 0
        v["qkv_weight"][nq, 0] = 1.0                # key, map 0, channel 0
        v["qkv_weight"][nq + nk, 0] = 1.0           # value channel 0
        v["qkv_weight"][nq + nk + 1, 1] = 1.0       # value channel 1
        v["out_weight"][0, 0] = 1.0                 # head 0's channel 0
        v["out_weight"][1, vdim] = 1.0              # head 1's channel 0
        v["out_weight"][2, 1] = 1.0                 # head 0's channel 1

    return spec, part, bind(part, dtype, change=change)


@pytest.mark.parametrize("segment", [5, 16, 17, 40])
@pytest.mark.parametrize("cuts", ["whole", "portions", "single"])
def test_one_loud_key_just_inside_and_just_outside_the_segment(segment, cuts):
    """The loud token sits at the third place of the second segment: every later token of that
    segment must show it, the first token of the next segment and all after it must not. Pages of 4
    and 8 tokens put the edges at page borders and inside pages; pages before the running segment
    are given back and used again."""
    hidden, dim, vdim = 32, 16, 8
    spec, part, w = _loud_two_map_part(hidden, dim, vdim, segment, torch.float32)
    T, loud = 3 * segment + 3, segment + 2
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    want = plain.two_map_block_attention(x.double(), _two_map_names(w, spec), "", _two_map_sizes(spec), 1e-6)
    top = (1 - 0.5) * vdim ** 0.5
    # the plain result itself shows the edges
    if segment > 3:
        assert float(want[2 * segment - 1, 0]) > 0.9 * top
    assert abs(float(want[2 * segment, 0])) < 1e-6 and abs(float(want[loud - 1, 0])) < 1e-6 and float(want[loud, 0]) > 0.9 * top
    for block_size in (4, 8):
        steps = {"whole": [T], "portions": [2, 7, 3, 16, 5, 2, 31, 4, 2, 60], "single": [loud + 1] + [1] * (T - loud - 1)}[cuts]
        done, kept = 0, []
        for n in steps:
            n = min(n, T - done)
            if n:
                kept.append(n)
                done += n
        if done < T:
            kept.append(T - done)
        got = _step_through(part, part.cache_need(), x, kept, torch.float32, block_size=block_size, num_blocks=32)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_decides_the_two_map_output(dtype):
    """The same loud key in segments of 400: it is one of up to 398 keys that a query of its
    segment sees, and gone at the first token of the next segment."""
    hidden, dim, vdim, segment = 32, 64, 64, 400
    spec, part, w = _loud_two_map_part(hidden, dim, vdim, segment, dtype)
    assert part.mfma == (dtype == torch.bfloat16)
    T, loud = 850, 402
    x = torch.zeros(T, hidden)
    x[:, 1] = 1.0
    x[loud, 0] = 4.0
    want = plain.two_map_block_attention(x.double(), _two_map_names(w, spec), "", _two_map_sizes(spec), 1e-6)
    assert float(want[799, 0]) > 3.5 and abs(float(want[800, 0])) < 1e-6 and abs(float(want[401, 0])) < 1e-6
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for steps in ([T], [2, 300, 107, 64, 329, 33, 15], [760] + [1] * 90):
        got = _step_through(part, part.cache_need(), x, steps, dtype, block_size=16, num_blocks=64)
        torch.testing.assert_close(got, want, **tol)


# ------------------------------------------------------------------------------- latent attention
def _latent_names(w, spec):
    a, b = spec.q_rank, spec.q_rank + spec.kv_rank + spec.rope_dim
    return {"dq": w["in_weight"][:a], "dkv": w["in_weight"][a:b], "g": w["in_weight"][b:], "dq.norm": w["q_norm"],
            "dkv.norm": w["kv_norm"], "uq": w["q_up_weight"], "uk": w["k_up_weight"], "uv": w["v_up_weight"],
            "sink": w["sink"], "o": w["out_weight"]}


def _latent_sizes(spec):
    return {"heads": spec.num_heads, "dim": spec.key_dim, "rot_dim": spec.rope_dim, "vdim": spec.value_dim, "q_rank": spec.q_rank,
            "kv_rank": spec.kv_rank, "scale": spec.scale, "rot": {"base": spec.rope_base, "dims": spec.rotary_dims}}


# heads, dim, rot_dim, rot dims, vdim, q_rank, kv_rank, hidden: partial rotation, sizes of 1 and 2, more
# heads than a workgroup takes at once, latents of 256 + 64 and 512 + 64 elements
LATENT_SHAPES = [(3, 24, 16, 8, 20, 40, 48, 96), (1, 2, 2, 2, 1, 4, 8, 48), (5, 8, 4, 4, 12, 20, 36, 100),
                 (20, 8, 8, 8, 8, 16, 16, 64), (4, 32, 64, 64, 32, 48, 256, 64), (2, 16, 8, 0, 16, 12, 24, 64),
                 (5, 16, 64, 64, 16, 32, 512, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", LATENT_SHAPES)
def test_latent_attention_whole_in_portions_and_token_by_token(dtype, shape):
    heads, dim, rot_dim, rot_dims, vdim, q_rank, kv_rank, hidden = shape
    spec = LatentAttentionSpec(hidden_size=hidden, num_heads=heads, key_dim=dim, rope_dim=rot_dim, value_dim=vdim, q_rank=q_rank,
                               kv_rank=kv_rank, scale=0.3 if kv_rank < 100 else 0.06, rope_base=77.0, rotary_dims=rot_dims,
                               norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, dtype, seed=heads, matrix_std=0.2)
    T = 61
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.latent_attention(x.double(), _latent_names(w, spec), "", _latent_sizes(spec), 1e-5)
    for cuts in ([T], [5, 1, 1, 17, 2, 1, 2, 32], [1] * T):
        got = _step_through(part, part.cache_need(), x, cuts, dtype)
        close(got, want, dtype)
    _matrix_cores_against_plain_arithmetic(part, x, want, dtype)


def test_latent_attention_options_each_matter():
    spec = LatentAttentionSpec(hidden_size=64, num_heads=3, key_dim=24, rope_dim=16, value_dim=20, q_rank=40, kv_rank=48,
                               scale=0.3, rope_base=77.0, rotary_dims=8, norm_eps=1e-5)
    part = build_part(spec)
    w = bind(part, torch.float32, seed=7, matrix_std=0.2)
    x = torch.randn(30, 64, generator=torch.Generator().manual_seed(5))
    got = _step_through(part, part.cache_need(), x, [30], torch.float32)
    base, sizes = _latent_names(w, spec), _latent_sizes(spec)
    torch.testing.assert_close(got, plain.latent_attention(x.double(), base, "", sizes, 1e-5), rtol=2e-5, atol=2e-5)
    for change in ({"sink": base["sink"] - 30.0}, {"g": base["g"] * 0}, {"dkv.norm": base["dkv.norm"] * 0 + 1.0},
                   {"dq.norm": base["dq.norm"] * 0 + 1.0}):
        other = plain.latent_attention(x.double(), dict(base, **change), "", sizes, 1e-5)
        assert float((other - got).abs().max()) > 3e-3, list(change)
    for change in ({"rot": {"base": 77.0, "dims": 16}}, {"rot": {"base": 1000.0, "dims": 8}}, {"scale": 0.5}):
        other = plain.latent_attention(x.double(), base, "", dict(sizes, **change), 1e-5)
        assert float((other - got).abs().max()) > 3e-3, list(change)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sharp_latent_attention_over_hundreds_of_keys(dtype):
    """A scale so large that every query gives nearly all its weight to the one or two keys that
    fit it best, wherever among up to 500 earlier tokens they lie: a key that is lost or taken from
    a wrong page changes the output wholly. Positions enter through the rotated part alone."""
    spec = LatentAttentionSpec(hidden_size=64, num_heads=6, key_dim=32, rope_dim=32, value_dim=32, q_rank=48, kv_rank=128,
                               scale=1.2, rope_base=10000.0, rotary_dims=32, norm_eps=1e-6)
    part = build_part(spec)
    w = bind(part, dtype, seed=11, matrix_std=0.25, change=lambda v: v["sink"].fill_(-5.0))
    assert part.mfma == (dtype == torch.bfloat16)   # in bfloat16 on the matrix cores, the keys of long ranges cut into runs
    T = 500
    x = torch.randn(T, 64, generator=torch.Generator().manual_seed(6)).to(dtype)
    want = plain.latent_attention(x.double(), _latent_names(w, spec), "", _latent_sizes(spec), 1e-6)
    for steps in ([T], [2, 300, 7, 64, 29, 33, 65], [440] + [1] * 60):
        got = _step_through(part, part.cache_need(), x, steps, dtype, block_size=16, num_blocks=40)
        if dtype == torch.float32:
            # scores of about a hundred before the softmax: their float32 rounding, some 1e-5, is a
            # relative error of the weights; a wrong key would be an error of the output's own size
            torch.testing.assert_close(got, want, rtol=2e-3, atol=2e-3)
        else:
            # sharp scores amplify the rounding of bfloat16 queries and latents: the error is judged
            # against the output's scale, and a wrong key would be an error of that scale itself
            scale = float(want.square().mean().sqrt())
            assert float((got - want).square().mean().sqrt()) < 0.08 * scale


# ------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def pesorax_dirs(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("pesorax")
    return {name: write_random_model(root / name, cfg, seed) for name, (cfg, seed, _) in PESORAX_CONFIGS.items()}


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
@pytest.mark.parametrize("name", list(PESORAX_CONFIGS))
def test_models_in_four_batching_modes(pesorax_dirs, name, mode, dtype):
    cfg, _, block_size = PESORAX_CONFIGS[name]
    requests = _requests(cfg["vocab"], [50, 9, 77, 30, 64, 1, 2], seed=11)
    # pages for the four longest requests and two more: freed pages are used again (NaN-poisoned
    # pools: a read outside a request's pages shows)
    runner = replay.make_runner(pesorax_dirs[name], dtype, block_size, replay.pages_needed(requests, 4, block_size) + 2)
    oracle = plain.PlainPesorax(pesorax_dirs[name])
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    assert len(got) == sum(len(t) for t in requests.values())
    _check(got, ref, dtype)
    assert not runner.manager.live_requests()
    assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


def test_the_stream_after_every_layer_run(pesorax_dirs):
    """Float32, one request: the residual stream after every run of a layer (repeated layers
    count each time) against the plain implementation's."""
    cfg, _, block_size = PESORAX_CONFIGS["PA"]
    runner = replay.make_runner(pesorax_dirs["PA"], "float32", block_size, 16)
    tokens = _requests(cfg["vocab"], [40], seed=2)["q0"]
    seen = []
    for layer in runner.model.layers:
        inner = layer.forward

        def forward(resid, delta, ctx, cache, inner=inner):
            out = inner(resid, delta, ctx, cache)
            seen.append((resid + cfg["residual_mult"] * out.float()).cpu())
            return out

        layer.forward = forward
    replay.run_trace(runner, replay.whole({"a": tokens}))
    want = plain.PlainPesorax(pesorax_dirs["PA"]).streams(tokens)
    assert len(seen) == want.shape[0] == 6
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_through_layers_of_unlike_sizes(tmp_path, dtype):
    """1400 and 333 tokens through five layers that share no size: segments of 77 to 1500 begin and
    end hundreds of tokens into the requests, the latent layers see every earlier token; whole,
    prefill then single tokens, portions of 2 to 512 tokens, and mixed."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import PESORAX_LONG

    model_dir = write_random_model(tmp_path / "long", PESORAX_LONG, 5)
    requests = _requests(211, [1400, 333], seed=3)
    oracle = plain.PlainPesorax(model_dir)
    ref = {rid: oracle.logits(toks) for rid, toks in requests.items()}
    for mode in ("whole", "prefill_then_decode", "portions", "mixed"):
        runner = replay.make_runner(model_dir, dtype, 16, 120, max_model_len=1600)
        if dtype == "bfloat16":
            assert [m.mfma for m in runner.model.mixers()] == [False, True, True, True, True]
        steps = replay.portions(requests, sizes=[2, 300, 7, 64, 129, 33, 512]) if mode == "portions" else getattr(replay, mode)(requests)
        _check(replay.run_trace(runner, steps), ref, dtype)
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


def test_cache_groups_of_a_model_whose_layers_differ(pesorax_dirs):
    runner = replay.make_runner(pesorax_dirs["PA"], "float32", 8, 40)
    groups = [(g.is_kv, g.segment, g.entries) for g in runner.manager.groups]
    assert groups == [(True, 9, (0,)), (True, None, (1, 3)), (True, 33, (2, 4)), (True, None, (5,))]
    assert not runner.manager.supports_prefix_sharing


@pytest.mark.parametrize("name", ["PA", "PB"])
def test_random_traces_with_forks(pesorax_dirs, name):
    """Random traces (portions of 2 to 200 tokens and single tokens in any mix, requests left out of
    steps, forks cut at any token: shared pages copied on the first write) on pools little larger
    than four requests, in float32."""
    cfg, _, _ = PESORAX_CONFIGS[name]
    oracle = plain.PlainPesorax(pesorax_dirs[name])
    for seed in range(6):
        steps, seqs = replay.random_trace(seed, cfg["vocab"], kinds=("fork",))
        block_size = (4, 8, 16)[seed % 3]
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(pesorax_dirs[name], "float32", block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: oracle.logits(toks) for rid, toks in seqs.items()}
        replay.compare(got, ref, rtol=3e-5, atol=3e-5)
        assert not runner.manager.live_requests()
        assert all(p.num_free == runner.manager.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_replays_graphs_and_equals_eager_steps(pesorax_dirs, dtype):
    """A prompt, then 150 single tokens (segments of 9 and 33 begin among the decoded tokens, pages
    before them are given back): with captured graphs, against the same steps run eagerly and
    against the plain implementation; two requests decode side by side."""
    cfg, _, block_size = PESORAX_CONFIGS["PA"]
    requests = _requests(cfg["vocab"], [200, 170], seed=12)
    steps = [{"entries": [{"id": rid, "tokens": toks[:20], "want": [19]}], "end": []} for rid, toks in requests.items()]
    for p in range(20, 170):
        steps.append({"entries": [{"id": rid, "tokens": toks[p : p + 1], "want": [0]} for rid, toks in requests.items()], "end": []})
    steps[-1]["end"] = list(requests)
    oracle = plain.PlainPesorax(pesorax_dirs["PA"])
    ref = {rid: oracle.logits(toks[:170]) for rid, toks in requests.items()}
    results = {}
    for graphs in (True, False):
        runner = replay.make_runner(pesorax_dirs["PA"], dtype, block_size, 64, use_graphs=graphs)
        results[graphs] = replay.run_trace(runner, steps)
        if graphs:
            assert any(isinstance(v, tuple) for v in runner._graphs.values()), "no decode step was captured"
        _check(results[graphs], ref, dtype)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=1e-5, atol=1e-5)


def test_greedy_generation_through_the_engine(pesorax_dirs):
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    oracle = plain.PlainPesorax(pesorax_dirs["PA"])
    prompts = [[3, 14, 15, 92, 65], list(range(100, 160)), [7], list(range(40))]
    want = [oracle.greedy(p, 8) for p in prompts]
    cfg = EngineConfig.defaults(str(pesorax_dirs["PA"]), dtype="float32", block_size=8, num_blocks=64, max_num_batched_tokens=24)
    engine = LLMEngine(cfg)
    outs = engine.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want
    # once more on the same engine: pages of the first round are used again
    outs = engine.generate(prompts[::-1], SamplingParams(max_tokens=8, temperature=0.0))
    assert [o.token_ids for o in outs] == want[::-1]


def test_the_command_line_and_the_trace_program(pesorax_dirs, tmp_path):
    oracle = plain.PlainPesorax(pesorax_dirs["PC"])
    prompt = [5, 17, 3, 60, 1]
    out = subprocess.run([sys.executable, str(REPO / "bin" / "clockwork-generate"), "--model", str(pesorax_dirs["PC"]),
                          "--set", "dtype=float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5"],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert json.loads(out.stdout.splitlines()[-1])["token_ids"] == oracle.greedy(prompt, 5), out.stdout
    tokens = _requests(64, [45], seed=13)["q0"]
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": tokens[30:32], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": tokens[32:], "want": [12]}], "end": ["a"]})]
    run = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(pesorax_dirs["PC"]), "--dtype", "float32",
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
