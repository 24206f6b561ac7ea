"""Pesorax without a GPU: the configuration reader and what it refuses, the order of layer runs,
the weight plan against the tensors a checkpoint of the design holds, cache groups whose pages are
given back segment by segment, and invariants of the plain implementation that the GPU tests lean
on (a segment's edge, the two maps against dense matrices, latent attention against the form in
which the up-projections are applied to queries and results)."""

import copy
import json

import pytest
import torch

from clockwork_amd.cache.manager import NO_PAGE, CacheManager, plan_groups
from clockwork_amd.config.spec import PagedRowsSpec
from clockwork_amd.parts.model import DecoderModel, model_param_specs
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import check_plan
from clockwork_amd.weights.random_init import random_checkpoint_tensors, write_random_model
from tests.configs import PESORAX_A, PESORAX_B, PESORAX_C, PESORAX_LONG
from tests.plain import pesorax_plain as plain


def _describe(config):
    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    spec = arch.build_spec(cfg)
    return arch, cfg, spec, arch.weight_plan(cfg, spec)


def test_the_design_is_found_and_every_constant_is_read():
    arch, cfg, spec, _ = _describe(PESORAX_A)
    assert arch.name == "Pesorax" and spec.architecture == "Pesorax"
    assert (cfg.vocab, cfg.width, cfg.residual_mult, cfg.eps) == (300, 96, 0.5, 1e-5)
    assert not spec.tie_embeddings and spec.final_norm.delta_scale == 0.5
    a, b, c, d = spec.layers
    assert all(l.arrangement == "prenorm" for l in spec.layers)
    assert a.feed_forward.intermediate_size == 72 and b.feed_forward is None and b.ffn_norm is None
    m = a.mixer
    assert (m.num_heads, m.num_kv_heads, m.key_dim, m.value_dim, m.scale, m.lambda_init, m.segment, m.norm_eps) == \
        (6, 2, 16, 24, 0.2, 0.3, 9, 1e-5)
    m = b.mixer
    assert (m.num_heads, m.key_dim, m.rope_dim, m.rotary_dims, m.value_dim, m.q_rank, m.kv_rank, m.scale, m.rope_base) == \
        (3, 24, 16, 8, 20, 40, 48, 0.15, 100.0)
    assert c.mixer.segment == 33 and c.mixer.lambda_init == 0.8 and d.mixer.rope_base == 10000.0


def test_the_order_of_layer_runs():
    _, cfg, spec, _ = _describe(PESORAX_A)
    assert [(e.layer, e.add_input) for e in spec.run] == [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]
    assert plain.layer_order(PESORAX_A) == [(e.layer, e.add_input) for e in spec.run]
    _, _, spec, _ = _describe(PESORAX_B)   # no "loop" key: every layer once
    assert [(e.layer, e.add_input) for e in spec.run] == [(0, False), (1, False), (2, False)]
    _, _, spec, _ = _describe(PESORAX_C)   # the whole model three times
    assert [(e.layer, e.add_input) for e in spec.run] == [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False)]
    assert plain.layer_order(PESORAX_C) == [(e.layer, e.add_input) for e in spec.run]
    once = dict(PESORAX_A, loop={"start": 2, "stop": 2, "times": 5})  # an empty run of layers repeats nothing
    assert [(e.layer, e.add_input) for e in _describe(once)[2].run] == [(i, False) for i in range(4)]
    assert plain.layer_order(once) == [(i, False) for i in range(4)]


@pytest.mark.parametrize("path, value, error", [
    (("layers", 0, "type"), "recurrent", NotImplementedError),
    (("layers", 0, "mlp", "kind"), "routed", NotImplementedError),
    (("layers", 0, "mixer", "kv_heads"), 4, ValueError),
    (("layers", 0, "mixer", "mask"), None, ValueError),
    (("layers", 0, "mixer", "diff"), None, ValueError),
    (("layers", 1, "mixer", "rot"), None, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 7, ValueError),
    (("layers", 1, "mixer", "rot", "dims"), 18, ValueError),
    (("layers", 1, "mixer", "kv_rank"), 0, ValueError),
    (("loop", "stop"), 9, ValueError),
    (("loop", "times"), 0, ValueError),
    (("norm",), None, ValueError),
    (("residual_mult",), None, ValueError),
    (("layers",), [], ValueError),
    (("width",), 0, ValueError),
])
def test_what_the_configuration_reader_refuses(path, value, error):
    config = copy.deepcopy(PESORAX_A)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(error):
        _describe(config)


def _tensor_names(config):
    """Names and shapes of a checkpoint of the design, written out from the layer list."""
    W = config["width"]
    names = {"embed": (config["vocab"], W), "head": (config["vocab"], W)}

    def norm(name):
        names.update({name: (W,), name + ".b": (W,), name + ".alpha": ()})

    norm("final.norm")
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1")
        if layer["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            names.update({p + "mix.q": (H * 2 * D, W), p + "mix.q.b": (H * 2 * D,), p + "mix.k": (G * 2 * D, W),
                          p + "mix.k.b": (G * 2 * D,), p + "mix.v": (G * V, W), p + "mix.v.b": (G * V,),
                          p + "mix.o": (W, H * V)})
            names.update({p + "mix." + n: (D,) for n in ("lq1", "lk1", "lq2", "lk2")})
        else:
            H, D, R, V, qr, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            names.update({p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (D + R), qr),
                          p + "mix.dkv": (kr + R, W), p + "mix.dkv.norm": (kr,), p + "mix.uk": (H * D, kr),
                          p + "mix.uv": (H * V, kr), p + "mix.sink": (H,), p + "mix.g": (H * V, W), p + "mix.o": (W, H * V)})
        if layer["mlp"] is not None:
            norm(p + "norm2")
            names.update({p + "mlp.up": (layer["mlp"]["ff"], W), p + "mlp.down": (W, layer["mlp"]["ff"])})
    return names


@pytest.mark.parametrize("config", [PESORAX_A, PESORAX_B, PESORAX_C, PESORAX_LONG])
def test_the_weight_plan_names_every_tensor_of_the_design(config):
    _, _, spec, plan = _describe(config)
    names = _tensor_names(config)
    assert check_plan(names, plan) == ([], [], [])
    specs = model_param_specs(spec)
    assert {t.param for t in plan} == set(specs)
    # one tensor more or less is named in the error
    missing, unexpected, _ = check_plan({k: v for k, v in names.items() if k != "l0.norm1.alpha"} | {"l0.mix.extra": (3,)}, plan)
    assert missing == ["l0.norm1.alpha"] and unexpected == ["l0.mix.extra"]
    # the scalar of every norm arrives as one float32 element
    assert all(specs[n].shape == (1,) and specs[n].precision == "float32" for n in specs if n.endswith(".alpha"))


def test_random_models_hold_what_the_plain_reader_needs(tmp_path):
    for name, config in (("a", PESORAX_A), ("b", PESORAX_B), ("c", PESORAX_C)):
        folder = write_random_model(tmp_path / name, config, 5)
        oracle = plain.PlainPesorax(folder)
        assert set(oracle.w) == set(_tensor_names(config))
        assert oracle.w["final.norm.alpha"].shape == ()
        logits = oracle.logits([1, 2, 3, 4, 5])
        assert logits.shape == (5, config["vocab"]) and torch.isfinite(logits).all()
        runs = len(plain.layer_order(config))
        assert oracle.streams([1, 2, 3]).shape == (runs, 3, config["width"])


def test_cache_groups_and_pages_given_back_segment_by_segment():
    model = DecoderModel(_describe(PESORAX_A)[2])
    from clockwork_amd.cache.manager import cache_needs_of

    needs = cache_needs_of(model.spec, model.mixers())
    groups = plan_groups(needs)
    # run entries 1 and 3 are the same layer in two passes: one group, a cache each
    assert [(g.segment, g.window, g.entries) for g in groups] == [(9, None, (0,)), (None, None, (1, 3)), (33, None, (2, 4)), (None, None, (5,))]
    assert [g.need.planes[0][0] for g in groups] == ["k", "latent", "k", "latent"]
    manager = CacheManager(groups, block_size=4, num_blocks=40, max_num_seqs=4)
    assert not manager.supports_prefix_sharing
    manager.admit("s", 70, portion_end=30)
    manager.extend("s", 0, 30)
    manager.release_behind_window("s", 30)
    rec = manager.record("s")
    # the next token, position 30, lies in the segment that begins at 27 (group 0) and at 0 (group 2)
    assert rec.released[0] == 27 // 4 and all(p == NO_PAGE for p in rec.tables[0][: 27 // 4]) and rec.tables[0][27 // 4] != NO_PAGE
    assert rec.released[2] == 0 and rec.released[1] == 0 and rec.released[3] == 0
    manager.extend("s", 30, 36)
    manager.release_behind_window("s", 36)   # position 36 begins a segment of group 0: everything before it goes
    assert rec.released[0] == 9 and rec.released[2] == 33 // 4
    manager.free("s")
    assert all(p.num_free == 40 for p in manager.pools)
    with pytest.raises(ValueError):
        PagedRowsSpec((("k", (1, 4)),), window=3, segment=5)


# ------------------------------------------------------------------------------- the plain implementation
def _two_map_weights(H, G, D, V, W, seed):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    w = {"q": r(H * 2 * D, W) * 0.3, "q.b": r(H * 2 * D) * 0.1, "k": r(G * 2 * D, W) * 0.3, "k.b": r(G * 2 * D) * 0.1,
         "v": r(G * V, W) * 0.3, "v.b": r(G * V) * 0.1, "o": r(W, H * V) * 0.2}
    w.update({n: r(D) * 0.2 for n in ("lq1", "lk1", "lq2", "lk2")})
    return w


def test_plain_two_map_attention_sees_exactly_its_segment():
    H, G, D, V, W, S = 2, 1, 8, 6, 16, 7
    w = _two_map_weights(H, G, D, V, W, 1)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.4, "diff": 0.3, "mask": {"size": S}}
    x = torch.randn(30, W, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    base = plain.two_map_block_attention(x, w, "", m, 1e-6)
    moved = x.clone()
    moved[10] += 1.0   # position 10 lies in the segment 7..13
    out = plain.two_map_block_attention(moved, w, "", m, 1e-6)
    changed = (out - base).abs().amax(dim=1) > 1e-9
    assert changed.nonzero().flatten().tolist() == [10, 11, 12, 13]
    # the first token of a segment sees itself alone: its output does not depend on anything else
    alone = plain.two_map_block_attention(x[14:15], w, "", m, 1e-6)
    torch.testing.assert_close(alone[0], base[14])


def test_plain_two_map_attention_against_dense_matrices():
    H, G, D, V, W, S = 4, 2, 8, 6, 16, 5
    w = _two_map_weights(H, G, D, V, W, 3)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.4, "diff": 0.25, "mask": {"size": S}}
    T = 23
    x = torch.randn(T, W, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    q = (x @ w["q"].t() + w["q.b"]).view(T, H, 2, D)
    k = (x @ w["k"].t() + w["k.b"]).view(T, G, 2, D).repeat_interleave(H // G, dim=1)
    v = (x @ w["v"].t() + w["v.b"]).view(T, G, V).repeat_interleave(H // G, dim=1)
    pos = torch.arange(T)
    seen = (pos[None, :] <= pos[:, None]) & (pos[None, :] // S == pos[:, None] // S)
    scores = torch.einsum("ihcd,jhcd->hcij", q, k) * 0.4
    probs = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
    lam = torch.exp(w["lq1"] @ w["lk1"]) - torch.exp(w["lq2"] @ w["lk2"]) + 0.25
    o = torch.einsum("hij,jhv->ihv", probs[:, 0] - lam * probs[:, 1], v)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * 0.75
    torch.testing.assert_close(plain.two_map_block_attention(x, w, "", m, 1e-6), o.reshape(T, -1) @ w["o"].t())


def _latent_weights(H, D, R, V, qr, kr, W, seed):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    return {"dq": r(qr, W) * 0.3, "dq.norm": 1 + r(qr) * 0.1, "uq": r(H * (D + R), qr) * 0.3, "dkv": r(kr + R, W) * 0.3,
            "dkv.norm": 1 + r(kr) * 0.1, "uk": r(H * D, kr) * 0.3, "uv": r(H * V, kr) * 0.3, "sink": r(H),
            "g": r(H * V, W) * 0.3, "o": r(W, H * V) * 0.2}


def test_plain_latent_attention_against_the_form_that_caches_the_latent_alone():
    """Scores as (uk^T q) . c + rotated parts, outputs as uv (sum of weights times c): what the
    engine computes, written out densely; it must equal the plain per-head keys and values."""
    H, D, R, V, qr, kr, W, dims = 3, 8, 6, 5, 10, 12, 16, 4
    w = _latent_weights(H, D, R, V, qr, kr, W, 5)
    m = {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "q_rank": qr, "kv_rank": kr, "scale": 0.3, "rot": {"base": 50.0, "dims": dims}}
    T = 19
    x = torch.randn(T, W, generator=torch.Generator().manual_seed(6), dtype=torch.float64)
    want = plain.latent_attention(x, w, "", m, 1e-6)
    cq = plain.rms(x @ w["dq"].t(), 1e-6) * w["dq.norm"]
    q = (cq @ w["uq"].t()).view(T, H, D + R)
    down = x @ w["dkv"].t()
    c = plain.rms(down[:, :kr], 1e-6) * w["dkv.norm"]
    pos = list(range(T))
    kr_part = plain.rotate_half_pairs(down[:, kr:], pos, 50.0, dims)
    qr_part = plain.rotate_half_pairs(q[..., D:], pos, 50.0, dims)
    q_abs = torch.einsum("thd,hdr->thr", q[..., :D], w["uk"].view(H, D, kr))
    scores = (torch.einsum("ihr,jr->hij", q_abs, c) + torch.einsum("ihr,jr->hij", qr_part, kr_part)) * 0.3
    causal = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    scores = scores.masked_fill(~causal, float("-inf"))
    e = torch.exp(scores)
    probs = e / (e.sum(-1, keepdim=True) + torch.exp(w["sink"])[:, None, None])
    latent_out = torch.einsum("hij,jr->ihr", probs, c)
    o = torch.einsum("ihr,hvr->ihv", latent_out, w["uv"].view(H, V, kr)).reshape(T, H * V)
    got = (o * plain.logistic(x @ w["g"].t())) @ w["o"].t()
    torch.testing.assert_close(got, want)
    # the sink takes weight away: without it (a sink far below every score) the output differs
    no_sink = plain.latent_attention(x, dict(w, sink=w["sink"] - 50.0), "", m, 1e-6)
    assert float((no_sink - want).abs().max()) > 1e-3
    # the rotation depends on the position: the same tokens at shifted positions differ ...
    shifted = plain.latent_attention(x, w, "", m, 1e-6, positions=[p + 3 for p in pos])
    # ... but only through rounding, since scores depend on position differences alone
    torch.testing.assert_close(shifted, want)
    # and with partial rotation the elements past rot.dims pass unchanged
    v = torch.randn(4, R, dtype=torch.float64)
    torch.testing.assert_close(plain.rotate_half_pairs(v, [5, 6, 7, 8], 50.0, dims)[:, dims:], v[:, dims:])


def test_plain_norm_feed_forward_and_repeated_runs(tmp_path):
    x = torch.tensor([[0.5, -2.0, 0.0]], dtype=torch.float64)
    w, b = torch.tensor([2.0, 1.0, 3.0], dtype=torch.float64), torch.tensor([0.1, 0.2, 0.3], dtype=torch.float64)
    torch.testing.assert_close(plain.dynamic_tanh(x, w, b, torch.tensor(0.7, dtype=torch.float64)),
                               torch.tanh(0.7 * x) * w + b)
    z = torch.linspace(-3, 3, 13, dtype=torch.float64)
    torch.testing.assert_close(plain.gelu_erf(z), torch.nn.functional.gelu(z))
    # a model whose repeated layers run twice differs from the same weights run once, and the
    # input that is added again matters
    folder = write_random_model(tmp_path / "a", PESORAX_A, 9)
    oracle = plain.PlainPesorax(folder)
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    twice = oracle.logits(tokens)
    oracle.cfg = dict(oracle.cfg, loop={"start": 1, "stop": 3, "times": 1})
    assert float((oracle.logits(tokens) - twice).abs().max()) > 1e-3
