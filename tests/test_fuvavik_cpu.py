"""Fuvavik without a GPU: the configuration reader and what it refuses, the weight plan against
the tensors a checkpoint of the design holds, cache groups of mixers that keep two caches, and
invariants of the plain implementation that the GPU tests lean on (a window's edge, the sink, the
recurrence against its closed form)."""

import copy
import json

import pytest
import torch

from clockwork_amd.cache.manager import CacheManager, plan_groups
from clockwork_amd.config.spec import CacheNeeds, KVPagesSpec, PagedRowsSpec, StateSpec
from clockwork_amd.parts.model import DecoderModel, model_param_specs
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import check_plan
from clockwork_amd.weights.random_init import random_checkpoint_tensors, write_random_model
from tests.configs import FUVAVIK_A, FUVAVIK_B, FUVAVIK_C
from tests.plain import fuvavik_plain as plain


def _describe(config):
    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    spec = arch.build_spec(cfg)
    return arch, cfg, spec, arch.weight_plan(cfg, spec)


def test_the_design_is_found_by_its_one_word_key():
    arch, cfg, spec, _ = _describe(FUVAVIK_A)
    assert arch.name == "Fuvavik" and spec.architecture == "Fuvavik"
    assert (cfg.vocab, cfg.width, cfg.max_positions, cfg.embedding_scale, cfg.eps, cfg.logit_softcap) == (300, 96, 640, 2.0, 1e-5, 20.0)
    assert spec.max_positions == 640 and spec.tie_embeddings and spec.head.softcap == 20.0 and spec.embedding.scale == 2.0
    first, second = spec.layers
    assert first.arrangement == "parallel" and first.feed_forward.intermediate_size == 72 and second.feed_forward is None
    assert dict(first.extra)["gate"].branches == 2 and dict(second.extra)["gate"].branches == 1
    left, right = first.mixer.left, first.mixer.right
    assert (left.num_heads, left.num_kv_heads, left.key_dim, left.value_dim, left.scale, left.window) == (4, 2, 24, 16, 0.2, 9)
    assert (right.num_heads, right.key_dim, right.value_dim, right.tau, right.decay_rank) == (2, 12, 20, 4.0, 5)
    assert second.mixer.left.window == 33 and second.mixer.right.tau == 16.0


@pytest.mark.parametrize("path, value, error", [
    (("layers", 0, "type"), "serial", NotImplementedError),
    (("layers", 0, "mlp", "kind"), "routed", NotImplementedError),
    (("layers", 0, "mixer", "left", "kv_heads"), 3, ValueError),
    (("layers", 0, "mixer", "left", "mask"), None, ValueError),
    (("layers", 0, "mixer", "right", "tau"), 0.0, ValueError),
    (("layers", 1, "mixer", "right"), None, ValueError),
    (("norm",), None, ValueError),
    (("logit_softcap",), None, ValueError),
    (("embedding", "scale"), None, ValueError),
    (("layers",), [], ValueError),
    (("width",), 0, ValueError),
])
def test_what_the_configuration_reader_refuses(path, value, error):
    config = copy.deepcopy(FUVAVIK_A)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(error):
        resolve_architecture(config).parse_config(config)


@pytest.mark.parametrize("config", [FUVAVIK_A, FUVAVIK_B, FUVAVIK_C])
def test_the_weight_plan_names_every_tensor_of_the_design(config):
    _, cfg, spec, plan = _describe(config)
    names = {}
    for target in plan:
        if not target.optional:
            names.update(zip(target.sources, target.source_shapes))
    W = config["width"]
    expected = {"embed": (config["vocab"], W), "pos": (config["max_positions"], W), "final.norm": (W,), "final.norm.b": (W,)}
    for i, entry in enumerate(config["layers"]):
        l, r = entry["mixer"]["left"], entry["mixer"]["right"]
        p = f"l{i}."
        expected.update({
            p + "norm1": (W,), p + "norm1.b": (W,), p + "rg1": (W, W), p + "rg1.b": (W,),
            p + "mix.left.q": (l["heads"] * l["dim"], W), p + "mix.left.k": (l["kv_heads"] * l["dim"], W),
            p + "mix.left.v": (l["kv_heads"] * l["vdim"], W), p + "mix.left.q.norm": (l["heads"] * l["dim"],),
            p + "mix.left.k.norm": (l["kv_heads"] * l["dim"],), p + "mix.left.r1": (l["heads"],), p + "mix.left.r2": (l["heads"],),
            p + "mix.left.talk": (l["heads"], l["heads"]), p + "mix.left.sink": (l["heads"],),
            p + "mix.left.o": (W, l["heads"] * l["vdim"]), p + "mix.left.out": (W,), p + "mix.right.out": (W,),
            p + "mix.right.q": (r["heads"] * r["dim"], W), p + "mix.right.k": (r["heads"] * r["dim"], W),
            p + "mix.right.v": (r["heads"] * r["vdim"], W), p + "mix.right.g": (r["heads"] * r["vdim"], W),
            p + "mix.right.o": (W, r["heads"] * r["vdim"]), p + "mix.right.norm": (r["vdim"],),
            p + "mix.right.a1": (r["rank"], W), p + "mix.right.a2": (r["heads"] * r["dim"], r["rank"]),
            p + "mix.right.a2.b": (r["heads"] * r["dim"],),
        })
        if entry["mlp"] is not None:
            ff = entry["mlp"]["ff"]
            expected.update({p + "rg2": (W, W), p + "rg2.b": (W,), p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W),
                             p + "mlp.down": (W, ff)})
    assert names == expected
    # every parameter of the model is filled, and a checkpoint of exactly these tensors passes
    assert set(model_param_specs(spec)) == {t.param for t in plan}
    assert check_plan(expected, plan) == ([], [], [])
    missing, unexpected, wrong = check_plan({**{k: v for k, v in expected.items() if k != "l0.mix.left.sink"},
                                             "l0.mix.left.talk": (9, 7), "stranger": (3,)}, plan)
    assert missing == ["l0.mix.left.sink"] and unexpected == ["stranger"] and len(wrong) == 1


def test_the_decay_rank_comes_from_the_checkpoint_when_the_configuration_is_silent():
    config = copy.deepcopy(FUVAVIK_A)
    for entry in config["layers"]:
        del entry["mixer"]["right"]["rank"]
    arch = resolve_architecture(config)
    shapes = {"l0.mix.right.a1": (7, 96), "l1.mix.right.a1": (2, 96)}
    filled = arch.sizes_from_checkpoint(config, shapes)
    spec = arch.build_spec(arch.parse_config(filled))
    assert [layer.mixer.right.decay_rank for layer in spec.layers] == [7, 2]
    assert "rank" not in config["layers"][0]["mixer"]["right"]  # the caller's dict is left as it was


def test_random_models_hold_what_the_plain_reader_needs(tmp_path):
    tensors = random_checkpoint_tensors(FUVAVIK_C, seed=3)
    assert tensors["l0.mix.left.talk"].shape == (1, 1) and tensors["embed"].dtype == torch.bfloat16
    model_dir = write_random_model(tmp_path / "m", FUVAVIK_C, seed=3)
    assert json.loads((model_dir / "config.json").read_text())["architecture"] == "Fuvavik"
    logits = plain.PlainFuvavik(model_dir).logits([1, 2, 3, 4, 5])
    assert logits.shape == (5, 64) and bool(torch.isfinite(logits).all())
    assert float(logits.abs().max()) < FUVAVIK_C["logit_softcap"]


def test_a_mixer_with_two_caches_joins_two_groups():
    rows = PagedRowsSpec((("k", (2, 24)), ("v", (2, 16))), window=9)
    state = StateSpec((2, 12, 20), "float32")
    groups = plan_groups([CacheNeeds((rows, state)), KVPagesSpec(2, 16, None), CacheNeeds((rows, state)), None, state])
    assert [(g.is_kv, g.window, g.entries) for g in groups] == [
        (True, 9, ((0, 0), (2, 0))), (False, None, ((0, 1), (2, 1), 4)), (True, None, (1,))]
    manager = CacheManager(groups, block_size=4, num_blocks=10, max_num_seqs=2)
    assert not manager.supports_prefix_sharing
    manager.admit("a", 30, 6)
    assert [len(t) for t in manager.record("a").tables] == [2, 8] and manager.state_slot("a") == 0
    manager.extend("a", 6, 22)
    assert manager.release_behind_window("a", 22) == 3  # positions 0 .. 13 left the window: pages 0 .. 2
    manager.admit("b", 4)
    with pytest.raises(Exception):
        manager.admit("c", 4)  # two state slots
    manager.free("a")
    manager.admit("c", 4)
    assert manager.state_slot("c") == 0  # the freed slot is used again
    for rid in ("b", "c"):
        manager.free(rid)
    assert all(p.num_free == 10 for p in manager.pools)
    with pytest.raises(ValueError):
        CacheNeeds(())
    with pytest.raises(ValueError):
        CacheNeeds((CacheNeeds((state,)),))
    model = DecoderModel(_describe(FUVAVIK_B)[2])
    needs = [m.cache_need() for m in model.mixers()]
    assert all(isinstance(n, CacheNeeds) and isinstance(n.needs[0], PagedRowsSpec) and isinstance(n.needs[1], StateSpec) for n in needs)
    assert model.graph_safe()


# ------------------------------------------------------------------------------- the plain implementation
def _left_weights(heads, kv_heads, dim, vdim, width, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float64)
    return {"q": r(heads * dim, width), "k": r(kv_heads * dim, width), "v": r(kv_heads * vdim, width),
            "q.norm": 1 + 0.1 * r(heads * dim), "k.norm": 1 + 0.1 * r(kv_heads * dim), "r1": r(heads).abs(), "r2": r(heads).abs(),
            "sink": r(heads), "talk": torch.eye(heads, dtype=torch.float64) + 0.2 * r(heads, heads), "o": r(width, heads * vdim)}


def test_plain_attention_sees_exactly_its_window():
    sizes = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.3, "mask": {"size": 7}}
    w = _left_weights(4, 2, 6, 5, 16, seed=1)
    x = torch.randn(20, 16, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    base = plain.sink_window_attention(x, w, "", sizes, 1e-6)
    moved = x.clone()
    moved[5] += 1.0
    other = plain.sink_window_attention(moved, w, "", sizes, 1e-6)
    changed = (other - base).abs().amax(dim=1) > 1e-9
    # token 5 is seen by positions 5 .. 11 (itself and the six after it) and by no other
    assert changed.tolist() == [5 <= i <= 11 for i in range(20)]


def test_plain_attention_against_a_second_way_of_writing_it():
    """Dense matrices instead of the loop over positions: the scores of all pairs at once, the sink
    as an extra column of the softmax that is dropped afterwards, the mixing as one einsum."""
    H, G, D, V, width, window, scale = 6, 3, 4, 3, 12, 5, 0.4
    sizes = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "mask": {"size": window}}
    w = _left_weights(H, G, D, V, width, seed=3)
    T = 13
    x = torch.randn(T, width, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    q = plain.rms_norm(x @ w["q"].t(), w["q.norm"], 1e-6).view(T, H, D)
    k = plain.rms_norm(x @ w["k"].t(), w["k.norm"], 1e-6).view(T, G, D).repeat_interleave(H // G, dim=1)
    v = (x @ w["v"].t()).view(T, G, V).repeat_interleave(H // G, dim=1)
    dist = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    s = torch.einsum("ihd,jhd->hij", q, k) * scale - w["r1"][:, None, None] * torch.log1p(w["r2"][:, None, None] * dist.clamp(min=0))
    s = s.masked_fill((dist < 0) | (dist >= window), float("-inf"))
    s = torch.cat([s, w["sink"][:, None, None].expand(H, T, 1)], dim=2)
    p = torch.softmax(s, dim=2)[:, :, :T]
    mixed = torch.einsum("ab,bij->aij", w["talk"], p)
    want = torch.einsum("hij,jhv->ihv", mixed, v).reshape(T, H * V) @ w["o"].t()
    torch.testing.assert_close(plain.sink_window_attention(x, w, "", sizes, 1e-6), want, rtol=1e-10, atol=1e-10)
    # the sink takes weight: without it (a sink far below every score) the rows sum to one
    assert float(p.sum(dim=2).max()) < 1.0


def test_plain_recurrence_against_its_closed_form():
    """o_t = sum over s <= t of (q_t * prod of the decays after s up to t) . k_s  v_s."""
    H, D, V, width, rank, tau = 2, 3, 4, 10, 2, 3.0
    g = torch.Generator().manual_seed(5)
    r = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float64)
    w = {"q": r(H * D, width), "k": r(H * D, width), "v": r(H * V, width), "g": r(H * V, width), "a1": r(rank, width),
         "a2": r(H * D, rank), "a2.b": r(H * D), "norm": 1 + 0.1 * r(V), "o": r(width, H * V)}
    T = 9
    x = r(T, width)
    got = plain.decayed_recurrence(x, w, "", {"heads": H, "dim": D, "vdim": V, "tau": tau}, 1e-6)
    q = (x @ w["q"].t()).view(T, H, D) * D ** -0.5
    k = (x @ w["k"].t()).view(T, H, D)
    v = (x @ w["v"].t()).view(T, H, V)
    decay = (torch.sigmoid((x @ w["a1"].t()) @ w["a2"].t() + w["a2.b"]) ** (1 / tau)).view(T, H, D)
    o = torch.zeros(T, H, V, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            carried = torch.ones(H, D, dtype=torch.float64)
            for u in range(s + 1, t + 1):
                carried = carried * decay[u]
            o[t] += ((q[t] * carried * k[s]).sum(-1))[:, None] * v[s]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * w["norm"]
    gate = x @ w["g"].t()
    want = (o.reshape(T, H * V) * gate * torch.sigmoid(gate)) @ w["o"].t()
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-10)
