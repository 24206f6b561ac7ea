"""Fuvavik: config.json keys -> typed config -> parts -> weight names.

A decoder whose every layer has one LayerNorm and, side by side on its output, a mixer and a
dense gated feed-forward (or none), each branch gated by a sigmoid of a projection of the same
normed input before it joins the float32 residual stream. The mixer ("parallel") is a pair:
windowed softmax attention with whole-projection query/key norms, a logarithmic distance bias, a
sink and a mixing of the weights across heads, beside linear attention with a decay per key
channel; their RMS-normed outputs are averaged. The input is a scaled embedding plus a learned
position vector; the output is a LayerNorm, the embedding table itself and a tanh cap.

Every size and every constant that can differ between models of the design is read from
config.json: ``vocab``, ``width``, ``max_positions``, ``embedding.scale``, ``norm.eps``,
``logit_softcap`` and, per entry of ``layers``, ``type``, ``mixer.left`` (``heads``, ``kv_heads``,
``dim``, ``vdim``, ``scale``, ``mask.size``), ``mixer.right`` (``heads``, ``dim``, ``vdim``,
``tau``) and ``mlp`` (``kind``, ``ff``; null: the layer has no feed-forward). The rank of the
decay's projection is the shape of the checkpoint's tensor and so comes with the weights: the
configuration may name it (``mixer.right.rank``), else the loader reads it from the file.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry, WeightTarget
from clockwork_amd.parts.specs import (BranchGateSpec, DecayedLinearAttentionSpec, GatedMLPSpec, LayerNormSpec,
                                       LinearHeadSpec, PairMixerSpec, PositionTableEmbeddingSpec, SinkAttentionSpec)
from clockwork_amd.registry import Architecture, register_architecture

NAME = "Fuvavik"
DEFAULT_DECAY_RANK = 16


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ValueError(f"config.json lacks {where}{key}")
    return d[key]


@dataclass(frozen=True)
class LeftMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int


@dataclass(frozen=True)
class RightMixerConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int]  # None: as the checkpoint's tensor has it


@dataclass(frozen=True)
class FuvavikLayerConfig:
    left: LeftMixerConfig
    right: RightMixerConfig
    ff: Optional[int]  # None: no feed-forward


@dataclass(frozen=True)
class FuvavikConfig:
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    eps: float
    logit_softcap: float
    layers: tuple

    @classmethod
    def from_dict(cls, d: dict) -> "FuvavikConfig":
        if d.get("architecture", NAME) != NAME and NAME not in (d.get("architectures") or []):
            raise ValueError(f"expected a {NAME} model, got architecture={d.get('architecture')!r}")
        layers = []
        entries = _need(d, "layers", "")
        if not isinstance(entries, list) or not entries:
            raise ValueError("config.json: 'layers' must be a list with at least one layer")
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            if kind != "parallel":
                raise NotImplementedError(f"{where}type {kind!r} is not a layer of this design ('parallel')")
            mixer = _need(entry, "mixer", where)
            lm, rm = _need(mixer, "left", where + "mixer."), _need(mixer, "right", where + "mixer.")
            lw, rw = where + "mixer.left.", where + "mixer.right."
            left = LeftMixerConfig(
                heads=int(_need(lm, "heads", lw)), kv_heads=int(_need(lm, "kv_heads", lw)), dim=int(_need(lm, "dim", lw)),
                vdim=int(_need(lm, "vdim", lw)), scale=float(_need(lm, "scale", lw)),
                window=int(_need(_need(lm, "mask", lw), "size", lw + "mask.")))
            right = RightMixerConfig(
                heads=int(_need(rm, "heads", rw)), dim=int(_need(rm, "dim", rw)), vdim=int(_need(rm, "vdim", rw)),
                tau=float(_need(rm, "tau", rw)), rank=int(rm["rank"]) if rm.get("rank") is not None else None)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if _need(mlp, "kind", where + "mlp.") != "dense":
                    raise NotImplementedError(f"{where}mlp.kind {mlp['kind']!r} is not a feed-forward of this design ('dense')")
                ff = int(_need(mlp, "ff", where + "mlp."))
            layers.append(FuvavikLayerConfig(left, right, ff))
        cfg = cls(
            vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
            max_positions=int(_need(d, "max_positions", "")),
            embedding_scale=float(_need(_need(d, "embedding", ""), "scale", "embedding.")),
            eps=float(_need(_need(d, "norm", ""), "eps", "norm.")),
            logit_softcap=float(_need(d, "logit_softcap", "")), layers=tuple(layers))
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab", "width", "max_positions"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if not self.eps > 0 or not self.logit_softcap > 0:
            raise ValueError("norm.eps and logit_softcap must be positive")
        for i, layer in enumerate(self.layers):
            l, r = layer.left, layer.right
            if min(l.heads, l.kv_heads, l.dim, l.vdim, l.window, r.heads, r.dim, r.vdim) <= 0 or not r.tau > 0:
                raise ValueError(f"layers[{i}]: sizes and tau must be positive")
            if l.heads % l.kv_heads:
                raise ValueError(f"layers[{i}]: {l.heads} heads are not a multiple of {l.kv_heads} kv_heads")
            if layer.ff is not None and layer.ff <= 0:
                raise ValueError(f"layers[{i}]: mlp.ff must be positive")


def with_checkpoint_shapes(config: dict, shapes: dict) -> dict:
    """``config`` with the decay rank of every layer set from the checkpoint's tensor shapes
    (``shapes``: name -> shape) where the configuration does not give it."""
    out = dict(config)
    out["layers"] = []
    for i, entry in enumerate(config["layers"]):
        entry = dict(entry)
        name = f"l{i}.mix.right.a1"
        right = (entry.get("mixer") or {}).get("right")
        if isinstance(right, dict) and right.get("rank") is None and name in shapes:
            entry["mixer"] = dict(entry["mixer"], right=dict(right, rank=int(shapes[name][0])))
        out["layers"].append(entry)
    return out


def build_spec(cfg: FuvavikConfig) -> ModelSpec:
    W = cfg.width
    norm = LayerNormSpec(size=W, eps=cfg.eps)
    layers = []
    for layer in cfg.layers:
        l, r = layer.left, layer.right
        left = SinkAttentionSpec(hidden_size=W, num_heads=l.heads, num_kv_heads=l.kv_heads, key_dim=l.dim, value_dim=l.vdim,
                                 scale=l.scale, window=l.window, qk_norm="projection", qk_norm_eps=cfg.eps,
                                 distance_bias=True, sink=True, talking_heads=True)
        right = DecayedLinearAttentionSpec(hidden_size=W, num_heads=r.heads, key_dim=r.dim, value_dim=r.vdim,
                                           decay_rank=r.rank if r.rank is not None else DEFAULT_DECAY_RANK, tau=r.tau,
                                           norm_eps=cfg.eps)
        branches = 2 if layer.ff is not None else 1
        layers.append(LayerSpec(
            arrangement="parallel",
            mixer=PairMixerSpec(hidden_size=W, left=left, right=right, eps=cfg.eps),
            feed_forward=GatedMLPSpec(W, layer.ff, activation="gelu_tanh") if layer.ff is not None else None,
            mixer_norm=norm,
            extra=(("gate", BranchGateSpec(hidden_size=W, branches=branches)),),
        ))
    spec = ModelSpec(
        architecture=NAME, vocab_size=cfg.vocab, hidden_size=W, layers=layers,
        run=[RunEntry(layer=i) for i in range(len(layers))],
        final_norm=norm, tie_embeddings=True,
        embedding=PositionTableEmbeddingSpec(cfg.vocab, W, scale=cfg.embedding_scale, max_positions=cfg.max_positions),
        head=LinearHeadSpec(cfg.vocab, W, tied=True, softcap=cfg.logit_softcap),
        max_positions=cfg.max_positions,
        info={"layers": len(layers), "hidden": W, "vocab": cfg.vocab, "max_positions": cfg.max_positions,
              "left": [(l.left.heads, l.left.kv_heads, l.left.dim, l.left.vdim, l.left.window) for l in cfg.layers],
              "right": [(l.right.heads, l.right.dim, l.right.vdim) for l in cfg.layers],
              "ff": [l.ff for l in cfg.layers], "tied": True},
    )
    spec.validate()
    return spec


def weight_plan(cfg: FuvavikConfig, spec: ModelSpec) -> list[WeightTarget]:
    """Checkpoint names -> the model's parameters. Projections that read the same input are run
    as one product each, so they are stacked along the output dimension here: the left mixer's
    q, k, v; the right mixer's q, k, v, g and a1; the two branch gates; the feed-forward's gate
    and up."""
    W = cfg.width
    plan = [WeightTarget("embed.weight", ("embed",), ((cfg.vocab, W),)),
            WeightTarget("embed.positions", ("pos",), ((cfg.max_positions, W),))]
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}", f"layers.{i}"
        l, r = layer.left, layer.right
        rank = spec.layers[i].mixer.right.decay_rank
        lq, lk, lv = l.heads * l.dim, l.kv_heads * l.dim, l.kv_heads * l.vdim
        rq, rv = r.heads * r.dim, r.heads * r.vdim
        ml, mr = f"{src}.mix.left", f"{src}.mix.right"
        plan += [
            WeightTarget(f"{dst}.mixer_norm.weight", (f"{src}.norm1",), ((W,),)),
            WeightTarget(f"{dst}.mixer_norm.bias", (f"{src}.norm1.b",), ((W,),)),
            WeightTarget(f"{dst}.mixer.left.qkv_weight", (f"{ml}.q", f"{ml}.k", f"{ml}.v"), ((lq, W), (lk, W), (lv, W))),
            WeightTarget(f"{dst}.mixer.left.q_norm", (f"{ml}.q.norm",), ((lq,),)),
            WeightTarget(f"{dst}.mixer.left.k_norm", (f"{ml}.k.norm",), ((lk,),)),
            WeightTarget(f"{dst}.mixer.left.r1", (f"{ml}.r1",), ((l.heads,),)),
            WeightTarget(f"{dst}.mixer.left.r2", (f"{ml}.r2",), ((l.heads,),)),
            WeightTarget(f"{dst}.mixer.left.sink", (f"{ml}.sink",), ((l.heads,),)),
            WeightTarget(f"{dst}.mixer.left.talk", (f"{ml}.talk",), ((l.heads, l.heads),)),
            WeightTarget(f"{dst}.mixer.left.out_weight", (f"{ml}.o",), ((W, l.heads * l.vdim),)),
            WeightTarget(f"{dst}.mixer.right.in_weight", (f"{mr}.q", f"{mr}.k", f"{mr}.v", f"{mr}.g", f"{mr}.a1"),
                         ((rq, W), (rq, W), (rv, W), (rv, W), (rank, W))),
            WeightTarget(f"{dst}.mixer.right.decay_weight", (f"{mr}.a2",), ((rq, rank),)),
            WeightTarget(f"{dst}.mixer.right.decay_bias", (f"{mr}.a2.b",), ((rq,),)),
            WeightTarget(f"{dst}.mixer.right.norm_weight", (f"{mr}.norm",), ((r.vdim,),)),
            WeightTarget(f"{dst}.mixer.right.out_weight", (f"{mr}.o",), ((W, rv),)),
            WeightTarget(f"{dst}.mixer.left_out_norm", (f"{ml}.out",), ((W,),)),
            WeightTarget(f"{dst}.mixer.right_out_norm", (f"{mr}.out",), ((W,),)),
        ]
        gates, biases = [f"{src}.rg1"], [f"{src}.rg1.b"]
        if layer.ff is not None:
            gates.append(f"{src}.rg2")
            biases.append(f"{src}.rg2.b")
            plan += [
                WeightTarget(f"{dst}.feed_forward.gate_up_weight", (f"{src}.mlp.gate", f"{src}.mlp.up"),
                             ((layer.ff, W), (layer.ff, W))),
                WeightTarget(f"{dst}.feed_forward.down_weight", (f"{src}.mlp.down",), ((W, layer.ff),)),
            ]
        plan += [
            WeightTarget(f"{dst}.gate.weight", tuple(gates), tuple((W, W) for _ in gates)),
            WeightTarget(f"{dst}.gate.bias", tuple(biases), tuple((W,) for _ in biases)),
        ]
    plan += [WeightTarget("final_norm.weight", ("final.norm",), ((W,),)),
             WeightTarget("final_norm.bias", ("final.norm.b",), ((W,),)),
             # the output head is the embedding table: the design has no tensor of its own for it
             WeightTarget("lm_head.weight", ("lm_head",), ((cfg.vocab, W),), optional=True)]
    return plan


ARCHITECTURE = Architecture(name=NAME, parse_config=FuvavikConfig.from_dict, build_spec=build_spec, weight_plan=weight_plan,
                            sizes_from_checkpoint=with_checkpoint_shapes)
register_architecture([NAME], ARCHITECTURE)
