"""Pesorax: config.json keys -> typed config -> parts -> weight names.

A pre-norm decoder whose norms are Dynamic Tanh (tanh(alpha x) * w + b, no statistics) and whose
branches join the float32 residual stream multiplied by ``residual_mult``. A layer's mixer is one
of two kinds: "attention", grouped attention with two score maps a head whose difference is
normed per head, over keys of the token's own run of ``mask.size`` positions, with biased
projections and no position encoding; or "latent_attention", causal attention over one cached
latent a token with low-rank queries, a rotated key part shared by the heads, a sink in the
softmax denominator and a sigmoid output gate. The feed-forward is dense, down(gelu(up x)), or
absent. A run of layers (``loop.start .. loop.stop - 1``) is repeated ``loop.times`` times with the
same weights and a cache per pass, the embedding output being added to the stream again before
every pass but the first. The output is the model's norm and an untied head.

Every size and every constant that can differ between models of the design is read from
config.json: ``vocab``, ``width``, ``residual_mult``, ``norm.eps``, ``loop`` and, per entry of
``layers``, ``type``, ``mixer`` (attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``,
``diff``, ``mask.size``; latent_attention: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``,
``kv_rank``, ``scale``, ``rot.base``, ``rot.dims``) and ``mlp`` (``kind``, ``ff``; null: no feed-forward).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry, WeightTarget
from clockwork_amd.parts.specs import (DenseMLPSpec, DifferentialAttentionSpec, DynamicTanhSpec, LatentAttentionSpec,
                                       LinearHeadSpec, TokenEmbeddingSpec)
from clockwork_amd.registry import Architecture, register_architecture

NAME = "Pesorax"


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ValueError(f"config.json lacks {where}{key}")
    return d[key]


@dataclass(frozen=True)
class TwoMapMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    segment: int


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class PesoraxLayerConfig:
    kind: str          # "attention" or "latent_attention"
    mixer: object
    ff: Optional[int]  # None: no feed-forward


@dataclass(frozen=True)
class LoopConfig:
    start: int = 0
    stop: int = 0
    times: int = 1


@dataclass(frozen=True)
class PesoraxConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    loop: LoopConfig
    layers: tuple

    @classmethod
    def from_dict(cls, d: dict) -> "PesoraxConfig":
        if d.get("architecture", NAME) != NAME and NAME not in (d.get("architectures") or []):
            raise ValueError(f"expected a {NAME} model, got architecture={d.get('architecture')!r}")
        entries = _need(d, "layers", "")
        if not isinstance(entries, list) or not entries:
            raise ValueError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            kind = _need(entry, "type", where)
            m, mw = _need(entry, "mixer", where), where + "mixer."
            if kind == "attention":
                mixer = TwoMapMixerConfig(
                    heads=int(_need(m, "heads", mw)), kv_heads=int(_need(m, "kv_heads", mw)), dim=int(_need(m, "dim", mw)),
                    vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)), diff=float(_need(m, "diff", mw)),
                    segment=int(_need(_need(m, "mask", mw), "size", mw + "mask.")))
            elif kind == "latent_attention":
                rot = _need(m, "rot", mw)
                mixer = LatentMixerConfig(
                    heads=int(_need(m, "heads", mw)), dim=int(_need(m, "dim", mw)), rot_dim=int(_need(m, "rot_dim", mw)),
                    vdim=int(_need(m, "vdim", mw)), q_rank=int(_need(m, "q_rank", mw)), kv_rank=int(_need(m, "kv_rank", mw)),
                    scale=float(_need(m, "scale", mw)), rot_base=float(_need(rot, "base", mw + "rot.")),
                    rot_dims=int(_need(rot, "dims", mw + "rot.")))
            else:
                raise NotImplementedError(f"{where}type {kind!r} is not a layer of this design "
                                          "('attention', 'latent_attention')")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if _need(mlp, "kind", where + "mlp.") != "dense":
                    raise NotImplementedError(f"{where}mlp.kind {mlp['kind']!r} is not a feed-forward of this design ('dense')")
                ff = int(_need(mlp, "ff", where + "mlp."))
            layers.append(PesoraxLayerConfig(kind, mixer, ff))
        loop = d.get("loop")
        if loop is None:
            loop_cfg = LoopConfig()
        else:
            loop_cfg = LoopConfig(int(_need(loop, "start", "loop.")), int(_need(loop, "stop", "loop.")), int(_need(loop, "times", "loop.")))
        cfg = cls(vocab=int(_need(d, "vocab", "")), width=int(_need(d, "width", "")),
                  eps=float(_need(_need(d, "norm", ""), "eps", "norm.")), residual_mult=float(_need(d, "residual_mult", "")),
                  loop=loop_cfg, layers=tuple(layers))
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab", "width"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if not self.eps > 0:
            raise ValueError("norm.eps must be positive")
        lp = self.loop
        if not (0 <= lp.start <= lp.stop <= len(self.layers)) or lp.times < 1:
            raise ValueError(f"loop {lp.start}..{lp.stop} x {lp.times} does not fit {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if layer.kind == "attention":
                if min(m.heads, m.kv_heads, m.dim, m.vdim, m.segment) <= 0:
                    raise ValueError(f"layers[{i}]: sizes must be positive")
                if m.heads % m.kv_heads:
                    raise ValueError(f"layers[{i}]: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
            else:
                if min(m.heads, m.dim, m.vdim, m.q_rank, m.kv_rank) <= 0 or m.rot_dim < 0:
                    raise ValueError(f"layers[{i}]: sizes must be positive")
                if m.rot_dims % 2 or not 0 <= m.rot_dims <= m.rot_dim:
                    raise ValueError(f"layers[{i}]: rot.dims {m.rot_dims} must be even and at most rot_dim {m.rot_dim}")
            if layer.ff is not None and layer.ff <= 0:
                raise ValueError(f"layers[{i}]: mlp.ff must be positive")

    def run_order(self) -> list:
        """(layer, does a pass after the first begin here) for every layer run, in order."""
        lp = self.loop
        order = [(i, False) for i in range(lp.start)]
        for rep in range(lp.times if lp.stop > lp.start else 0):
            order += [(i, rep > 0 and i == lp.start) for i in range(lp.start, lp.stop)]
        order += [(i, False) for i in range(lp.stop, len(self.layers))]
        return order


def build_spec(cfg: PesoraxConfig) -> ModelSpec:
    W = cfg.width
    norm = DynamicTanhSpec(size=W, delta_scale=cfg.residual_mult)
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.kind == "attention":
            mixer = DifferentialAttentionSpec(hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim,
                                              value_dim=m.vdim, scale=m.scale, lambda_init=m.diff, norm_eps=cfg.eps,
                                              segment=m.segment)
        else:
            mixer = LatentAttentionSpec(hidden_size=W, num_heads=m.heads, key_dim=m.dim, rope_dim=m.rot_dim, value_dim=m.vdim,
                                        q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, rope_base=m.rot_base,
                                        rotary_dims=m.rot_dims, norm_eps=cfg.eps)
        layers.append(LayerSpec(arrangement="prenorm", mixer=mixer, mixer_norm=norm,
                                feed_forward=DenseMLPSpec(W, layer.ff) if layer.ff is not None else None,
                                ffn_norm=norm if layer.ff is not None else None))
    spec = ModelSpec(
        architecture=NAME, vocab_size=cfg.vocab, hidden_size=W, layers=layers,
        run=[RunEntry(layer=i, add_input=again) for i, again in cfg.run_order()],
        final_norm=norm, tie_embeddings=False,
        embedding=TokenEmbeddingSpec(cfg.vocab, W), head=LinearHeadSpec(cfg.vocab, W),
        info={"layers": len(layers), "runs": len(cfg.run_order()), "hidden": W, "vocab": cfg.vocab,
              "kinds": [l.kind for l in cfg.layers], "ff": [l.ff for l in cfg.layers], "tied": False},
    )
    spec.validate()
    return spec


def weight_plan(cfg: PesoraxConfig, spec: ModelSpec) -> list[WeightTarget]:
    """Checkpoint names -> the model's parameters. Projections that read the same input are run
    as one product, so they are stacked along the output dimension: q, k, v of the two-map
    attention (and their biases); the two low-rank steps and the gate of the latent attention."""
    W = cfg.width
    plan = [WeightTarget("embed.weight", ("embed",), ((cfg.vocab, W),))]

    def norm(dst: str, src: str):
        return [WeightTarget(f"{dst}.weight", (src,), ((W,),)), WeightTarget(f"{dst}.bias", (f"{src}.b",), ((W,),)),
                WeightTarget(f"{dst}.alpha", (f"{src}.alpha",), ((),), transform=("as_vector",))]

    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}", f"layers.{i}"
        m, mix = layer.mixer, f"l{i}.mix"
        plan += norm(f"{dst}.mixer_norm", f"{src}.norm1")
        if layer.kind == "attention":
            nq, nk, nv = m.heads * 2 * m.dim, m.kv_heads * 2 * m.dim, m.kv_heads * m.vdim
            plan += [
                WeightTarget(f"{dst}.mixer.qkv_weight", (f"{mix}.q", f"{mix}.k", f"{mix}.v"), ((nq, W), (nk, W), (nv, W))),
                WeightTarget(f"{dst}.mixer.qkv_bias", (f"{mix}.q.b", f"{mix}.k.b", f"{mix}.v.b"), ((nq,), (nk,), (nv,))),
                WeightTarget(f"{dst}.mixer.out_weight", (f"{mix}.o",), ((W, m.heads * m.vdim),)),
            ]
            plan += [WeightTarget(f"{dst}.mixer.{n}", (f"{mix}.{n}",), ((m.dim,),)) for n in ("lq1", "lk1", "lq2", "lk2")]
        else:
            no = m.heads * m.vdim
            plan += [
                WeightTarget(f"{dst}.mixer.in_weight", (f"{mix}.dq", f"{mix}.dkv", f"{mix}.g"),
                             ((m.q_rank, W), (m.kv_rank + m.rot_dim, W), (no, W))),
                WeightTarget(f"{dst}.mixer.q_norm", (f"{mix}.dq.norm",), ((m.q_rank,),)),
                WeightTarget(f"{dst}.mixer.kv_norm", (f"{mix}.dkv.norm",), ((m.kv_rank,),)),
                WeightTarget(f"{dst}.mixer.q_up_weight", (f"{mix}.uq",), ((m.heads * (m.dim + m.rot_dim), m.q_rank),)),
                WeightTarget(f"{dst}.mixer.k_up_weight", (f"{mix}.uk",), ((m.heads * m.dim, m.kv_rank),)),
                WeightTarget(f"{dst}.mixer.v_up_weight", (f"{mix}.uv",), ((no, m.kv_rank),)),
                WeightTarget(f"{dst}.mixer.sink", (f"{mix}.sink",), ((m.heads,),)),
                WeightTarget(f"{dst}.mixer.out_weight", (f"{mix}.o",), ((W, no),)),
            ]
        if layer.ff is not None:
            plan += norm(f"{dst}.ffn_norm", f"{src}.norm2")
            plan += [WeightTarget(f"{dst}.feed_forward.up_weight", (f"{src}.mlp.up",), ((layer.ff, W),)),
                     WeightTarget(f"{dst}.feed_forward.down_weight", (f"{src}.mlp.down",), ((W, layer.ff),))]
    plan += norm("final_norm", "final.norm")
    plan.append(WeightTarget("lm_head.weight", ("head",), ((cfg.vocab, W),)))
    return plan


ARCHITECTURE = Architecture(name=NAME, parse_config=PesoraxConfig.from_dict, build_spec=build_spec, weight_plan=weight_plan)
register_architecture([NAME], ARCHITECTURE)
