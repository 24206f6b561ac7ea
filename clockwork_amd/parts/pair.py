"""Two mixers side by side on the same input (``PairMixerSpec``): the result is the mean of their
outputs, each RMS-normed over the model width with a weight of its own (one kernel, float32
statistics). Each mixer keeps its own cache: the pair states both needs as ``CacheNeeds`` and
hands each member of the entry's cache to the mixer it belongs to."""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import CacheNeeds, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.specs import PairMixerSpec
from clockwork_amd.registry import build_part


class PairMixer(Part):
    SIDES = ("left", "right")

    def __init__(self, spec: PairMixerSpec) -> None:
        self.spec = spec
        self.left, self.right = build_part(spec.left), build_part(spec.right)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(m, "graph_safe", False) for m in (self.left, self.right))

    def _sides(self):
        return zip(self.SIDES, (self.left, self.right))

    def param_specs(self):
        specs = {}
        for side, mixer in self._sides():
            for name, p in mixer.param_specs().items():
                specs[f"{side}.{name}"] = p
            specs[f"{side}_out_norm"] = ParamSpec((self.spec.hidden_size,), precision="float32", init=("one_plus_uniform", 0.1))
        return specs

    def cache_need(self):
        needs = [m.cache_need() for m in (self.left, self.right)]
        kept = [n for n in needs if n is not None]
        self._member_of = []  # per side: index into the entry cache's members, or None
        for n in needs:
            self._member_of.append(None if n is None else sum(1 for m in self._member_of if m is not None))
        return CacheNeeds(tuple(kept)) if kept else None

    def kernel_libraries(self) -> list:
        jobs = [("rowwise", None)]
        for m in (self.left, self.right):
            jobs += [j for j in getattr(m, "kernel_libraries", lambda: [])() if j not in jobs]
        return jobs

    def bind(self, params, device, dtype) -> None:
        for side, mixer in self._sides():
            prefix = side + "."
            mixer.bind({k[len(prefix):]: v for k, v in params.items() if k.startswith(prefix)}, device, dtype)
        self.left_norm, self.right_norm = params["left_out_norm"], params["right_out_norm"]
        if not hasattr(self, "_member_of"):
            self.cache_need()

    def prepare(self, ctx) -> None:
        for m in (self.left, self.right):
            prepare = getattr(m, "prepare", None)
            if prepare is not None:
                prepare(ctx)

    def shape_class(self, q_lens, ctx_lens):
        return tuple(getattr(m, "shape_class", lambda a, b: None)(q_lens, ctx_lens) for m in (self.left, self.right))

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        outs = []
        for mixer, member in zip((self.left, self.right), self._member_of):
            own = cache.members[member] if member is not None else EntryCache(writes=False)
            outs.append(mixer.forward(x, ctx, own))
        return ops.rms_mean2(outs[0], outs[1], self.left_norm, self.right_norm, self.spec.eps)
