"""Two mixers side by side: both read the same input, and the layer's mixer output is a weighted sum
of theirs.

``parallel``: ``out = left_scale * left(h) + right_scale * right(h)``.  The two are any registered
mixers, named by :class:`PartSpec` like a layer's own mixer, with their tensors under ``left.`` and
``right.`` below this part's prefix.  At most one of them may keep a cache of tokens; what they keep
per request lies side by side in the layer's state slot, each seeing its own columns only.
"""
from __future__ import annotations

import dataclasses

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Part, TensorGetter
from tensorline_amd.parts.registry import build_part, register_mixer
from tensorline_amd.parts.spec import PartSpec, StateNeed


@register_mixer("parallel")
class ParallelMixers(Part):
    def __init__(self, hidden_size, prefix, dtype, device, left: PartSpec, right: PartSpec, left_scale: float = 1.0,
                 right_scale: float = 1.0):
        super().__init__(hidden_size, prefix, dtype, device)
        common = dict(hidden_size=hidden_size, dtype=dtype, device=device)
        self.sides = [build_part("mixer", left, layer_prefix=prefix, **common),
                      build_part("mixer", right, layer_prefix=prefix, **common)]
        self.scales = (float(left_scale), float(right_scale))
        needs = [getattr(m, "cache_need", lambda: None)() for m in self.sides]
        if all(n is not None for n in needs):
            raise ValueError(f"{prefix}: both mixers keep a cache of tokens; a layer has one")
        self._cache_need = needs[0] if needs[0] is not None else needs[1]
        self._state_needs = [getattr(m, "state_need", lambda: None)() for m in self.sides]
        for n in self._state_needs:
            if n is not None and (len(n.shape) != 1 or n.dtype != "float32"):
                raise ValueError(f"{prefix}: states kept side by side are flat float32 vectors")
        self._state_spans, at = [], 0
        for n in self._state_needs:
            self._state_spans.append(None if n is None else (at, at + n.shape[0]))
            at += 0 if n is None else n.shape[0]
        self._state_size = at

    def tensors(self):
        out = {}
        for m in self.sides:
            out.update(m.tensors())
        return out

    def load(self, get: TensorGetter) -> None:
        for m in self.sides:
            m.load(get)

    def weight_tensors(self):
        return [t for m in self.sides for t in m.weight_tensors()]

    def library_products(self):
        return [p for m in self.sides for p in m.library_products()]

    def cache_need(self):
        return self._cache_need

    def state_need(self):
        return StateNeed((self._state_size,), "float32") if self._state_size else None

    @property
    def step_vectors_key(self):
        return tuple(getattr(m, "step_vectors_key", type(m)) for m in self.sides)

    def step_vectors(self, facts) -> dict:
        out: dict = {}
        for m in self.sides:
            if hasattr(m, "step_vectors"):
                out.update(m.step_vectors(facts))
        return out

    def forward(self, h, ctx, cache):
        outs = []
        for m, span in zip(self.sides, self._state_spans):
            mine = cache
            if cache.state is not None and span is not None and (span[0] or span[1] != cache.state.shape[1]):
                mine = dataclasses.replace(cache, state=cache.state[:, span[0]:span[1]])
            outs.append(m.forward(h, ctx, mine))
        return kernels.scaled_sum(outs[0], outs[1], self.scales[0], self.scales[1])
