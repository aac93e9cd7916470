"""Two mixers side by side: both read the same input, and the layer's mixer output is a weighted sum
of theirs.

``parallel``: ``out = left_scale * left(h) + right_scale * right(h)``.  The two are any registered
mixers, named by :class:`PartSpec` like a layer's own mixer, with their tensors under ``left.`` and
``right.`` below this part's prefix.  At most one of them may keep a cache of tokens; what they keep
per request lies side by side in the layer's state slot, each seeing its own columns only.  Where
both offer the product they apply to the input first (``input_linear`` / ``forward_projected``), the two
products are fused into one over the shared input and each mixer is handed its columns.
"""
from __future__ import annotations

import dataclasses

from tensorline_amd.ops import kernels
import torch

from tensorline_amd.parts.base import Part, TensorGetter, fuse_linears
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
        self.fused = None                 # the two input products as one, where both mixers offer theirs
        self._split = 0

    def tensors(self):
        out = {}
        for m in self.sides:
            out.update(m.tensors())
        return out

    def load(self, get: TensorGetter) -> None:
        for m in self.sides:
            m.load(get)
        self.fused = None
        if all(hasattr(m, "input_linear") and hasattr(m, "forward_projected") for m in self.sides):
            firsts = [m.input_linear() for m in self.sides]
            self.fused = fuse_linears(self.prefix + "in", firsts)
            self._split = firsts[0].out_features
            for lin in firsts:            # the fused copy is the one that is kept
                lin.weight = lin.bias = lin.shuffled = lin.shuffled_float = None

    def weight_tensors(self):
        return (self.fused.tensors_kept() if self.fused is not None else []) + [t for m in self.sides for t in m.weight_tensors()]

    def library_products(self):
        own = [(self.fused.weight, torch.float32)] if self.fused is not None else []
        return own + [p for m in self.sides for p in m.library_products()]

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
        proj = self.fused(h, out_dtype=torch.float32) if self.fused is not None else None
        for i, (m, span) in enumerate(zip(self.sides, self._state_spans)):
            mine = cache
            if cache.state is not None and span is not None and (span[0] or span[1] != cache.state.shape[1]):
                mine = dataclasses.replace(cache, state=cache.state[:, span[0]:span[1]])
            if proj is not None:
                outs.append(m.forward_projected(proj[:, :self._split] if i == 0 else proj[:, self._split:], ctx, mine))
            else:
                outs.append(m.forward(h, ctx, mine))
        return kernels.scaled_sum(outs[0], outs[1], self.scales[0], self.scales[1])
