"""Mixers side by side: "parallel".

Several mixers read the same input rows and their results are added, each times a constant:

    y = sum over the branches b of scale_b * mixer_b(h)

A branch is any registered mixer kind (attention over pages beside a mixer with a fixed-size state, for
instance); its tensors lie under `<prefix>.<branch name>`.  The branches' results are added in float32,
in the order of the spec, and handed on as float32 rows (the block's norm adds them to the stream).
What the branches keep: at most one of them may keep pages and at most one a state, which become the
layer's own (`cache_need` / `state_need`); each branch gets the layer's cache and finds its part there.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import KVNeed, LayerCache, Mixer, StateNeed, StepContext, mixer_class, register_mixer


@register_mixer("parallel")
class ParallelMixers(Mixer):
    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.branches: List[Tuple[str, float, Mixer]] = []
        for name, scale, sub in spec["branches"]:
            self.branches.append((str(name), float(scale), mixer_class(sub.kind)(sub, dtype)))
        if not self.branches:
            raise ValueError("a parallel mixer needs at least one branch")
        if len({n for n, _, _ in self.branches}) != len(self.branches):
            raise ValueError("the branches of a parallel mixer need names of their own")
        if sum(1 for _, _, m in self.branches if m.cache_need() is not None) > 1:
            raise NotImplementedError("a parallel mixer with more than one branch that keeps pages")
        if sum(1 for _, _, m in self.branches if m.state_need() is not None) > 1:
            raise NotImplementedError("a parallel mixer with more than one branch that keeps a state")

    @property
    def graph_safe(self) -> bool:
        return all(m.graph_safe for _, _, m in self.branches)

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        out: List[TensorDecl] = []
        for name, _, sub in spec["branches"]:
            out += mixer_class(sub.kind).declare(sub, f"{prefix}.{name}")
        return out

    def load(self, store: WeightStore, prefix: str, device) -> None:
        for name, _, m in self.branches:
            m.load(store, f"{prefix}.{name}", device)

    def cache_need(self) -> Optional[KVNeed]:
        for _, _, m in self.branches:
            if m.cache_need() is not None:
                return m.cache_need()
        return None

    def state_need(self) -> Optional[StateNeed]:
        for _, _, m in self.branches:
            if m.state_need() is not None:
                return m.state_need()
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        total = None
        for _, scale, m in self.branches:
            y = m.forward(x, ctx, cache)
            total = kernels.scaled_sum(total, y, scale)
        return total
