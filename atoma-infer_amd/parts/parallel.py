"""Mixers that run side by side on the same input: ``sum_i scale_i * branch_i(x)``.

A branch is any mixer; at most one of them may keep a paged cache and at most one a per-request state, which become
the cache and the state of the whole (a layer call owns one cache entry and one state).  The branches' outputs are
not added here: they go to the norm behind the mixer as a ``WeightedSum``, whose kernel scales and sums them in
float32 on its way.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

from .base import Mixer, WeightedSum, WeightSpec, register_mixer


class ParallelMixer(Mixer):
    def __init__(self, branches: Sequence[Mixer], scales: Sequence[float], names: Sequence[str]):
        if not (len(branches) == len(scales) == len(names)) or not 1 <= len(branches) <= 2:
            raise ValueError("one or two branches, each with a scale and a name")
        self.branches, self.scales, self.names = list(branches), [float(s) for s in scales], list(names)
        if sum(b.cache_spec() is not None for b in self.branches) > 1:
            raise ValueError("at most one branch may keep a paged cache")
        if sum(b.state_spec() is not None for b in self.branches) > 1:
            raise ValueError("at most one branch may keep a state")

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {f"{n}.{k}": ws for n, b in zip(self.names, self.branches) for k, ws in b.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        for n, b in zip(self.names, self.branches):
            b.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)

    def device_bytes(self) -> int:
        return sum(b.device_bytes() for b in self.branches)

    def graph_safe(self) -> bool:
        return all(b.graph_safe() for b in self.branches)

    def cache_spec(self):
        return next((b.cache_spec() for b in self.branches if b.cache_spec() is not None), None)

    def state_spec(self):
        return next((b.state_spec() for b in self.branches if b.state_spec() is not None), None)

    def step_planner(self, page_size: int, cache_dtype):
        for b in self.branches:
            plan = getattr(b, "step_planner", None)
            got = plan(page_size, cache_dtype) if plan is not None else None
            if got is not None:
                return got
        return None

    def forward(self, x, ctx, cache) -> WeightedSum:
        return WeightedSum([(b.forward(x, ctx, cache), s) for b, s in zip(self.branches, self.scales)])


register_mixer("parallel", ParallelMixer)
