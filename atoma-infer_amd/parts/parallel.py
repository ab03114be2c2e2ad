"""Mixers that run side by side on the same input: ``sum_i scale_i * branch_i(x)``.

A branch is any mixer; at most one of them may keep a paged cache and at most one a per-request state, which become
the cache and the state of the whole (a layer call owns one cache entry and one state).  The branches' outputs are
not added here: they go to the norm behind the mixer as a ``WeightedSum``, whose kernel scales and sums them in
float32 on its way.

With ``out_norms`` (an RMS norm per branch, over the model's width) the result is one tensor,
``sum_i scale_i * norm_i(branch_i(x) + bias_i)``, made by one kernel; ``bias_i`` is a branch's ``out_bias`` (the bias of
its output projection, which the branch leaves to whoever reads its output).  The norms' tensors lie below the
branches' prefixes (``<branch>.<norm's name>``).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

from .base import Mixer, WeightedSum, WeightSpec, register_mixer


class ParallelMixer(Mixer):
    def __init__(self, branches: Sequence[Mixer], scales: Sequence[float], names: Sequence[str], out_norms=None):
        if not (len(branches) == len(scales) == len(names)) or not 1 <= len(branches) <= 2:
            raise ValueError("one or two branches, each with a scale and a name")
        self.branches, self.scales, self.names = list(branches), [float(s) for s in scales], list(names)
        self.out_norms = list(out_norms) if out_norms is not None else None
        if self.out_norms is not None and (len(self.out_norms) != 2 or len(self.branches) != 2
                                           or self.scales[0] != self.scales[1]
                                           or self.out_norms[0].eps != self.out_norms[1].eps):
            raise ValueError("normed outputs: two branches with one scale, and a norm for each with one eps")
        if sum(b.cache_spec() is not None for b in self.branches) > 1:
            raise ValueError("at most one branch may keep a paged cache")
        if sum(b.state_spec() is not None for b in self.branches) > 1:
            raise ValueError("at most one branch may keep a state")

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {f"{n}.{k}": ws for n, b in zip(self.names, self.branches) for k, ws in b.weight_specs().items()}
        for n, norm in zip(self.names, self.out_norms or ()):
            specs.update({f"{n}.{k}": ws for k, ws in norm.weight_specs().items()})
        return specs

    def load(self, get, device, act_dtype) -> None:
        for n, b in zip(self.names, self.branches):
            b.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)
        for n, norm in zip(self.names, self.out_norms or ()):
            norm.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)

    def device_bytes(self) -> int:
        return sum(b.device_bytes() for b in self.branches)

    def graph_safe(self) -> bool:
        return all(b.graph_safe() for b in self.branches)

    def cache_spec(self):
        return next((b.cache_spec() for b in self.branches if b.cache_spec() is not None), None)

    def state_spec(self):
        return next((b.state_spec() for b in self.branches if b.state_spec() is not None), None)

    def step_planners(self, page_size: int, cache_dtype):
        """The planners of all branches: a list of (key, fn) as ``Mixer.step_planner`` gives one."""
        found = []
        for b in self.branches:
            plan = getattr(b, "step_planner", None)
            got = plan(page_size, cache_dtype) if plan is not None else None
            if got is not None:
                found.append(got)
        return found

    def step_planner(self, page_size: int, cache_dtype):
        found = self.step_planners(page_size, cache_dtype)
        return found[0] if found else None

    def forward(self, x, ctx, cache):
        outs = [b.forward(x, ctx, cache) for b in self.branches]
        if self.out_norms is None:
            return WeightedSum(list(zip(outs, self.scales)))
        from ..kernels import ops
        (na, nb), (a, b) = self.out_norms, self.branches
        return ops.normed_branches(outs[0], outs[1], na.weight_f32, nb.weight_f32, na.eps, self.scales[0],
                                   getattr(a, "out_bias", None), getattr(b, "out_bias", None))


register_mixer("parallel", ParallelMixer)
