"""Mixers side by side: every branch reads the same rows, and the result is the mean of the
branches' outputs, each first RMS-normed over the model's width with a weight of its own:

    out = (1 / n) sum_b rmsnorm(branch_b(x)) * w_b          (float32)

The branches are mixers of any registered kind (`spec.branches`); branch b's parameters are
prefixed `spec.names[b]`, its output norm's weight is `<name>_out.weight`, and what it asks of
the cache is found under the cache id `(id, name)` of the layer's entry.  Kernel:
`norm_mean` of `csrc/norms.hip`.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .registry import lookup


@dataclass(frozen=True)
class BranchEntry:
    """A branch's view of the layer's schedule entry: its own part of the cache entry."""
    layer: int
    cache: object
    writes_cache: bool
    own_id: object


class ParallelMixer:
    @classmethod
    def _branches(cls, spec):
        if not spec.branches or len(spec.branches) != len(spec.names) or len(spec.branches) > 4 \
                or len(set(spec.names)) != len(spec.names):
            raise ValueError("parallel: 1 to 4 branches, each with a name of its own")
        if len({branch.kind for branch in spec.branches}) != len(spec.branches):
            # (parts of one kind name their workspace buffers alike)
            raise ValueError("parallel: the branches must be mixers of different kinds")
        return [(name, lookup("mixer", branch.kind), branch)
                for name, branch in zip(spec.names, spec.branches)]

    @classmethod
    def parameters(cls, spec, hidden):
        params = {}
        for name, owner, branch in cls._branches(spec):
            for inner, param in owner.parameters(branch, hidden).items():
                params[f"{name}.{inner}"] = param
            params[f"{name}_out.weight"] = ParamSpec((hidden,), init="norm")
        return params

    @classmethod
    def cache_request(cls, spec):
        wanted = {name: owner.cache_request(branch) for name, owner, branch in cls._branches(spec)}
        return {name: request for name, request in wanted.items() if request is not None} or None

    @classmethod
    def own_cache_request(cls, spec):
        wanted = {}
        for name, owner, branch in cls._branches(spec):
            ask = getattr(owner, "own_cache_request", None)
            request = None if ask is None else ask(branch)
            if request is not None:
                wanted[name] = request
        return wanted or None

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        names = ["norms"]
        for _, owner, branch in cls._branches(spec):
            ask = getattr(owner, "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(branch, dtype))
        return tuple(names)

    def __init__(self, spec, hidden, params, dtype, device, positions=None):
        self.spec = spec
        self.hidden = hidden
        self.names = tuple(spec.names)
        self.branches = []
        self.out_norms = []
        for name, owner, branch in self._branches(spec):
            own = {key[len(name) + 1:]: tensor for key, tensor in params.items()
                   if key.startswith(name + ".")}
            self.branches.append(owner(branch, hidden, own, dtype, device, positions=positions))
            self.out_norms.append(params[f"{name}_out.weight"].to(
                device=device, dtype=torch.float32).contiguous())

    def members(self):
        return tuple(self.branches)

    @property
    def capture_safe(self):
        return all(bool(getattr(branch, "capture_safe", False)) for branch in self.branches)

    @property
    def capture_rows(self):
        return min(getattr(branch, "capture_rows", 1 << 30) for branch in self.branches)

    @property
    def plan_key(self):
        return ("parallel", tuple(getattr(branch, "plan_key", id(branch))
                                  for branch in self.branches))

    def plan_step(self, plan):
        sections = {}
        for branch in self.branches:
            if hasattr(branch, "plan_step"):
                sections.update(branch.plan_step(plan))
        return sections

    def forward(self, ctx, x, entry):
        outputs = []
        for name, branch in zip(self.names, self.branches):
            outputs.append(branch.forward(ctx, x, BranchEntry(
                layer=entry.layer, cache=(entry.cache, name), writes_cache=entry.writes_cache,
                own_id=(entry.own_id, name))))
        out = ctx.buffer("parallel.out", (x.shape[0], self.hidden), torch.float32)
        lib.norm_mean(outputs, self.out_norms, self.spec.norm_eps, out)
        ctx.release(*outputs)
        return out
