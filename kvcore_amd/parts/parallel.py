"""Several mixers side by side on the same input.

``ParallelMixer`` runs its branches on the same rows; each branch's output is divided by its
root mean square over the model width (eps inside the root) and multiplied by a gain of its
own, and the result is the mean of the branches.  A branch is any registered mixer: its cache
need and its per-request states become the composite's (at most one branch may keep a paged
cache, since a schedule entry names one cache).
"""

from __future__ import annotations

from dataclasses import replace

import torch

from kvcore_amd.ops import library as ops

from .base import MIXERS, CacheNeed, Mixer, ParamSource, ParamSpec, PartSpec, StateNeed, register_mixer


class ParallelMixer(Mixer):
    """``branches``: ``(name, PartSpec)`` pairs; a branch's tensors live under ``name.`` and its
    output gain is the tensor ``name + gain_suffix``."""

    def __init__(self, *, hidden_size: int, eps: float, branches: tuple[tuple[str, PartSpec], ...],
                 gain_suffix: str = ".out", position=None) -> None:
        if not 1 <= len(branches) <= 4:
            raise ValueError("one to four branches")
        self.hidden_size = hidden_size
        self.eps = eps
        self.gain_suffix = gain_suffix
        self.names = [name for name, _ in branches]
        self.branches: list[Mixer] = []
        for _, spec in branches:
            args = dict(spec.args)
            args["float32_result"] = True  # the branch norm reads the products' float32 sums
            self.branches.append(MIXERS.build(PartSpec(spec.kind, args), position=position))
        if sum(b.cache_need() is not None for b in self.branches) > 1:
            raise ValueError("at most one branch of a parallel mixer may keep a paged cache")

    @property
    def graph_safe(self) -> bool:
        return all(getattr(b, "graph_safe", True) for b in self.branches)

    def setup(self, runtime) -> None:
        super().setup(runtime)
        for b in self.branches:
            b.setup(runtime)

    def check_limits(self, limits) -> None:
        for b in self.branches:
            b.check_limits(limits)

    def param_specs(self) -> list[ParamSpec]:
        specs = []
        for name, branch in zip(self.names, self.branches):
            for ps in branch.param_specs():
                sources = tuple(ParamSource(f"{name}.{s.name}" if s.name else name, s.row, s.rows)
                                for s in ps.resolved_sources())
                specs.append(replace(ps, name=f"{name}.{ps.name}", sources=sources))
        for name in self.names:
            specs.append(ParamSpec(f"{name}.branch_gain", (self.hidden_size,), kind="vector", init="gain",
                                   sources=(ParamSource(name + self.gain_suffix, 0, self.hidden_size),)))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return tuple(f"{name}.{w}" for name, b in zip(self.names, self.branches) for w in b.product_weights())

    def bind(self, params: dict[str, torch.Tensor]) -> None:
        super().bind(params)
        for name, branch in zip(self.names, self.branches):
            head = name + "."
            branch.bind({k[len(head):]: v for k, v in params.items()
                         if k.startswith(head) and k != f"{name}.branch_gain"})

    def cache_need(self) -> CacheNeed | None:
        return next((n for n in (b.cache_need() for b in self.branches) if n is not None), None)

    def state_needs(self) -> tuple[StateNeed, ...]:
        return tuple(n for b in self.branches for n in b.state_needs())

    def forward(self, x, ctx, call, sink=None):
        outs = []
        at = 0
        for name, branch in zip(self.names, self.branches):
            n = len(branch.state_needs())
            own = call.state_indices[at: at + n]
            at += n
            sub = replace(call, state_index=own[0] if own else None, state_indices=tuple(own))
            y = branch.forward(x, ctx, sub)
            if y.dtype != torch.float32:
                raise RuntimeError(f"branch {name!r} must hand over float32 rows")
            # the mean reads all branches at the end: two branches of one kind, which write
            # the same step buffer, are told apart by a copy
            if any(prev.data_ptr() == y.data_ptr() for prev, _ in outs):
                keep = ctx.buf(f"parallel_branch_{len(outs)}", self.hidden_size, torch.float32)
                keep.copy_(y)
                y = keep
            outs.append((y, self.params[f"{name}.branch_gain"]))
        out = ctx.buf("mixer_out", self.hidden_size)
        ops.rms_branches_mean(out, outs, self.eps)
        return out


register_mixer("parallel", ParallelMixer)
