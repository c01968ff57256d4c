"""Several mixers side by side (``ParallelMixerSpec``): every branch reads the same input, and the results are
added with a constant each.  A branch is any registered mixer; it keeps its cache or state in a slot of its own
(branch k of a layer call with slot c uses slot c + k), so pages, windows and state slots are managed for it as for
a mixer that stands alone.  Every branch stores its result in a 32-bit buffer, which then joins the target times the
branch's constant (the first one stores when the block asked the mixer to store)."""
from __future__ import annotations

import dataclasses

import torch

from ..kernels import ops
from .base import Mixer, StepContext, build_mixer, register_mixer


class ParallelMixer(Mixer):
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        if len(spec.branches) != len(spec.scales) or not spec.branches:
            raise ValueError(f"{len(spec.branches)} branches with {len(spec.scales)} constants")
        if len(params["branches"]) != len(spec.branches):
            raise ValueError(f"{len(spec.branches)} branches with parameters for {len(params['branches'])}")
        self.branches = [build_mixer(b, p, dtype, device) for b, p in zip(spec.branches, params["branches"])]
        self.scales = [float(s) for s in spec.scales]
        for b in self.branches:
            if isinstance(b.cache_need(), (tuple, list)):
                raise ValueError("a branch of a parallel mixer cannot itself be made of several mixers")

    @property
    def graph_safe(self) -> bool:
        return all(b.graph_safe for b in self.branches)

    def cache_need(self):
        return tuple(b.cache_need() for b in self.branches)

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        accumulate = ctx.part_accumulate
        for k, (branch, scale) in enumerate(zip(self.branches, self.scales)):
            sub = dataclasses.replace(call, cache=call.cache + k)
            if getattr(branch, "can_store", False):
                part = ctx.buf("branch_out", x.shape[0], x.shape[1], torch.float32)
                ctx.part_accumulate = False
            else:
                part = ops.fill_zero(ctx.buf("branch_out", x.shape[0], x.shape[1], torch.float32))
                ctx.part_accumulate = True
            try:
                branch.forward(ctx, h, part, sub)
            finally:
                ctx.part_accumulate = accumulate
            ops.copy_rows(part, x, accumulate=accumulate or k > 0, scale=scale)


register_mixer("parallel", ParallelMixer)
