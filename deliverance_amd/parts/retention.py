"""Retention as a mixer (``RetentionSpec``): linear attention with a fixed decay per head.

Per head a matrix S [head_dim, v_head_dim] is carried from token to token in 32-bit:

    S <- decay_h * S + k v^T
    o  = S^T q              (sees the token's own write)

q and k are projections of the input that are turned by the position (``spec.rotary``); k is then multiplied by
head_dim^-1/2.  There is no softmax and no denominator.  Each head's o is divided by its root mean square (no gain),
multiplied by the gate (SiLU of one more projection) and projected back.  A request's state is one 32-bit row
[ S: heads x v_head_dim x head_dim ]; the kernel finds it through ``ctx.state_slots`` on the device, so decode steps can
be recorded.

Products of a step: [q | k | v | gate] in the compute dtype (one product), and the output projection.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, StateNeed, StepContext, build_position, register_mixer, to_matrix


class Retention(Mixer):
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        E, H, D, Dv = spec.width, spec.n_heads, spec.head_dim, spec.v_head_dim
        self.H, self.D, self.Dv = H, D, Dv
        if not (1 <= D <= ops.RETENTION_MAX_DIM):
            raise ValueError(f"a key size of {D} is outside 1..{ops.RETENTION_MAX_DIM}")
        if len(spec.decay) != H:
            raise ValueError(f"{len(spec.decay)} decays for {H} heads")
        if spec.gate != "silu":
            raise ValueError(f"the gate of a retention mixer is 'silu', not {spec.gate!r}")
        self.eps = float(spec.norm_eps)
        self.qk_cols, self.v_cols = H * D, H * Dv

        def shaped(name, shape):
            t = params[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {list(t.shape)}, expected {list(shape)}")
            return t

        self.in_weight = to_matrix(torch.cat([shaped("q_weight", (self.qk_cols, E)), shaped("k_weight", (self.qk_cols, E)),
                                              shaped("v_weight", (self.v_cols, E)), shaped("gate_weight", (self.v_cols, E))], 0),
                                   dtype, device)
        self.out_weight = to_matrix(shaped("out_weight", (E, self.v_cols)), dtype, device)
        self.decay = torch.tensor([float(g) for g in spec.decay], dtype=torch.float32, device=device)
        self.k_scale = float(D) ** -0.5
        self.unit_gain = torch.ones(Dv, dtype=torch.float32, device=device)     # the read-out norm has no gain
        self.rotary = None if spec.rotary is None else build_position(spec.rotary, {}, dtype, device)
        if self.rotary is not None and self.rotary.dims > D:
            raise ValueError(f"{self.rotary.dims} turned entries, a head has {D}")
        self.v_off, self.gate_off = 2 * self.qk_cols, 2 * self.qk_cols + self.v_cols

    def cache_need(self):
        return StateNeed(self.H * self.Dv * self.D)

    normed_into = True

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor, call, into=None) -> bool:
        """Small steps: the root-mean-square norm in front and the one product in one kernel."""
        N = x.shape[0]
        rms = getattr(norm, "rms_params", lambda: None)()
        if rms is None or not ops.can_fuse_ln(N, x, self.in_weight):
            return False
        gain, offset, eps = rms
        proj = ctx.buf("retention_in", N, self.in_weight.shape[0], ctx.dtype)
        ops.linear_rms(x, None, N, gain, offset, eps, self.in_weight, None, proj)
        self._mix(ctx, proj, x if into is None else into, call)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        proj = ctx.buf("retention_in", h.shape[0], self.in_weight.shape[0], ctx.dtype)
        ops.linear(h, self.in_weight, None, proj)
        self._mix(ctx, proj, x, call)

    def _mix(self, ctx: StepContext, proj: torch.Tensor, x: torch.Tensor, call) -> None:
        N, H = proj.shape[0], self.H
        state = ctx.cache.state[call.cache]
        if self.rotary is not None and self.rotary.dims:
            qk = proj[:, :2 * self.qk_cols]                 # q and k are 2 H heads side by side: one launch, in place
            self.rotary.apply(ctx, qk, qk, 2 * H, self.D, self.D, self.D)
        o = ctx.buf("retention_o", N, self.v_cols, torch.float32)
        ops.retention(ctx, proj, 0, self.qk_cols, self.v_off, self.decay, self.k_scale, state, o, H, self.D, self.Dv,
                      write=call.write)
        y = ctx.buf("retention_y", N, self.v_cols, ctx.dtype)
        ops.delta_gate_norm(o, proj[:, self.gate_off:self.gate_off + self.v_cols], self.unit_gain, self.eps, "silu", H,
                            self.Dv, y)
        if ctx.debug_hook is not None:
            ctx.emit(call.layer, "attention_value", y)
        ops.linear(y, self.out_weight, None, x, accumulate=ctx.part_accumulate)


register_mixer("retention", Retention)
