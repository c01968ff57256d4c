"""A gated delta-rule mixer (``DeltaRuleSpec``).

Per value head a matrix S [head_dim, v_head_dim] is carried from token to token in 32-bit:

    S <- g * S              g in (0, 1): one number a head, or one a head and key channel (a row of S)
    u  = beta * (v - S^T k)
    S <- S + k u^T
    o  = S^T q              (sees the token's own write)

q, k (``n_kv_heads`` heads, shared by groups of value heads) and v are projections of the input that pass a short
causal filter per channel and SiLU; q and k are scaled to unit length per head inside the recurrence kernel, q also by
head_dim^-1/2.  beta = logistic(W_b h); g = exp(-exp(A_log) * softplus(a + dt_bias)), a = W_a h or W_a2 (W_a1 h).
o is divided by its root mean square per head, multiplied by a gain shared by the heads and by the gate (SiLU or the
logistic function of W_g h or W_g2 (W_g1 h)), then projected back.  What enters the recurrence besides the filtered
projections is 32-bit: beta and a before their functions (the products' unrounded sums), the decay, the unit norms,
the state.  A request's state is one 32-bit row [ S: heads x v_head_dim x head_dim | the filters' last taps - 1
inputs: (taps - 1) x (q | k | v channels) ]; kernels find it through ``ctx.state_slots`` on the device, so decode
steps can be recorded.

Products of a step: [q | k | v | gate or its low rank | the decay's low rank] in the compute dtype, [beta | decay] (or
beta alone) in 32-bit, the low-rank second factors, and the output projection.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, StateNeed, StepContext, register_mixer, to_matrix, to_vector


class GatedDeltaRule(Mixer):
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        E, H, G, D, Dv, K = spec.width, spec.n_heads, spec.n_kv_heads, spec.head_dim, spec.v_head_dim, spec.conv_taps
        self.H, self.G, self.D, self.Dv, self.taps = H, G, D, Dv, K
        if H % G != 0:
            raise ValueError(f"{H} value heads are not a multiple of {G} key heads")
        if not (1 <= K <= ops.CONV_MAX_TAPS):
            raise ValueError(f"a filter of {K} taps is outside 1..{ops.CONV_MAX_TAPS}")
        if not (1 <= D <= ops.DELTA_MAX_DIM):
            raise ValueError(f"a key size of {D} is outside 1..{ops.DELTA_MAX_DIM}")
        if spec.decay not in ("head", "channel") or spec.gate not in ("silu", "sigmoid"):
            raise ValueError(f"decay {spec.decay!r} / gate {spec.gate!r}: 'head' or 'channel', 'silu' or 'sigmoid'")
        self.channel_decay = spec.decay == "channel"
        self.gate_act = spec.gate
        self.eps, self.unit_eps = float(spec.norm_eps), float(spec.unit_eps)
        self.q_cols, self.v_cols = G * D, H * Dv
        self.conv_cols = 2 * self.q_cols + self.v_cols
        decay_cols = H * D if self.channel_decay else H

        def shaped(name, shape):
            t = params[name]
            if t.dim() != len(shape) or any(e not in (-1, f) for e, f in zip(shape, t.shape)):
                raise ValueError(f"{name} is {list(t.shape)}, expected {list(shape)}")
            return t

        # a low rank that the spec leaves open (-1) is whatever the two matrices share
        low_decay, low_gate = spec.decay_rank != 0, spec.gate_rank != 0
        first = [shaped("q_weight", (self.q_cols, E)), shaped("k_weight", (self.q_cols, E)), shaped("v_weight", (self.v_cols, E))]
        if low_gate:
            g_down = shaped("gate_down", (spec.gate_rank, E))
            self.gate_rank = g_down.shape[0]
            self.gate_up = to_matrix(shaped("gate_up", (self.v_cols, self.gate_rank)), dtype, device)
            first.append(g_down)
        else:
            self.gate_rank, self.gate_up = 0, None
            first.append(shaped("gate_weight", (self.v_cols, E)))
        self.gate_off = self.conv_cols
        self.decay_off = self.gate_off + (self.gate_rank or self.v_cols)
        second = [shaped("beta_weight", (H, E))]
        if low_decay:
            a_down = shaped("decay_down", (spec.decay_rank, E))
            self.decay_rank = a_down.shape[0]
            self.decay_up = to_matrix(shaped("decay_up", (decay_cols, self.decay_rank)), dtype, device)
            first.append(a_down)
        else:
            self.decay_rank, self.decay_up = 0, None
            second.append(shaped("decay_weight", (decay_cols, E)))
        self.in_weight = to_matrix(torch.cat(first, 0), dtype, device)          # -> the compute dtype
        self.raw_weight = to_matrix(torch.cat(second, 0), dtype, device)        # -> 32-bit sums
        self.decay_cols = decay_cols
        self.conv_weight = to_vector(torch.cat([shaped("q_conv", (self.q_cols, K)), shaped("k_conv", (self.q_cols, K)),
                                                shaped("v_conv", (self.v_cols, K))], 0), dtype, device)
        # exp(A_log) and the step bias in 32-bit
        self.rate = torch.exp(shaped("a_log", (H,)).to(device=device, dtype=torch.float32)).contiguous()
        self.dt_bias = shaped("dt_bias", (decay_cols,)).to(device=device, dtype=torch.float32).contiguous()
        self.out_norm = to_vector(shaped("out_norm", (Dv,)), dtype, device)
        self.out_weight = to_matrix(shaped("out_weight", (E, self.v_cols)), dtype, device)
        self.s_elems = H * Dv * D
        self.conv_off = self.s_elems                 # where the filters' inputs start in a state row

    def cache_need(self):
        return StateNeed(self.s_elems + (self.taps - 1) * self.conv_cols)

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        N, H = h.shape[0], self.H
        state = ctx.cache.state[call.cache]
        proj = ctx.buf("delta_in", N, self.in_weight.shape[0], ctx.dtype)
        ops.linear(h, self.in_weight, None, proj)
        raw = ctx.buf("delta_raw", N, self.raw_weight.shape[0], torch.float32)      # [beta | decay], unrounded
        ops.linear(h, self.raw_weight, None, raw)
        if self.decay_up is not None:
            a = ctx.buf("delta_decay", N, self.decay_cols, torch.float32)
            ops.linear(proj[:, self.decay_off:self.decay_off + self.decay_rank], self.decay_up, None, a)
            a_off = 0
        else:
            a, a_off = raw, H
        if self.gate_up is not None:
            gate = ctx.buf("delta_gate", N, self.v_cols, ctx.dtype)
            ops.linear(proj[:, self.gate_off:self.gate_off + self.gate_rank], self.gate_up, None, gate)
        else:
            gate = proj[:, self.gate_off:self.gate_off + self.v_cols]
        qkv = ctx.buf("delta_qkv", N, self.conv_cols, ctx.dtype)
        ops.conv_causal(ctx, proj[:, :self.conv_cols], state, self.conv_off, self.conv_weight, None, "silu", qkv)
        if call.write:
            ops.conv_state_update(ctx, proj[:, :self.conv_cols], state, self.conv_off, self.conv_cols, self.taps)
        o = ctx.buf("delta_o", N, self.v_cols, torch.float32)
        ops.delta_rule(ctx, qkv, self.q_cols, 2 * self.q_cols, raw, a, self.dt_bias, self.rate, state, o,
                       H, self.G, self.D, self.Dv, self.channel_decay, self.unit_eps, write=call.write, decay_off=a_off)
        y = ctx.buf("delta_y", N, self.v_cols, ctx.dtype)
        ops.delta_gate_norm(o, gate, self.out_norm, self.eps, self.gate_act, H, self.Dv, y)
        ops.linear(y, self.out_weight, None, x, accumulate=ctx.part_accumulate)


register_mixer("delta_rule", GatedDeltaRule)
