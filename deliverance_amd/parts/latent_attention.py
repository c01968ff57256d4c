"""Attention over one narrow vector a token, as a mixer (``LatentAttentionSpec``).

Optional: a window (``spec.window``: position i sees j when 0 <= i - j < window), and a learned number per head whose
exponential joins the softmax's denominator without a key or a value (``spec.sink``).

What a token leaves in the cache is the normalised latent c (``kv_rank`` entries) and one key piece turned by
its position (``rot_dim`` entries); every head's keys and values are linear maps of c.  The maps are never
applied to cached rows: a head's key map is folded into its query (q'_h = [Wk_h^T q_h | turned q_h], so that
q'_h . [c | piece] is the head's score), and its value map is applied to the weighted sum of the c rows.  All
heads therefore read the same rows, once as keys and once (their first ``kv_rank`` entries) as values.

One step: down-projection [query latent | c | piece] (32-bit result); both norms, the turn of the piece, the cache
write and the normalised query latent in one kernel; the queries' up-projection; per head the fold and the turn
into q'; attention; per head the value map; the output projection added into the stream.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import KVNeed, Mixer, StepContext, build_position, register_mixer, to_matrix, to_vector


class LatentAttention(Mixer):
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        E = spec.width
        self.n_heads, self.dn, self.dr, self.dv = spec.n_heads, spec.head_dim, spec.rot_dim, spec.v_head_dim
        self.q_rank, self.kv_rank = spec.q_rank, spec.kv_rank
        self.row_dim = self.kv_rank + self.dr               # what a token's cache row holds
        self.scale, self.eps, self.window = float(spec.scale), float(spec.norm_eps), spec.window
        if not (1 <= self.row_dim <= ops.LATENT_MAX_ROW):
            raise ValueError(f"a cache row of {self.row_dim} entries is outside 1..{ops.LATENT_MAX_ROW}")
        H, qd = self.n_heads, self.dn + self.dr

        def shaped(name, shape):
            t = params[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {list(t.shape)}, expected {list(shape)}")
            return t

        # one matrix for both down-projections: rows [query latent | c | key piece]
        self.down_weight = to_matrix(torch.cat([shaped("q_down_weight", (self.q_rank, E)),
                                                shaped("kv_down_weight", (self.row_dim, E))], dim=0), dtype, device)
        self.q_gain = to_vector(shaped("q_norm_weight", (self.q_rank,)), dtype, device)
        self.kv_gain = to_vector(shaped("kv_norm_weight", (self.kv_rank,)), dtype, device)
        self.q_up_weight = to_matrix(shaped("q_up_weight", (H * qd, self.q_rank)), dtype, device)
        # head h's key map transposed, [kv_rank, dn]: applied to the head's unrotated query entries
        k_up = shaped("k_up_weight", (H * self.dn, self.kv_rank)).reshape(H, self.dn, self.kv_rank)
        self.k_fold = to_matrix(k_up.transpose(1, 2).contiguous(), dtype, device)              # [H, kv_rank, dn]
        self.v_up = to_matrix(shaped("v_up_weight", (H * self.dv, self.kv_rank)).reshape(H, self.dv, self.kv_rank),
                              dtype, device)                                                     # [H, dv, kv_rank]
        self.out_weight = to_matrix(shaped("out_weight", (E, H * self.dv)), dtype, device)
        # exp(sink_h) in the softmax's denominator: 32-bit, one a head
        self.sink = None
        if getattr(spec, "sink", False):
            self.sink = shaped("sink", (H,)).to(device=device, dtype=torch.float32).contiguous()
        self.rotary = build_position(spec.rotary, {}, dtype, device)
        if self.rotary.dims > self.dr:
            raise ValueError(f"{self.rotary.dims} turned entries, the rotated piece has {self.dr}")

    def cache_need(self):
        return KVNeed(1, self.row_dim, self.window, self.kv_rank, values_in_keys=True)

    normed_into = True

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor, call, into=None) -> bool:
        """Small steps: the root-mean-square norm in front and the down-projection in one kernel."""
        N = x.shape[0]
        rms = getattr(norm, "rms_params", lambda: None)()
        if rms is None or not ops.can_fuse_ln(N, x, self.down_weight):
            return False
        gain, offset, eps = rms
        down = ctx.buf("latent_down", N, self.q_rank + self.row_dim, torch.float32)
        ops.linear_rms(x, None, N, gain, offset, eps, self.down_weight, None, down)
        self._attend(ctx, down, x if into is None else into, call)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        down = ctx.buf("latent_down", h.shape[0], self.q_rank + self.row_dim, torch.float32)
        ops.linear(h, self.down_weight, None, down)
        self._attend(ctx, down, x, call)

    def _attend(self, ctx: StepContext, down: torch.Tensor, x: torch.Tensor, call) -> None:
        N, H = down.shape[0], self.n_heads
        qd = self.dn + self.dr
        slot = ctx.cache.kv[call.cache]
        group = ctx.group_of(call.cache)
        cq = ctx.buf("latent_cq", N, self.q_rank, ctx.dtype)
        ops.latent_prepare(down, self.q_rank, self.kv_rank, self.dr, self.q_gain, self.kv_gain, self.eps, ctx.positions,
                           ctx.slot_maps[group] if call.write else None, self.rotary.speeds, self.rotary.dims,
                           self.rotary.interleaved, cq, slot, ctx.cache.page_size, magnitude=self.rotary.magnitude)
        q = ctx.buf("latent_q", N, H * qd, ctx.dtype)
        ops.linear(cq, self.q_up_weight, None, q)
        # q'_h = [Wk_h^T q_h[:dn] | turned q_h[dn:]]
        qf = ctx.buf("latent_q_folded", N, H * self.row_dim, ctx.dtype)
        ops.linear_heads(q, qd, 0, self.k_fold, qf, self.row_dim, 0)
        self.rotary.apply(ctx, q[:, self.dn:], qf[:, self.kv_rank:], H, qd, self.row_dim, self.dr)
        mix = ctx.buf("latent_mix", N, H * self.kv_rank, ctx.dtype)
        ops.paged_attention_latent(ctx, qf, slot, group, H, self.row_dim, self.kv_rank, self.scale, self.window, mix,
                                   sink=self.sink)
        o = ctx.buf("attn_out", N, H * self.dv, ctx.dtype)
        ops.linear_heads(mix, self.kv_rank, 0, self.v_up, o, self.dv, 0)
        if ctx.debug_hook is not None:
            ctx.emit(call.layer, "query_projection", q)
            ctx.emit(call.layer, "attention_value", o)
        ops.linear(o, self.out_weight, None, x, accumulate=ctx.part_accumulate)


register_mixer("latent_attention", LatentAttention)
