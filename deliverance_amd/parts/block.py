"""The arrangement of one block: optional norms around a mixer and a feed-forward, each
adding into the 32-bit residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:161-200
(five optional norm places :26-32; GPT-2 uses the two pre-norms :35-41; a norm after a part acts
on the part's output before the residual add :172-176,184-188; the part's output may join the stream
times a constant :260-272; the fifth norm acts on the stream at the block's end :199)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import StepContext, build_feed_forward, build_mixer, build_norm, to_vector
from .norms import STREAM_ITSELF


class Block:
    def __init__(self, spec, params, dtype, device):
        def norm(s, key):
            return None if s is None else build_norm(s, params[key], dtype, device)

        self.pre_mixer_norm = norm(spec.pre_mixer_norm, "pre_mixer_norm")
        self.post_mixer_norm = norm(spec.post_mixer_norm, "post_mixer_norm")
        self.pre_ff_norm = norm(spec.pre_ff_norm, "pre_ff_norm")
        self.post_ff_norm = norm(spec.post_ff_norm, "post_ff_norm")
        self.post_block_norm = norm(getattr(spec, "post_block_norm", None), "post_block_norm")
        self.residual_multiplier = float(getattr(spec, "residual_multiplier", 1.0))
        # A learned scale per channel on a part's result ("layer scale").  Behind a norm that can take it into its
        # gain (``Norm.scaled_by``) it costs nothing; else it is applied while the result joins the stream.
        self.mixer_scale, self.post_mixer_norm = self._scale(spec, params, "mixer_scale", self.post_mixer_norm, dtype, device)
        self.ff_scale, self.post_ff_norm = self._scale(spec, params, "ff_scale", self.post_ff_norm, dtype, device)
        self.mixer = build_mixer(spec.mixer, params["mixer"], dtype, device)
        self.feed_forward = None if spec.feed_forward is None else \
            build_feed_forward(spec.feed_forward, params["feed_forward"], dtype, device)

    @staticmethod
    def _scale(spec, params, key, post, dtype, device):
        """(scale vector still to apply or None, the norm behind the part)."""
        if not getattr(spec, key, False):
            return None, post
        vec = params[key]
        fold = getattr(post, "scaled_by", None)
        if fold is not None:
            return None, fold(vec)
        return to_vector(vec, torch.float32, device), post

    @staticmethod
    def _normed(ctx, x, pre):
        if pre is not None:
            return pre.forward(ctx, x)
        h = ctx.buf("norm", x.shape[0], x.shape[1], ctx.dtype)      # no norm in front: the stream, converted
        return ops.copy_rows(x, h)

    def _part(self, ctx, x, pre, post, run, run_normed, part=None, h_ready=None, next_pre=None, scale=None):
        """One part of the block.  Parts add into the tensor they are given.  Without a norm behind
        the part (and without a multiplier) that tensor is the residual stream; else the part gets
        a buffer of its own (cleared by a fill kernel of the engine's, so that a recorded step
        holds no memset; a part with ``can_store`` stores into it instead and nothing is cleared), whose
        norm, kept in 32-bit, times the multiplier is then added to the stream.  ``h_ready``: the part's
        normalised input, when the norm behind the part before has already made it.  Returns the
        normalised input of the part that follows (``next_pre`` of the new stream) when the norm behind
        this part could make it in the same pass (``Norm.add_into``), else None."""
        target = x
        own = post is not None or self.residual_multiplier != 1.0 or scale is not None
        stores = own and getattr(part, "can_store", False)
        if own:
            target = ctx.buf("part_out", x.shape[0], x.shape[1], torch.float32)
            if not stores:
                ops.fill_zero(target)
        ctx.part_accumulate = not stores
        try:
            # A part may offer `forward_normed(ctx, norm, x, ..., into=None)`: it then applies the norm in
            # front of it itself (fused into its first product) and returns True, or returns False to
            # decline this step.  `into` is where its result goes when that is not the stream itself; a
            # part that declares `normed_into` takes it.
            if h_ready is not None:
                run(h_ready, target)
            elif not (pre is not None and run_normed is not None and (not own or getattr(part, "normed_into", False))
                      and run_normed(pre, target if own else None)):
                run(Block._normed(ctx, x, pre), target)
        finally:
            ctx.part_accumulate = True
        if own:
            add_into = None if post is None or self.residual_multiplier != 1.0 or scale is not None else \
                getattr(post, "add_into", None)
            if add_into is not None:         # norm, addition and the next part's norm in one pass over the rows
                return add_into(ctx, target, x, next_pre, next_name="norm_ahead")
            out = target if post is None else post.forward(ctx, target, out_name="post_norm", out_dtype=torch.float32)
            if scale is not None:
                ops.scale_add_rows(out, scale, x, self.residual_multiplier)
            else:
                ops.copy_rows(out, x, accumulate=True, scale=self.residual_multiplier)
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor, call) -> None:
        fused = getattr(self.mixer, "forward_normed", None)
        h_ff = self._part(ctx, x, self.pre_mixer_norm, self.post_mixer_norm,
                          lambda h, into: self.mixer.forward(ctx, h, into, call),
                          None if fused is None else (lambda norm, into: fused(ctx, norm, x, call) if into is None
                                                      else fused(ctx, norm, x, call, into=into)), part=self.mixer,
                          scale=self.mixer_scale,
                          next_pre=None if self.feed_forward is None or ctx.debug_hook is not None else
                          (self.pre_ff_norm if self.pre_ff_norm is not None else STREAM_ITSELF))
        if ctx.debug_hook is not None:
            ctx.emit(call.layer, "post_attention_residual", x)
        if self.feed_forward is not None:
            fused = getattr(self.feed_forward, "forward_normed", None)
            self._part(ctx, x, self.pre_ff_norm, self.post_ff_norm,
                       lambda h, into: self.feed_forward.forward(ctx, h, into),
                       None if fused is None else (lambda norm, into: fused(ctx, norm, x) if into is None
                                                   else fused(ctx, norm, x, into=into)), part=self.feed_forward,
                       h_ready=h_ff, scale=self.ff_scale)
            if ctx.debug_hook is not None:
                chosen = getattr(self.feed_forward, "last_choice", None)
                if chosen is not None:             # a routed feed-forward: the experts of every row, [N, top]
                    ctx.emit(call.layer, "expert_choice", chosen)
                ctx.emit(call.layer, "post_ff_residual", x)
        if self.post_block_norm is not None:                # the stream itself, normalised in place
            ops.copy_rows(self.post_block_norm.forward(ctx, x, out_name="post_norm", out_dtype=torch.float32), x)
