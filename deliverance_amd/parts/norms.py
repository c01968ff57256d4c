"""LayerNorm as a part.  Formula: core/src/main/java/io/teknek/deliverance/generator/
LayerNorm.java:127-150 (mean, biased variance, eps inside the root, gain and bias)."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Norm, StepContext, register_norm, to_vector


class LayerNorm(Norm):
    def __init__(self, spec, params, dtype, device):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.weight = to_vector(params["weight"], dtype, device)
        self.bias = to_vector(params.get("bias"), dtype, device) if spec.bias else None
        if self.weight.numel() != self.width:
            raise ValueError(f"LayerNorm gain has {self.weight.numel()} entries for width {self.width}")

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, out_name: str = "norm",
                out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        R = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.buf(out_name, R, self.width, out_dtype or ctx.dtype)
        return ops.layernorm(x, self.weight, self.bias, self.eps, out, rows)

    def fusable_params(self):
        return self.weight, self.bias, self.eps


register_norm("layernorm", LayerNorm)


# Handed to ``add_into`` in place of the next part's norm when that part has none in front of it.
STREAM_ITSELF = object()


class RmsNorm(Norm):
    """The row divided by its root mean square (eps inside the root), times ``gain_offset + weight``; all in
    32-bit.  Behind a part it can do three things in one pass over the row (``add_into``): normalise the
    part's output, add it to the residual stream, and normalise the new stream for the part that follows."""

    def __init__(self, spec, params, dtype, device):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.gain_offset = float(getattr(spec, "gain_offset", 0.0))
        self.weight = to_vector(params["weight"], dtype, device)
        if self.weight.numel() != self.width:
            raise ValueError(f"RMS norm gain has {self.weight.numel()} entries for width {self.width}")

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, out_name: str = "norm",
                out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        R = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.buf(out_name, R, self.width, out_dtype or ctx.dtype)
        return ops.rmsnorm(x, self.weight, self.gain_offset, self.eps, out, rows)

    def scaled_by(self, scale: torch.Tensor) -> "RmsNorm":
        """This norm followed by a multiplication with ``scale``, element by element, as one norm: its gain is
        (gain_offset + weight) * scale, worked out once in 32-bit."""
        import copy
        if scale.numel() != self.width:
            raise ValueError(f"a scale of {scale.numel()} entries behind a norm of width {self.width}")
        out = copy.copy(self)
        out.weight = ((self.weight.to(torch.float32) + self.gain_offset)
                      * scale.to(device=self.weight.device, dtype=torch.float32).reshape(-1)).contiguous()
        out.gain_offset = 0.0
        return out

    def rms_params(self):
        """(gain, gain_offset, eps): for kernels that apply this norm to their own rows."""
        return self.weight, self.gain_offset, self.eps

    def add_into(self, ctx: StepContext, src: torch.Tensor, x: torch.Tensor, next_norm=None,
                 next_name: str = "norm") -> Optional[torch.Tensor]:
        """x += norm(src).  With ``next_norm`` (an RMS norm of the same eps and offset) also returns
        ``next_norm(x)`` of the new x in the compute dtype; returns None when it did not do that."""
        if next_norm is STREAM_ITSELF:             # the next part reads the stream without a norm: its copy, converted
            h = ctx.buf(next_name, x.shape[0], self.width, ctx.dtype)
            ops.rmsnorm_add(src, self.weight, x, self.gain_offset, self.eps, None, h)
            return h
        nxt = next_norm if (type(next_norm) is RmsNorm and next_norm.eps == self.eps
                            and next_norm.gain_offset == self.gain_offset and next_norm.width == self.width) else None
        if nxt is None:
            ops.rmsnorm_add(src, self.weight, x, self.gain_offset, self.eps)
            return None
        h = ctx.buf(next_name, x.shape[0], self.width, ctx.dtype)
        ops.rmsnorm_add(src, self.weight, x, self.gain_offset, self.eps, nxt.weight, h)
        return h


register_norm("rmsnorm", RmsNorm)
