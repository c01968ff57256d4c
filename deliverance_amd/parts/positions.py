"""Position encodings.  GPT-2 adds a learned table row to the token embedding
(core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Model.java:42-48) and does nothing
to queries and keys (its rotary step is skipped: core/.../generator/CausalSelfAttention.java:341)."""
from __future__ import annotations

from .base import PositionEncoding, register_position, to_vector


class LearnedPositions(PositionEncoding):
    def __init__(self, spec, params, dtype, device):
        self.max_positions = spec.max_positions
        self.table = to_vector(params["table"], dtype, device)
        if self.table.shape[0] != self.max_positions:
            raise ValueError(f"position table has {self.table.shape[0]} rows, config says {self.max_positions}")

    def embed_table(self):
        return self.table


class NoPositions(PositionEncoding):
    def __init__(self, spec=None, params=None, dtype=None, device=None):
        pass


register_position("learned", LearnedPositions)
register_position("none", NoPositions)


def ramped_speeds(speeds, dims: int, base: float, scaling):
    """(speeds, magnitude) under a ``RampedSpeedsSpec``: pair i keeps its speed below ``lo`` and turns ``factor``
    times slower from ``hi`` on, with a straight ramp between; lo and hi are the places (among the ``dims`` entries)
    of the pairs that make ``fast`` and ``slow`` turns within ``original`` positions.  Sine and cosine grow by
    0.1 ln(factor) + 1.  Double precision."""
    import math
    factor, original = float(scaling.factor), float(scaling.original)
    if not (factor > 0.0 and original > 0.0 and scaling.fast > 0.0 and scaling.slow > 0.0 and base > 0.0 and base != 1.0):
        raise ValueError(f"speed scaling needs positive constants and a base other than 1, found {scaling} with base {base}")

    def place(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(float(scaling.fast))), 0)
    hi = min(math.ceil(place(float(scaling.slow))), dims - 1)
    out = []
    for i, f in enumerate(speeds):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


class RotaryPositions(PositionEncoding):
    """Pairs of a vector's first ``dims`` entries turned by position * base^(-2i / dims) (``RotarySpec``).  The
    speeds are worked out once in double precision; the kernel takes the sine and cosine of the double angle.
    With ``spec.scaling`` the speeds are ramped (``ramped_speeds``) and the turned pairs grow by ``magnitude``."""

    def __init__(self, spec, params=None, dtype=None, device=None):
        import torch
        self.dims, self.base, self.interleaved = int(spec.dims), float(spec.base), bool(spec.interleaved)
        if self.dims < 0 or self.dims % 2 != 0:
            raise ValueError(f"{self.dims} turned entries: an even number is needed")
        if not (self.base > 0.0):
            raise ValueError(f"rotation base {self.base} must be positive")
        speeds = [self.base ** (-2.0 * i / self.dims) for i in range(self.dims // 2)]
        self.magnitude = 1.0
        scaling = getattr(spec, "scaling", None)
        if scaling is not None and self.dims:
            speeds, self.magnitude = ramped_speeds(speeds, self.dims, self.base, scaling)
        self.speeds = torch.tensor(speeds or [0.0], dtype=torch.float64, device=device)

    def apply(self, ctx, src, dst, n_heads: int, src_head_stride: int, dst_head_stride: int, width: int):
        """dst[n, h, :width] = turned src[n, h, :width]; heads lie ``*_head_stride`` entries apart in the rows of
        src and dst (views into wider rows are fine, and src may be dst)."""
        from ..kernels import ops
        return ops.rotary(src, dst, ctx.positions, self.speeds, n_heads, src_head_stride, dst_head_stride, width,
                          self.dims, self.interleaved, self.magnitude)

    def apply_qk(self, ctx, qkv, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
        """Queries and keys of a fused q | k | v row, in place: they lie side by side as heads of one size, so one
        launch turns both."""
        qk = qkv[:, :(n_heads + n_kv_heads) * head_dim]
        self.apply(ctx, qk, qk, n_heads + n_kv_heads, head_dim, head_dim, head_dim)


register_position("rotary", RotaryPositions)
