"""Python faces of the HIP kernels.

Each function checks on the host that the operands have the shapes, dtypes and layout the
kernel and its grid assume, then launches on torch's current stream.  Nothing here falls
back to a library or to the CPU: a missing kernel library is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build
from ..profiler import KernelProfiler

F32, BF16 = 0, 1
MAX_HEAD_DIM = 256          # what the plain attention kernel takes; the matrix-core kernels: multiples of 16 up to it
ACTIVATIONS = {None: 0, "none": 0, "gelu_new": 1, "gelu_pytorch_tanh": 1, "gelu": 2, "relu": 3, "silu": 4,
               "relu2": 5,       # relu2: the square of max(x, 0)
               # only for a gated pair, with a limit c: g = min(gate, c), u = clamp(up, -c, c), g * logistic(1.702 g) * (u + 1)
               "glu_capped": 6}


class KernelError(RuntimeError):
    pass


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, found {t.dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


_PINNED_STREAM = None


def _stream():
    if _PINNED_STREAM is not None:
        return _PINNED_STREAM
    return torch.cuda.current_stream().cuda_stream


class pinned_stream:
    """Inside this context every kernel goes to the stream that was current on entry, without asking
    torch again for each launch (a model step launches about a hundred kernels)."""

    def __enter__(self):
        global _PINNED_STREAM
        self._old = _PINNED_STREAM
        _PINNED_STREAM = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _PINNED_STREAM
        _PINNED_STREAM = self._old
        return False


def _check(rc: int):
    if rc != 0:
        raise KernelError(build.load().da_last_error().decode())


_VP, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_ARGTYPES = {
    "da_embed": [_VP, _VP, _VP, _I, _VP, _I, _VP, _I, _I, _F, _VP],
    "da_copy_rows": [_VP, _I, _VP, _VP, _I, _I, _I, _I, _F, _VP],
    "da_take_tokens": [_VP, _VP, _VP, _I, _I, _I, _VP],
    "da_fill_zero": [_VP, ctypes.c_long, _VP],
    "da_state_gather": [_VP, _VP, _VP, _VP, _I, _I, _I, _VP],
    "da_state_scatter": [_VP, _VP, _VP, _VP, _I, _I, _I, _VP],
    "da_layernorm": [_VP, _VP, _VP, _I, _VP, _I, _F, _VP, _I, _I, _I, _VP],
    "da_gemm_ref": [_VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP],
    "da_gemm_bf16": [_VP, _I, _VP, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_gemm_bf16_wide": [_VP, _I, _VP, _I, _VP, _I, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP],
    "da_gemm_wide_choice": [_I, _I, _I],
    "da_gemm_bf16_ln": [_VP, _VP, _VP, _I, _VP, _I, _F, _VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP,
                        _I, _I, _I, _I, _I, _VP],
    "da_gemm_bf16_rms": [_VP, _VP, _VP, _I, _F, _F, _VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _I, _I, _VP, _VP,
                         _I, _I, _I, _I, _I, _VP],
    "da_kv_write": [_VP, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _VP],
    "da_attn_ref": [_VP, _I, _VP, _I, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _VP],
    "da_attn_decode": [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _VP],
    "da_attn_decode_split": [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I, _VP, ctypes.c_long, _VP],
    "da_attn_prefill": [_VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I, _VP],
    "da_sample": [_VP, _I, _I, _I, _VP, _VP, _VP],
    "da_decode_splits": [_I, _I, _I, _I],
    "da_can_fuse_ln": [_I, _I, _I],
    "da_run_step": [_VP, _VP],
    "da_top_logprobs": [_VP, _I, _I, _I, _VP, _I, _VP, _VP, _VP],
    "da_attn_decode_rel": [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _F, _I, _VP, _I, _I, _VP, ctypes.c_long, _VP],
    "da_attn_prefill_rel": [_VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _F, _I, _VP, _I, _I, _VP],
    "da_rmsnorm": [_VP, _VP, _VP, _I, _F, _F, _VP, _I, _I, _I, _VP],
    "da_rmsnorm_add": [_VP, _VP, _I, _VP, _VP, _I, _F, _F, _VP, _I, _I, _I, _VP],
    "da_attn_rel_ref": [_VP, _I, _VP, _I, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _F, _I, _F, _I, _VP, _VP, _I,
                        _VP, _I, _VP],
    "da_attn_window": [_VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _F, _VP, _VP, _I, _VP, _I, _I,
                       _VP],
    "da_attn_window_takes": [_I, _I, _I],
    "da_attn_prepare": [_VP, _I, _I, _I, _I, _I, _VP, _I, _VP, _I, _F, _I, _VP, _VP, _I, _I, _VP, _I, _I, _VP, _VP, _I, _I, _I, _I, _F,
                        _VP],
    "da_delta_rule": [_VP, _I, _I, _I, _I, _VP, _I, _VP, _I, _I, _VP, _VP, _VP, ctypes.c_long, _VP, _VP, _VP, _I, _I, _I, _I, _I,
                      _I, _I, _F, _I, _I, _VP],
    "da_delta_gate_norm": [_VP, _I, _VP, _I, _I, _VP, _I, _F, _I, _VP, _I, _I, _I, _I, _VP],
    "da_scale_add_rows": [_VP, _VP, _VP, _I, _I, _F, _VP],
    "da_kv_write_split": [_VP, _I, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_gated_act": [_VP, _I, _I, _VP, _I, _I, _I, _I, _F, _VP],
    "da_concat_rows": [_VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_retention": [_VP, _I, _I, _I, _I, _I, _VP, _F, _VP, ctypes.c_long, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP,
                     ctypes.c_long, _VP],
    "da_moe_top": [_VP, _I, _VP, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP],
    "da_softcap": [_VP, ctypes.c_long, _F, _VP],
    "da_moe_route": [_VP, _VP, _I, _VP, _I, _I, _I, _I, _VP, _VP, _VP, _I, _I, _VP, _VP, _VP],
    "da_moe_gated_ref": [_VP, _I, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _VP],
    "da_moe_down_ref": [_VP, _I, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _VP],
    "da_moe_gated_mfma": [_VP, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _VP],
    "da_moe_down_mfma": [_VP, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _VP],
    "da_moe_gather": [_VP, _I, _VP, _VP, _I, _I, _VP, _VP],
    "da_gemm_bf16_grouped": [_VP, _I, _VP, _I, ctypes.c_long, _VP, _I, _VP, _I, _I, _I, _I, _I, _VP, _I],
    "da_moe_up_ref": [_VP, _I, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_moe_up_mfma": [_VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP],
    "da_moe_top_logistic": [_VP, _I, _I, _I, _I, _I, _VP, _VP, _VP],
    "da_moe_slot_weights": [_VP, _VP, _I, _VP, _VP],
    "da_rotary": [_VP, _I, _I, _VP, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _F, _VP],
    "da_latent_prepare": [_VP, _I, _I, _I, _I, _I, _VP, _I, _VP, _I, _F, _VP, _VP, _VP, _I, _I, _F, _VP, _I, _VP, _I, _I, _I, _VP],
    "da_attn_latent_ref": [_VP, _I, _VP, _I, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _VP, _I, _VP],
    "da_attn_latent_mfma": [_VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I, _VP, ctypes.c_long, _VP,
                            _VP],
    "da_attn_latent_splits": [_I, _I, _I, _I],
    "da_attn_latent_mfma_takes": [_I, _I],
    "da_gemm_heads": [_VP, _I, _I, _I, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _VP],
    "da_gemm_heads_takes": [_I, _I, _I, _I],
    "da_conv_causal": [_VP, _I, _I, _VP, ctypes.c_long, _I, _VP, _VP, _VP, _VP, _I, _VP, _I, _I, _VP, _I, _I, _I, _I, _VP],
    "da_conv_state_update": [_VP, _I, _I, _VP, ctypes.c_long, _I, _VP, _VP, _I, _I, _I, _VP],
    "da_selective_scan": [_VP, _I, _I, _VP, _I, _VP, _I, _I, _I, _VP, _I, _VP, _VP, _I, _VP, ctypes.c_long, _VP, _VP,
                          _VP, _I, _I, _I, _I, _I, _I, _VP, _VP, _VP],
    "da_moe_combine": [_VP, _I, _VP, _VP, _F, _I, _VP, _I, _I, _I, _I, _VP],
}
_LIB = None


def _lib():
    """The kernel library with its argument types declared (conversion is then cheap and checked)."""
    global _LIB
    if _LIB is None:
        lib = build.load()
        for name, types in _ARGTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes = types
            fn.restype = ctypes.c_int
        _LIB = lib
    return _LIB


class _NoTiming:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_TIMING = _NoTiming()


def _timed(name: str, nbytes, flops, precision: str = "bf16"):
    """The kernel profiler's bracket around one launch, or nothing when it is off."""
    if not KernelProfiler.enabled:
        return _NO_TIMING
    return KernelProfiler.launch(name, nbytes, flops, precision)


def _nbytes(*ts) -> int:
    return sum(t.numel() * t.element_size() for t in ts if t is not None)


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")


def _rows_2d(t: torch.Tensor, name: str):
    if not (t.dim() == 2 and t.stride(1) == 1):
        raise KernelError(f"{name} must be 2-D with a contiguous last dimension")


# ------------------------------------------------------------------------------- embedding
def embed(tokens: torch.Tensor, positions: torch.Tensor, wte: torch.Tensor,
          wpe: Optional[torch.Tensor], out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[n] = wte[tokens[n]] * scale + wpe[positions[n]] in 32-bit."""
    _dev(tokens, positions, wte, wpe, out)
    N, E = out.shape
    _need(tokens.dtype == torch.int32 and positions.dtype == torch.int32, "embed: ids must be int32")
    _need(tokens.numel() >= N and positions.numel() >= N, "embed: fewer ids than rows")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
    _need(wte.is_contiguous() and wte.shape[1] == E, "embed: token table width differs from out")
    if wpe is not None:
        _need(wpe.is_contiguous() and wpe.shape[1] == E, "embed: position table width differs from out")
    with _timed("embed", N * E * (wte.element_size() * (2 if wpe is not None else 1) + 4), N * E, "fp32"):
        _check(_lib().da_embed(_ptr(tokens), _ptr(positions), _ptr(wte), _dt(wte), _ptr(wpe),
                               _dt(wpe) if wpe is not None else 0, _ptr(out), N, E, float(scale), _stream()))
    return out


def copy_rows(src: torch.Tensor, dst: torch.Tensor, rows: Optional[torch.Tensor] = None,
              accumulate: bool = False, scale: float = 1.0) -> torch.Tensor:
    """dst[r] (+)= scale * src[rows[r]] (or src[r]); 32-bit and bfloat16 on either side, += into 32-bit."""
    _dev(src, dst, rows)
    _need(src.dim() == 2 and dst.dim() == 2 and src.is_contiguous() and dst.is_contiguous() and
          src.shape[1] == dst.shape[1], "copy_rows: contiguous matrices of one width are needed")
    R = dst.shape[0]
    if rows is None:
        _need(src.shape[0] >= R, "copy_rows: fewer source rows than destination rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= R, "copy_rows: rows must be int32 with a row each")
    _need(not accumulate or dst.dtype == torch.float32, "copy_rows: accumulation needs a float32 destination")
    _check(_lib().da_copy_rows(_ptr(src), _dt(src), _ptr(rows), _ptr(dst), _dt(dst), R, dst.shape[1],
                               int(accumulate), float(scale), _stream()))
    return dst


def take_tokens(tokens: torch.Tensor, src: torch.Tensor, sampled: torch.Tensor, vocab: int) -> torch.Tensor:
    """tokens[n] = sampled[src[n]] wherever src[n] >= 0 (in place)."""
    _dev(tokens, src, sampled)
    _need(tokens.dtype == src.dtype == sampled.dtype == torch.int32, "take_tokens: int32 tensors needed")
    _need(src.numel() >= tokens.numel(), "take_tokens: fewer sources than tokens")
    _check(_lib().da_take_tokens(_ptr(tokens), _ptr(src), _ptr(sampled), tokens.numel(), sampled.numel(), int(vocab),
                                 _stream()))
    return tokens


def fill_zero(t: torch.Tensor) -> torch.Tensor:
    """Zeros over a contiguous tensor of whole 4-byte words, by a kernel of the engine's own (a recorded
    step then holds no memset node)."""
    _dev(t)
    _need(t.is_contiguous() and (t.numel() * t.element_size()) % 4 == 0, "fill_zero: a contiguous tensor of whole words")
    _check(_lib().da_fill_zero(_ptr(t), t.numel() * t.element_size(), _stream()))
    return t


def _state_rows(state: torch.Tensor, rows: torch.Tensor, name: str) -> int:
    _need(state.is_contiguous() and rows.is_contiguous() and state.dtype == rows.dtype and state.dim() >= 2,
          f"{name}: state [slots, ...] and rows [N, ...] must be contiguous and of one dtype")
    row_bytes = state[0].numel() * state.element_size()
    _need(rows.dim() >= 1 and rows.numel() == rows.shape[0] * state[0].numel() and row_bytes % 4 == 0,
          f"{name}: a row of the state is {state[0].numel()} entries ({row_bytes} bytes, whole words)")
    return row_bytes


def state_gather(state: torch.Tensor, state_slots: torch.Tensor, seq_of_token: torch.Tensor,
                 out: torch.Tensor) -> torch.Tensor:
    """out[n] = state[state_slots[seq_of_token[n]]]: every row of the step gets its sequence's state (zeros
    for a sequence without a slot, i.e. a padding row of a fixed-shape step)."""
    _dev(state, state_slots, seq_of_token, out)
    row_bytes = _state_rows(state, out, "state_gather")
    N = out.shape[0]
    _need(state_slots.dtype == torch.int32 and seq_of_token.dtype == torch.int32 and seq_of_token.numel() >= N,
          "state_gather: slots and sequence ids must be int32, one id a row")
    _check(_lib().da_state_gather(_ptr(state), _ptr(state_slots), _ptr(seq_of_token), _ptr(out), N, state.shape[0],
                                  row_bytes, _stream()))
    return out


def state_scatter(state: torch.Tensor, state_slots: torch.Tensor, q_start: torch.Tensor, rows: torch.Tensor,
                  n_seqs: int) -> None:
    """state[state_slots[s]] = rows[q_start[s + 1] - 1] for every sequence s with a slot: what the last row
    of a sequence's portion leaves is the request's state after the step."""
    _dev(state, state_slots, q_start, rows)
    row_bytes = _state_rows(state, rows, "state_scatter")
    _need(state_slots.dtype == torch.int32 and q_start.dtype == torch.int32 and state_slots.numel() >= n_seqs
          and q_start.numel() >= n_seqs + 1, "state_scatter: slots [S] and q_start [S+1] must be int32")
    _check(_lib().da_state_scatter(_ptr(state), _ptr(state_slots), _ptr(q_start), _ptr(rows), n_seqs, state.shape[0],
                                   row_bytes, _stream()))


# ------------------------------------------------------------------------------- norms
def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
              out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm of 32-bit rows; with ``rows`` the output row r is the norm of x[rows[r]]."""
    _dev(x, weight, bias, out, rows)
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2, "layernorm: x must be contiguous float32 [N, E]")
    E = x.shape[1]
    R = out.shape[0]
    _need(out.is_contiguous() and out.shape[1] == E, "layernorm: out must be contiguous [R, E]")
    _need(weight.numel() == E and (bias is None or bias.numel() == E), "layernorm: parameter length differs from E")
    if rows is None:
        _need(R <= x.shape[0], "layernorm: more output rows than input rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= R, "layernorm: rows must be int32 with R entries")
    with _timed("layernorm", R * E * (4 + out.element_size()) + _nbytes(weight, bias), 8 * R * E, "fp32"):
        _check(_lib().da_layernorm(_ptr(x), _ptr(rows), _ptr(weight), _dt(weight), _ptr(bias),
                                   _dt(bias) if bias is not None else 0, eps, _ptr(out),
                                   _dt(out), R, E, _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, gain_offset: float, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = x[rows[r] or r] / sqrt(mean(x^2) + eps) * (gain_offset + weight), in 32-bit."""
    _dev(x, weight, out, rows)
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2, "rmsnorm: x must be contiguous float32 [N, E]")
    E, R = x.shape[1], out.shape[0]
    _need(out.is_contiguous() and out.dim() == 2 and out.shape[1] == E, "rmsnorm: out must be contiguous [R, E]")
    _need(weight.numel() == E and weight.is_contiguous(), "rmsnorm: the gain's length differs from E")
    if rows is None:
        _need(R <= x.shape[0], "rmsnorm: more output rows than input rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= R, "rmsnorm: rows must be int32 with R entries")
    with _timed("rmsnorm", R * E * (4 + out.element_size()) + _nbytes(weight), 4 * R * E, "fp32"):
        _check(_lib().da_rmsnorm(_ptr(x), _ptr(rows), _ptr(weight), _dt(weight), float(gain_offset), float(eps),
                                 _ptr(out), _dt(out), R, E, _stream()))
    return out


def rmsnorm_add(src: torch.Tensor, weight: torch.Tensor, x: torch.Tensor, gain_offset: float, eps: float,
                next_weight: Optional[torch.Tensor] = None, next_out: Optional[torch.Tensor] = None) -> None:
    """x += rms(src) with ``weight``; with ``next_weight``, ``next_out = rms(x)`` of the new x in the same pass
    (the norm behind a part, the residual addition and the norm in front of the next part); with ``next_out`` alone,
    the new x itself in ``next_out``'s dtype (the next part reads the stream without a norm)."""
    _dev(src, weight, x, next_weight, next_out)
    _need(src.dtype == torch.float32 and x.dtype == torch.float32 and src.is_contiguous() and x.is_contiguous()
          and src.dim() == 2 and src.shape == x.shape, "rmsnorm_add: src and x must be contiguous float32 of one shape")
    R, E = x.shape
    _need(weight.numel() == E and weight.is_contiguous(), "rmsnorm_add: the gain's length differs from E")
    _need(next_weight is None or next_out is not None, "rmsnorm_add: the second norm needs its output")
    if next_out is not None:
        _need((next_weight is None or (next_weight.numel() == E and next_weight.is_contiguous())) and next_out.is_contiguous()
              and tuple(next_out.shape) == (R, E), "rmsnorm_add: the second norm's operands differ from [R, E]")
    nb = R * E * 12 + _nbytes(weight, next_weight) + (0 if next_out is None else _nbytes(next_out))
    with _timed("rmsnorm_add", nb, 8 * R * E, "fp32"):
        _check(_lib().da_rmsnorm_add(_ptr(src), _ptr(weight), _dt(weight), _ptr(x), _ptr(next_weight),
                                     _dt(next_weight) if next_weight is not None else 0, float(gain_offset), float(eps),
                                     _ptr(next_out), _dt(next_out) if next_out is not None else 0, R, E, _stream()))


def scale_add_rows(src: torch.Tensor, scale: torch.Tensor, dst: torch.Tensor, mult: float = 1.0) -> torch.Tensor:
    """dst[r, c] += mult * scale[c] * src[r, c], all 32-bit: a part's result joins the stream times a learned scale
    per channel."""
    _dev(src, scale, dst)
    _need(src.dtype == dst.dtype == scale.dtype == torch.float32 and src.is_contiguous() and dst.is_contiguous()
          and scale.is_contiguous() and src.dim() == 2 and src.shape == dst.shape and scale.numel() == src.shape[1],
          "scale_add_rows: contiguous float32 [R, E], [E] and [R, E] are needed")
    with _timed("scale_add_rows", 3 * _nbytes(src), 2 * src.numel(), "fp32"):
        _check(_lib().da_scale_add_rows(_ptr(src), _ptr(scale), _ptr(dst), src.shape[0], src.shape[1], float(mult), _stream()))
    return dst


def gated_act(gu: torch.Tensor, mid: torch.Tensor, act: str, limit: float = 0.0) -> torch.Tensor:
    """mid[r, j] = act(gu[r, j]) * gu[r, inner + j]: the halves of a fused gate | up product ("glu_capped" with its
    ``limit``: see ``ACTIVATIONS``)."""
    _dev(gu, mid)
    _rows_2d(gu, "gu"); _rows_2d(mid, "mid")
    R, inner = mid.shape
    _need(gu.shape[0] == R and gu.shape[1] == 2 * inner and gu.dtype == mid.dtype, "gated_act: gu must be [R, 2 * inner] of mid's dtype")
    if not (act in ACTIVATIONS):
        raise KernelError(f"gated_act: unknown activation {act!r}")
    with _timed("gated_act", _nbytes(gu, mid), 10 * R * inner, "fp32"):
        _check(_lib().da_gated_act(_ptr(gu), gu.stride(0), _dt(gu), _ptr(mid), mid.stride(0), R, inner, ACTIVATIONS[act],
                                   float(limit), _stream()))
    return mid


def concat_rows(src: torch.Tensor, dst: torch.Tensor, col: int) -> torch.Tensor:
    """dst[r, col : col + E] = src[r, :]: a 32-bit matrix [R, E] into columns of a wider matrix of either dtype."""
    _dev(src, dst)
    _rows_2d(dst, "dst")
    _need(src.dtype == torch.float32 and src.dim() == 2 and src.is_contiguous(), "concat_rows: src must be contiguous float32")
    R, E = src.shape
    _need(dst.shape[0] >= R and 0 <= col and col + E <= dst.shape[1], "concat_rows: the columns leave the row")
    _check(_lib().da_concat_rows(_ptr(src), _ptr(dst), _dt(dst), dst.stride(0), int(col), R, E, _stream()))
    return dst


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "softcap: contiguous float32 logits")
    _check(_lib().da_softcap(_ptr(logits), logits.numel(), float(cap), _stream()))
    return logits


# ------------------------------------------------------------------------------- experts
MOE_TILE_ROWS = 64       # rows of a tile of the plain grouped products
MOE_TILE_ROWS_MFMA = 32  # ... of the matrix-core grouped products for few rows an expert (csrc/moe.hip)
MOE_TILE_ROWS_BLOCK = 128  # ... of the block-tile product with a matrix per group of rows (csrc/gemm_mfma.hip)


def moe_slot_space(n_tokens: int, top: int, n_experts: int, tile: int):
    """(tiles, rows) of the slot space that holds every (token, choice) pair with each expert's pairs starting
    at a multiple of ``tile`` rows, whatever the routing."""
    tiles = -(-n_tokens * top // tile) + n_experts
    return tiles, tiles * tile


def moe_route(tokens: Optional[torch.Tensor], table: Optional[torch.Tensor], ids: Optional[torch.Tensor], n_tokens: int,
              top: int, n_experts: int, tile: int, slot_of_pair: torch.Tensor, row_of_slot: torch.Tensor,
              tile_expert: torch.Tensor, pair_weights: Optional[torch.Tensor] = None,
              slot_weight: Optional[torch.Tensor] = None) -> None:
    """Every (token, choice) pair gets a slot; an expert's slots lie together and start at a multiple of ``tile``.
    The experts come from ``table[tokens[n], k]`` or from ``ids[n, k]``.  With ``pair_weights`` [N, top] the weight of
    every pair is also written where its slot is (``slot_weight``, float32, one a slot)."""
    _dev(tokens, table, ids, slot_of_pair, row_of_slot, tile_expert)
    for t_ in (tokens, table, ids, slot_of_pair, row_of_slot, tile_expert):
        _need(t_ is None or (t_.dtype == torch.int32 and t_.is_contiguous()), "moe_route: int32 contiguous operands")
    vocab = 0
    if table is not None:
        _need(tokens is not None and tokens.numel() >= n_tokens and table.dim() == 2 and table.shape[1] == top,
              "moe_route: a table [vocab, top] with a token id a row")
        vocab = table.shape[0]
    else:
        _need(ids is not None and ids.numel() >= n_tokens * top, "moe_route: expert ids [N, top]")
    tiles, rows = moe_slot_space(n_tokens, top, n_experts, tile)
    _need(slot_of_pair.numel() >= n_tokens * top and row_of_slot.numel() >= rows and tile_expert.numel() >= tiles,
          "moe_route: the outputs are smaller than the slot space")
    _need((pair_weights is None) == (slot_weight is None), "moe_route: weights a pair need a place a slot")
    if pair_weights is not None:
        _dev(pair_weights, slot_weight)
        _need(pair_weights.dtype == torch.float32 and pair_weights.numel() >= n_tokens * top and pair_weights.is_contiguous()
              and slot_weight.dtype == torch.float32 and slot_weight.numel() >= rows and slot_weight.is_contiguous(),
              "moe_route: float32 weights, one a pair and one a slot")
    with _timed("moe_route", 4 * (n_tokens * top * 3 + rows + tiles), 0, "fp32"):
        _check(_lib().da_moe_route(_ptr(tokens), _ptr(table), vocab, _ptr(ids), n_tokens, top, n_experts, tile,
                                   _ptr(slot_of_pair), _ptr(row_of_slot), _ptr(tile_expert), rows, tiles, _stream(),
                                   _ptr(pair_weights), _ptr(slot_weight)))


def _moe_common(a, row_of_slot, tile_expert, w, tiles, tile, name):
    _dev(a, row_of_slot, tile_expert, w)
    _rows_2d(a, "a")
    _need(w.dim() == 3 and w.is_contiguous() and w.dtype == a.dtype, f"{name}: stacked weights [experts, out, in] of a's dtype")
    _need(row_of_slot.dtype == torch.int32 and tile_expert.dtype == torch.int32 and tile_expert.numel() >= tiles
          and row_of_slot.numel() >= tiles * tile, f"{name}: the routing arrays are smaller than the slot space")


def moe_gated_ref(a: torch.Tensor, row_of_slot: torch.Tensor, tile_expert: torch.Tensor, w: torch.Tensor,
                  mid: torch.Tensor, tiles: int, act: str, limit: float = 0.0) -> torch.Tensor:
    """mid[slot] = act(Wg_e a[row_of_slot[slot]]) * (Wu_e a[...]) for every used slot; w: [experts, 2 F, K]."""
    _moe_common(a, row_of_slot, tile_expert, w, tiles, MOE_TILE_ROWS, "moe_gated")
    K, F = a.shape[1], w.shape[1] // 2
    _rows_2d(mid, "mid")
    _need(w.shape[2] == K and w.shape[1] == 2 * F and mid.shape[1] == F and mid.shape[0] >= tiles * MOE_TILE_ROWS
          and mid.dtype == a.dtype, "moe_gated: shapes differ")
    if not (act in ACTIVATIONS):
        raise KernelError(f"moe_gated: unknown activation {act!r}")
    with _timed("moe_gated_plain", _nbytes(a, w, mid), 4 * tiles * MOE_TILE_ROWS * F * K, "fp32" if a.dtype == torch.float32 else "bf16"):
        _check(_lib().da_moe_gated_ref(_ptr(a), a.stride(0), _dt(a), _ptr(row_of_slot), _ptr(tile_expert), _ptr(w),
                                       _ptr(mid), mid.stride(0), tiles, K, F, ACTIVATIONS[act], float(limit), _stream()))
    return mid


def moe_down_ref(mid: torch.Tensor, row_of_slot: torch.Tensor, tile_expert: torch.Tensor, w: torch.Tensor,
                 out: torch.Tensor, tiles: int) -> torch.Tensor:
    """out[slot] = Wd_e mid[slot] (32-bit) for every used slot; w: [experts, width, F]."""
    _moe_common(mid, row_of_slot, tile_expert, w, tiles, MOE_TILE_ROWS, "moe_down")
    F, width = mid.shape[1], w.shape[1]
    _rows_2d(out, "out")
    _need(w.shape[2] == F and out.shape[1] == width and out.dtype == torch.float32 and
          out.shape[0] >= tiles * MOE_TILE_ROWS and mid.shape[0] >= tiles * MOE_TILE_ROWS, "moe_down: shapes differ")
    with _timed("moe_down_plain", _nbytes(mid, w, out), 2 * tiles * MOE_TILE_ROWS * F * width, "fp32" if mid.dtype == torch.float32 else "bf16"):
        _check(_lib().da_moe_down_ref(_ptr(mid), mid.stride(0), _dt(mid), _ptr(row_of_slot), _ptr(tile_expert), _ptr(w),
                                      _ptr(out), out.stride(0), tiles, F, width, _stream()))
    return out


def moe_combine(out: torch.Tensor, slot_of_pair: torch.Tensor, weights: Optional[torch.Tensor], uniform: float,
                top: int, y: torch.Tensor, accumulate: bool) -> torch.Tensor:
    """y[n] (+)= sum_k weight * out[slot_of_pair[n, k]] with ``weights[n, k]`` or the one weight ``uniform``."""
    _dev(out, slot_of_pair, weights, y)
    _rows_2d(out, "out"); _rows_2d(y, "y")
    N, width = y.shape
    _need(out.dtype == torch.float32 and y.dtype == torch.float32 and out.shape[1] == width, "moe_combine: float32 [.., width]")
    _need(slot_of_pair.dtype == torch.int32 and slot_of_pair.numel() >= N * top, "moe_combine: a slot a pair")
    _need(weights is None or (weights.dtype == torch.float32 and weights.numel() >= N * top), "moe_combine: a weight a pair")
    with _timed("moe_combine", (top + 2) * N * width * 4, top * N * width, "fp32"):
        _check(_lib().da_moe_combine(_ptr(out), out.stride(0), _ptr(slot_of_pair), _ptr(weights), float(uniform), top,
                                     _ptr(y), y.stride(0), N, width, int(accumulate), _stream()))
    return y


# ------------------------------------------------------------------------------- products
def linear_ref(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
               act: Optional[str] = None, accumulate: bool = False) -> torch.Tensor:
    """out (+)= act(a @ w.T + bias) with the plain tiled kernel; w is [N, K]."""
    _dev(a, w, bias, out)
    _rows_2d(a, "a"); _rows_2d(w, "w"); _rows_2d(out, "out")
    M, K = a.shape
    N = w.shape[0]
    if not (w.shape[1] == K):
        raise KernelError(f"linear: a is [{M},{K}] but w is {list(w.shape)}")
    if not (out.shape[0] == M and out.shape[1] == N):
        raise KernelError(f"linear: out is {list(out.shape)}, expected [{M},{N}]")
    _need(a.dtype == w.dtype, "linear: a and w must share a dtype")
    _need(bias is None or bias.numel() == N, "linear: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear: unknown activation {act!r}")
    _need(not accumulate or out.dtype == torch.float32, "linear: accumulation needs a float32 output")
    with _timed("linear_ref", _product_bytes(a, w, bias, out, accumulate), 2 * M * N * K, "fp32"):
        _check(_lib().da_gemm_ref(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _dt(a), _ptr(bias),
                                  _dt(bias) if bias is not None else 0, ACTIVATIONS[act], int(accumulate),
                                  _ptr(out), _dt(out), out.stride(0), M, N, K, _stream()))
    return out


def _product_bytes(a, w, bias, out, accumulate) -> int:
    """What a product must move at least: a, w and the bias once, the output once (twice when it adds)."""
    return _nbytes(a, w, bias) + _nbytes(out) * (2 if accumulate else 1)


# ------------------------------------------------------------------------------- cache write
def kv_write(qkv: torch.Tensor, k_off: int, v_off: int, cache_slot: torch.Tensor,
             slot_map: torch.Tensor, n_kv_heads: int, head_dim: int) -> None:
    """Rows of k and v (columns k_off.., v_off.. of qkv) go to cache rows ``slot_map``.
    cache_slot: [n_pages, 2, Hkv, page, D]."""
    _dev(qkv, cache_slot, slot_map)
    _rows_2d(qkv, "qkv")
    N = qkv.shape[0]
    _need(cache_slot.dim() == 5 and cache_slot.is_contiguous(), "kv_write: cache slot must be contiguous [pages,2,Hkv,page,D]")
    P, two, Hkv, page, D = cache_slot.shape
    _need(two == 2 and Hkv == n_kv_heads and D == head_dim, "kv_write: cache slot shape differs from the heads")
    _need(cache_slot.dtype == qkv.dtype, "kv_write: cache and activations differ in dtype")
    _need(slot_map.dtype == torch.int32 and slot_map.numel() >= N, "kv_write: slot_map must be int32 [N]")
    with _timed("kv_write", 4 * N * Hkv * D * qkv.element_size(), 0, "fp32"):
        _check(_lib().da_kv_write(_ptr(qkv), _dt(qkv), qkv.stride(0), k_off, v_off, _ptr(cache_slot),
                                  _ptr(slot_map), N, Hkv, D, page, _stream()))


# ------------------------------------------------------------------------------- attention
def attention_ref(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                  seq_of_token: torch.Tensor, positions: torch.Tensor, n_heads: int, scale: float,
                  window: Optional[int], out: torch.Tensor) -> torch.Tensor:
    """Plain paged attention for any rows.  q: [N, >= Hq*D] view (row stride free)."""
    _dev(q, cache_slot, block_table, seq_of_token, positions, out)
    _rows_2d(q, "q"); _rows_2d(out, "out")
    N = q.shape[0]
    P, two, Hkv, page, D = cache_slot.shape
    _need(cache_slot.is_contiguous() and two == 2, "attention: cache slot must be contiguous [pages,2,Hkv,page,D]")
    _need(q.shape[1] == n_heads * D and out.shape[1] == n_heads * D and out.shape[0] == N,
          "attention: q/out must be [N, Hq*D]")
    _need(q.dtype == cache_slot.dtype == out.dtype, "attention: q, cache and out must share a dtype")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention: block_table must be contiguous int32 [S, max_blocks]")
    _need(seq_of_token.dtype == torch.int32 and positions.dtype == torch.int32, "attention: ids must be int32")
    _need(seq_of_token.numel() >= N and positions.numel() >= N, "attention: fewer ids than rows")
    _check(_lib().da_attn_ref(_ptr(q), q.stride(0), _ptr(cache_slot), _dt(q), _ptr(block_table),
                              block_table.shape[1], _ptr(seq_of_token), _ptr(positions), N, n_heads, Hkv,
                              D, page, scale, int(window or 0), _ptr(out), out.stride(0),
                              _stream()))
    return out


def cache_page_elems(cache_slot: torch.Tensor) -> int:
    return cache_slot[0].numel()


def kv_write_split(qkv: torch.Tensor, k_off: int, v_off: int, cache_slot: torch.Tensor, slot_map: torch.Tensor,
                   n_kv_heads: int, head_dim: int, v_head_dim: int, page: int) -> None:
    """Keys (``head_dim`` a head) and values (``v_head_dim`` a head) go to cache rows ``slot_map``; a page of the
    slot holds Hkv * page * head_dim keys, then Hkv * v_head_dim * page values."""
    _dev(qkv, cache_slot, slot_map)
    _rows_2d(qkv, "qkv")
    N = qkv.shape[0]
    _need(cache_slot.is_contiguous() and cache_page_elems(cache_slot) == n_kv_heads * page * (head_dim + v_head_dim),
          "kv_write_split: a page of the cache slot does not hold Hkv * page * (D + Dv) entries")
    _need(cache_slot.dtype == qkv.dtype, "kv_write_split: cache and activations differ in dtype")
    _need(slot_map.dtype == torch.int32 and slot_map.numel() >= N, "kv_write_split: slot_map must be int32 [N]")
    with _timed("kv_write", 2 * N * n_kv_heads * (head_dim + v_head_dim) * qkv.element_size(), 0, "fp32"):
        _check(_lib().da_kv_write_split(_ptr(qkv), _dt(qkv), qkv.stride(0), k_off, v_off, _ptr(cache_slot), _ptr(slot_map),
                                        N, n_kv_heads, head_dim, v_head_dim, page, _stream()))


def attention_rel_ref(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor, seq_of_token: torch.Tensor,
                      positions: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int, page: int,
                      scale: float, window: Optional[int], dist_bias: Optional[torch.Tensor], temp_coef: float,
                      temp_every: int, out: torch.Tensor, softcap: float = 0.0, keep_first: int = 0,
                      sink: Optional[torch.Tensor] = None, gate_col: int = -1) -> torch.Tensor:
    """Plain paged attention with a bias by distance (``dist_bias`` [Hq, n_dist] float32, the last column for every
    larger distance), a query temperature by position, values of their own size, a cap on the scores
    (``softcap * tanh(score / softcap)``) and, with a window, ``keep_first`` first keys that stay visible.  ``sink``
    (float32 [Hq]): exp(sink[h]) joins the softmax's denominator; ``gate_col`` >= 0: out * logistic(gate), the gate's
    Hq * Dv entries lying in q's rows from that column on (q is then wider than its Hq * D query entries)."""
    _dev(q, cache_slot, block_table, seq_of_token, positions, dist_bias, out, sink)
    gate_ptr, gate_ld = _sink_gate_args(sink, gate_col, n_heads, n_heads * head_dim, n_heads * v_head_dim, q, "attention")
    _rows_2d(q, "q"); _rows_2d(out, "out")
    N = q.shape[0]
    _need(cache_slot.is_contiguous() and cache_page_elems(cache_slot) == n_kv_heads * page * (head_dim + v_head_dim),
          "attention: a page of the cache slot does not hold Hkv * page * (D + Dv) entries")
    _need((q.shape[1] == n_heads * head_dim or gate_col >= 0) and out.shape[1] == n_heads * v_head_dim and out.shape[0] == N,
          "attention: q must be [N, Hq*D] and out [N, Hq*Dv]")
    _need(q.dtype == cache_slot.dtype == out.dtype, "attention: q, cache and out must share a dtype")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention: block_table must be contiguous int32 [S, max_blocks]")
    _need(seq_of_token.dtype == torch.int32 and positions.dtype == torch.int32, "attention: ids must be int32")
    _need(seq_of_token.numel() >= N and positions.numel() >= N, "attention: fewer ids than rows")
    n_dist = 0
    if dist_bias is not None:
        _need(dist_bias.dtype == torch.float32 and dist_bias.is_contiguous() and dist_bias.dim() == 2
              and dist_bias.shape[0] == n_heads, "attention: the bias by distance must be float32 [Hq, n_dist]")
        n_dist = dist_bias.shape[1]
    _check(_lib().da_attn_rel_ref(_ptr(q), q.stride(0), _ptr(cache_slot), _dt(q), _ptr(block_table), block_table.shape[1],
                                  _ptr(seq_of_token), _ptr(positions), N, n_heads, n_kv_heads, head_dim, v_head_dim, page,
                                  float(scale), int(window or 0), _ptr(dist_bias), n_dist, float(temp_coef),
                                  int(temp_every), float(softcap), int(keep_first if window else 0), _ptr(sink),
                                  gate_ptr, gate_ld, _ptr(out), out.stride(0), _stream()))
    return out


def _sink_gate_args(sink, gate_col, n_heads, q_cols, cols, q, name):
    """Checks a sink vector and a gate that lies in q's rows; returns the gate's (address, row length)."""
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == n_heads,
              f"{name}: the sink must be float32 with one entry a query head")
    if gate_col < 0:
        return None, 0
    _need(gate_col >= q_cols and gate_col + cols <= q.shape[1], f"{name}: the gate's columns leave q's rows or meet the queries")
    return _ptr(q) + gate_col * q.element_size(), q.stride(0)


# ------------------------------------------------------------------------------- sampling
SAMPLE_ROW_FLOATS = 8     # one SampleRow record is 8 four-byte fields


def sample(logits: torch.Tensor, params: torch.Tensor, out_tokens: torch.Tensor) -> torch.Tensor:
    """params: int32/float32-punned [R, 8] records (see sampling.device_rows)."""
    _dev(logits, params, out_tokens)
    _rows_2d(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "sample: logits must be float32")
    _need(params.is_contiguous() and params.numel() >= R * SAMPLE_ROW_FLOATS and params.element_size() == 4,
          "sample: params must hold R records of 8 four-byte fields")
    _need(out_tokens.dtype == torch.int32 and out_tokens.numel() >= R, "sample: out must be int32 [R]")
    with _timed("sample", R * V * 4, R * V, "fp32"):
        _check(_lib().da_sample(_ptr(logits), logits.stride(0), R, V, _ptr(params), _ptr(out_tokens), _stream()))
    return out_tokens


def top_logprobs(logits: torch.Tensor, params: torch.Tensor, n: int, out_idx: torch.Tensor,
                 out_lp: torch.Tensor) -> None:
    _dev(logits, params, out_idx, out_lp)
    _rows_2d(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "top_logprobs: logits must be float32")
    _need(0 < n <= V, "top_logprobs: n must be in [1, V]")
    _need(out_idx.dtype == torch.int32 and out_idx.numel() >= R * n and out_idx.is_contiguous(), "top_logprobs: out_idx")
    _need(out_lp.dtype == torch.float32 and out_lp.numel() >= R * n and out_lp.is_contiguous(), "top_logprobs: out_lp")
    _check(_lib().da_top_logprobs(_ptr(logits), logits.stride(0), R, V, _ptr(params), n, _ptr(out_idx),
                                        _ptr(out_lp), _stream()))


# ------------------------------------------------------------------------------- dispatch
# "tuned": MFMA products and the prefill/decode attention kernels in bfloat16;
# "reference": the plain kernels everywhere (for A/B checks).  32-bit always runs the plain
# kernels: they are its product path.
_MODE = "tuned"


def set_kernel_mode(mode: str) -> None:
    global _MODE
    if mode not in ("tuned", "reference"):
        raise ValueError("kernel mode must be 'tuned' or 'reference'")
    _MODE = mode


def kernel_mode() -> str:
    return _MODE


class kernel_mode_scope:
    """The kernel mode of one engine while one of its steps is put on the device (two engines of
    one process may differ)."""

    def __init__(self, mode: str):
        if mode not in ("tuned", "reference"):
            raise ValueError("kernel mode must be 'tuned' or 'reference'")
        self.mode = mode

    def __enter__(self):
        global _MODE
        self._old, _MODE = _MODE, self.mode
        return self

    def __exit__(self, *exc):
        global _MODE
        _MODE = self._old
        return False


def _kv_args(kv_cache, slot_map, q_cols, n_rows, N, out, name):
    """The cache-scatter arguments of a fused q|k|v projection (zeros when there is none)."""
    if kv_cache is None:
        return None, None, 0, 0, 0, 0, 0
    _need(kv_cache.dim() == 5 and kv_cache.is_contiguous() and kv_cache.dtype == torch.bfloat16 and
          out.dtype == torch.bfloat16, f"{name}: cache slot must be contiguous bfloat16 [pages,2,Hkv,page,D]")
    _, _, Hkv, page, D = kv_cache.shape
    _need(slot_map is not None and slot_map.dtype == torch.int32 and slot_map.numel() >= n_rows,
          f"{name}: slot_map must be int32 [rows]")
    if not (q_cols + 2 * Hkv * D == N):
        raise KernelError(f"{name}: q|k|v columns do not add up to N")
    return _ptr(kv_cache), _ptr(slot_map), q_cols, Hkv * D, Hkv, D, page


WIDE_TILE_SHAPES = {"wide": 0, "wide_256x128": 1, "wide_128x128": 2}


def _wide_tiles(M, N, K, act, accumulate, out) -> bool:
    """Whether the library gives this product to its tiles whose operands go straight into LDS (the
    profiler's name for it only; the choice itself is the library's: csrc/gemm_wide.hip)."""
    takes = K % 64 == 0 and (ACTIVATIONS[act] == 0 or (not accumulate and out.dtype == torch.bfloat16))
    return takes and _lib().da_gemm_wide_choice(M, N, K) >= 0


def linear_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                act: Optional[str] = None, accumulate: bool = False, kv_cache: Optional[torch.Tensor] = None,
                slot_map: Optional[torch.Tensor] = None, q_cols: int = 0, form: str = "auto") -> torch.Tensor:
    """out (+)= act(a @ w.T + bias) on the matrix cores; a, w bfloat16, K a multiple of 8.  With
    ``kv_cache`` the columns from ``q_cols`` on (k | v) also go to the cache rows ``slot_map``.
    ``form``: "auto" lets the library choose by shape; "wide", "wide_256x128" and "wide_128x128" ask for the
    tiles of 256 x 256, 256 x 128 and 128 x 128 whose operands go from memory straight into LDS, whatever
    the product's sizes (K a multiple of 64; tests and timing)."""
    _dev(a, w, bias, out)
    _rows_2d(a, "a"); _rows_2d(w, "w"); _rows_2d(out, "out")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "linear_mfma: a and w must be bfloat16")
    if not (w.shape[1] == K):
        raise KernelError(f"linear: a is [{M},{K}] but w is {list(w.shape)}")
    if not (out.shape[0] == M and out.shape[1] == N):
        raise KernelError(f"linear: out is {list(out.shape)}, expected [{M},{N}]")
    _need(bias is None or bias.numel() == N, "linear: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear: unknown activation {act!r}")
    _need(not accumulate or out.dtype == torch.float32, "linear: accumulation needs a float32 output")
    _need(kv_cache is None or not accumulate, "linear: a cache scatter goes with a plain store")
    kvp = _kv_args(kv_cache, slot_map, q_cols, M, N, out, "linear_mfma")
    timing = _NO_TIMING
    if KernelProfiler.enabled:           # (the cost model is worked out only when someone reads it)
        name = "product_skinny" if (M <= 32 or (M <= 64 and N <= 8192)) else ("product_wide" if _wide_tiles(M, N, K, act, accumulate, out) else "product_tile")
        timing = _timed(name, _product_bytes(a, w, bias, out, accumulate), 2 * M * N * K)
    if form != "auto" and form not in WIDE_TILE_SHAPES:
        raise KernelError(f"linear_mfma: unknown form {form!r}")
    args = (_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(bias), _dt(bias) if bias is not None else 0,
            ACTIVATIONS[act], int(accumulate), _ptr(out), _dt(out), out.stride(0), M, N, K, *kvp)
    with timing:
        if form == "auto":
            _check(_lib().da_gemm_bf16(*args, _stream()))
        else:
            _check(_lib().da_gemm_bf16_wide(*args, WIDE_TILE_SHAPES[form], _stream()))
    return out


# Which steps the fused norm + product kernel takes (few rows, a width it holds; measured limits) is the
# library's rule, da_can_fuse_ln in csrc/run_step.hip, so that the parts here and the step issued from C++
# decide alike.
FUSED_LN_KERNEL_MAX_ROWS = 32


def can_fuse_ln(n_rows: int, x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``linear_ln`` takes this step: few rows, bfloat16 weights, a width the kernel holds."""
    return (_MODE == "tuned" and w.dtype == torch.bfloat16 and x.dtype == torch.float32 and w.stride(0) % 8 == 0
            and bool(_lib().da_can_fuse_ln(int(n_rows), int(w.shape[1]), int(w.shape[0]))))


def linear_ln(x: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, norm_weight: torch.Tensor,
              norm_bias: Optional[torch.Tensor], eps: float, w: torch.Tensor, bias: Optional[torch.Tensor],
              out: torch.Tensor, act: Optional[str] = None, kv_cache: Optional[torch.Tensor] = None,
              slot_map: Optional[torch.Tensor] = None, q_cols: int = 0) -> torch.Tensor:
    """out = act(LayerNorm(x[rows]) @ w.T + bias) in one kernel, for steps of at most 32 rows; with
    ``kv_cache`` the columns from ``q_cols`` on (k | v of a fused projection) also go to the cache
    rows ``slot_map``."""
    _dev(x, rows, norm_weight, norm_bias, w, bias, out, kv_cache, slot_map)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "linear_ln: x must be contiguous float32")
    _rows_2d(w, "w"); _rows_2d(out, "out")
    N, K = w.shape
    _need(x.shape[1] == K and norm_weight.numel() == K and (norm_bias is None or norm_bias.numel() == K),
          "linear_ln: widths differ")
    _need(w.dtype == torch.bfloat16, "linear_ln: w must be bfloat16")
    _need(0 < n_rows <= FUSED_LN_KERNEL_MAX_ROWS and out.shape[0] >= n_rows and out.shape[1] == N, "linear_ln: bad row count")
    if rows is None:
        _need(x.shape[0] >= n_rows, "linear_ln: fewer rows in x than asked")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows, "linear_ln: rows must be int32")
    _need(bias is None or bias.numel() == N, "linear_ln: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear_ln: unknown activation {act!r}")
    kvp = _kv_args(kv_cache, slot_map, q_cols, n_rows, N, out, "linear_ln")
    with _timed("norm_product_fused", n_rows * K * 4 + _nbytes(w, bias, norm_weight, norm_bias) + n_rows * N * out.element_size(),
                2 * n_rows * N * K):
        _check(_lib().da_gemm_bf16_ln(
            _ptr(x), _ptr(rows), _ptr(norm_weight), _dt(norm_weight), _ptr(norm_bias),
            _dt(norm_bias) if norm_bias is not None else 0, eps, _ptr(w), w.stride(0), _ptr(bias),
            _dt(bias) if bias is not None else 0, ACTIVATIONS[act], _ptr(out), _dt(out), out.stride(0), n_rows, N, K,
            *kvp, _stream()))
    return out


def linear_rms(x: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, norm_weight: torch.Tensor,
               gain_offset: float, eps: float, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
               act: Optional[str] = None, kv_cache: Optional[torch.Tensor] = None,
               slot_map: Optional[torch.Tensor] = None, q_cols: int = 0) -> torch.Tensor:
    """``linear_ln`` with a root-mean-square norm in front of the product:
    out = act((x[rows] / sqrt(mean(x^2) + eps) * (gain_offset + norm_weight)) @ w.T + bias), for steps that
    ``can_fuse_ln`` takes."""
    _dev(x, rows, norm_weight, w, bias, out, kv_cache, slot_map)
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "linear_rms: x must be contiguous float32")
    _rows_2d(w, "w"); _rows_2d(out, "out")
    N, K = w.shape
    _need(x.shape[1] == K and norm_weight.numel() == K, "linear_rms: widths differ")
    _need(w.dtype == torch.bfloat16, "linear_rms: w must be bfloat16")
    _need(0 < n_rows <= FUSED_LN_KERNEL_MAX_ROWS and out.shape[0] >= n_rows and out.shape[1] == N, "linear_rms: bad row count")
    if rows is None:
        _need(x.shape[0] >= n_rows, "linear_rms: fewer rows in x than asked")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= n_rows, "linear_rms: rows must be int32")
    _need(bias is None or bias.numel() == N, "linear_rms: bias length differs from N")
    if not (act in ACTIVATIONS):
        raise KernelError(f"linear_rms: unknown activation {act!r}")
    kvp = _kv_args(kv_cache, slot_map, q_cols, n_rows, N, out, "linear_rms")
    with _timed("norm_product_fused", n_rows * K * 4 + _nbytes(w, bias, norm_weight) + n_rows * N * out.element_size(),
                2 * n_rows * N * K):
        _check(_lib().da_gemm_bf16_rms(
            _ptr(x), _ptr(rows), _ptr(norm_weight), _dt(norm_weight), float(gain_offset), float(eps), _ptr(w), w.stride(0),
            _ptr(bias), _dt(bias) if bias is not None else 0, ACTIVATIONS[act], _ptr(out), _dt(out), out.stride(0),
            n_rows, N, K, *kvp, _stream()))
    return out


def _mfma_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[1] % 8 == 0
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


# Measured on MI355X (q|k|v of 768 to 1,600 wide, 128 to 2,048 rows): the cache write in the product's
# epilogue adds 1.3 to 3.4 us where the rows' places are runs of consecutive cache rows (a prompt
# portion: keys and values both go over in 16-byte pieces), the write kernel after the product 3.7 to
# 9.2 us; with places in any order the two are level at 2,048 rows and the epilogue is ahead below.


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           act: Optional[str] = None, accumulate: bool = False, kv_cache: Optional[torch.Tensor] = None,
           slot_map: Optional[torch.Tensor] = None, q_cols: int = 0) -> torch.Tensor:
    """out (+)= act(a @ w.T + bias); picks the kernel by dtype and mode.  Shapes the matrix-core
    kernel does not take (K not a multiple of 8) go to the plain kernel, which takes any.  With
    ``kv_cache`` the k | v columns (from ``q_cols`` on) are also written to the cache rows
    ``slot_map``: in the product's epilogue on the matrix cores, by the write kernel otherwise."""
    if _MODE == "tuned" and _mfma_ok(a, w):
        return linear_mfma(a, w, bias, out, act, accumulate, kv_cache, slot_map, q_cols)
    linear_ref(a, w, bias, out, act, accumulate)
    if kv_cache is not None:
        _, _, Hkv, _, D = kv_cache.shape
        kv_write(out, q_cols, q_cols + Hkv * D, kv_cache, slot_map, Hkv, D)
    return out


def _attn_common(q, cache_slot, block_table, n_heads, out, name):
    _dev(q, cache_slot, block_table, out)
    _rows_2d(q, "q"); _rows_2d(out, "out")
    P, two, Hkv, page, D = cache_slot.shape
    if not (cache_slot.is_contiguous() and two == 2):
        raise KernelError(f"{name}: cache slot must be contiguous [pages,2,Hkv,page,D]")
    if not (q.shape[1] == n_heads * D and out.shape[1] == n_heads * D):
        raise KernelError(f"{name}: q/out must be [rows, Hq*D]")
    _need(q.dtype == torch.bfloat16 and cache_slot.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          f"{name}: q, cache and out must be bfloat16")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          f"{name}: block_table must be contiguous int32 [S, max_blocks]")
    return Hkv, page, D


def decode_splits(n_seqs: int, n_heads: int, max_blocks: int, page: int) -> int:
    """How many workgroups share a (sequence, head) pair's keys in decode attention (1: one workgroup a
    pair).  The library's rule (da_decode_splits in csrc/run_step.hip): from the step's shape only (pairs
    and the width of the block table), so that a recorded step keeps it."""
    return int(_lib().da_decode_splits(int(n_seqs), int(n_heads), int(max_blocks), int(page)))


def attention_decode(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                     seq_lens: torch.Tensor, n_seqs: int, n_heads: int, scale: float,
                     window: Optional[int], out: torch.Tensor, n_splits: int = 1,
                     workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One query row per sequence: row s of q belongs to sequence s and sits at position
    seq_lens[s] - 1.  With ``n_splits`` > 1 every (sequence, head) pair's keys are shared out over
    that many workgroups, whose partial results pass through ``workspace`` (float32,
    ``decode_workspace_floats`` elements)."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_decode")
    _need(q.shape[0] >= n_seqs and out.shape[0] >= n_seqs and block_table.shape[0] >= n_seqs,
          "attention_decode: fewer rows than sequences")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= n_seqs, "attention_decode: seq_lens must be int32 [S]")
    if n_splits <= 1:
        _check(_lib().da_attn_decode(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                     block_table.shape[1], _ptr(seq_lens), n_seqs, n_heads, Hkv, D, page,
                                     scale, int(window or 0), _ptr(out), out.stride(0), _stream()))
        return out
    need = decode_workspace_floats(n_seqs, n_heads, D, n_splits)
    _need(workspace is not None and workspace.dtype == torch.float32 and workspace.is_contiguous()
          and workspace.numel() >= need, f"attention_decode: the workspace must hold {need} float32")
    _dev(workspace)
    _check(_lib().da_attn_decode_split(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                       block_table.shape[1], _ptr(seq_lens), n_seqs, n_heads, Hkv, D, page,
                                       scale, int(window or 0), _ptr(out), out.stride(0), n_splits,
                                       _ptr(workspace), workspace.numel() * 4, _stream()))
    return out


def decode_workspace_floats(n_seqs: int, n_heads: int, head_dim: int, n_splits: int) -> int:
    return n_seqs * n_heads * n_splits * (head_dim + 2)


def attention_prefill(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor,
                      q_start: torch.Tensor, seq_lens: torch.Tensor, seq0: int, n_seqs: int,
                      max_query_len: int, n_heads: int, scale: float, window: Optional[int],
                      out: torch.Tensor, form: int = 0) -> torch.Tensor:
    """Portions: sequence s (seq0 <= s < seq0 + n_seqs) owns rows q_start[s] .. q_start[s+1]-1 of q
    and out; its last row sits at position seq_lens[s] - 1.  ``form``: a workgroup's row blocks of 32 and
    the wavefronts that share out a row block's keys, as a two-digit number (41: any head size; 22: up to
    128; 42 and 14: up to 64); 0 lets the kernel choose from the step's shape."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_prefill")
    _need(q_start.dtype == torch.int32 and q_start.numel() >= seq0 + n_seqs + 1, "attention_prefill: q_start must be int32 [S+1]")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= seq0 + n_seqs, "attention_prefill: seq_lens must be int32 [S]")
    _need(block_table.shape[0] >= seq0 + n_seqs, "attention_prefill: block table has fewer rows than sequences")
    _need(q.shape[0] == out.shape[0], "attention_prefill: q and out differ in rows")
    _check(_lib().da_attn_prefill(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table),
                                        block_table.shape[1], _ptr(q_start), _ptr(seq_lens), seq0, n_seqs,
                                        max_query_len, n_heads, Hkv, D, page, scale,
                                        int(window or 0), _ptr(out), out.stride(0), form, _stream()))
    return out


def paged_attention(ctx, q: torch.Tensor, cache_slot: torch.Tensor, group: int, n_heads: int,
                    scale: float, window: Optional[int], out: torch.Tensor) -> torch.Tensor:
    """Attention of every row of the step over its sequence's pages.  In bfloat16 the one-token
    sequences (the first ``ctx.n_decode``) go to the decode kernel and the portions to the
    prefill kernel; 32-bit, the reference mode and head sizes that are no multiple of 16 (which the
    matrix-core kernels do not take) use the plain kernel for all rows."""
    bt = ctx.block_tables[group]
    Hkv, page, D = cache_slot.shape[2], cache_slot.shape[3], cache_slot.shape[4]
    el = cache_slot.element_size()
    nd = ctx.n_decode
    lens, starts = ctx.seq_lens_host, ctx.q_start_host        # for the profiler's cost model only

    def cost(first, last):
        """(bytes, flops) of the sequences first..last-1: every visible key and value once, q and out once;
        two products of 2 * D flops for every (query row, visible key, head)."""
        if not KernelProfiler.enabled or not lens:
            return 0, 0
        keys = pairs = rows = 0
        for s_ in range(first, last):
            t = starts[s_ + 1] - starts[s_]
            n = lens[s_]
            lo = 0 if not window else max(0, n - t - window + 1)
            keys += n - lo
            rows += t
            pairs += sum(min(n - t + i + 1, window or n) for i in range(t)) if t > 1 else min(n, window or n)
        return keys * 2 * Hkv * D * el + 2 * rows * n_heads * D * el, 4 * pairs * n_heads * D

    if _MODE == "tuned" and q.dtype == torch.bfloat16 and D % 16 == 0 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0:
        if nd:
            n_splits = decode_splits(nd, n_heads, bt.shape[1], page)
            ws = None
            if n_splits > 1:
                ws = ctx.buf("decode_partial", 1, decode_workspace_floats(nd, n_heads, D, n_splits), torch.float32)
            with _timed("attention_decode", *cost(0, nd)):
                attention_decode(q, cache_slot, bt, ctx.seq_lens, nd, n_heads, scale, window, out, n_splits, ws)
        if ctx.n_seqs > nd:
            with _timed("attention_prefill", *cost(nd, ctx.n_seqs)):
                attention_prefill(q, cache_slot, bt, ctx.q_start, ctx.seq_lens, nd, ctx.n_seqs - nd,
                                  ctx.max_query_len, n_heads, scale, window, out)
        return out
    with _timed("attention_plain", *cost(0, ctx.n_seqs), "fp32" if q.dtype == torch.float32 else "bf16"):
        return attention_ref(q, cache_slot, bt, ctx.seq_of_token, ctx.positions, n_heads, scale, window, out)


PREFILL_REL_MAX_DIST = 1024     # entries of a bias row that the prefill kernel keeps in LDS (csrc/attn_prefill.hip)
PREFILL_REL_MAX_HEAD_DIM = 128


def _rel_bias_args(dist_bias, n_heads, name):
    if dist_bias is None:
        return None, 0
    _need(dist_bias.dtype == torch.float32 and dist_bias.is_contiguous() and dist_bias.dim() == 2
          and dist_bias.shape[0] == n_heads, f"{name}: the bias by distance must be float32 [Hq, n_dist]")
    return _ptr(dist_bias), dist_bias.shape[1]


def attention_decode_rel(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
                         n_seqs: int, n_heads: int, scale: float, window: Optional[int],
                         dist_bias: Optional[torch.Tensor], temp_coef: float, temp_every: int, out: torch.Tensor,
                         n_splits: int = 1, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``attention_decode`` with a bias by distance and a query temperature on the scores."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_decode_rel")
    _need(q.shape[0] >= n_seqs and out.shape[0] >= n_seqs and block_table.shape[0] >= n_seqs,
          "attention_decode_rel: fewer rows than sequences")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= n_seqs, "attention_decode_rel: seq_lens must be int32 [S]")
    bias_ptr, n_dist = _rel_bias_args(dist_bias, n_heads, "attention_decode_rel")
    _dev(dist_bias, workspace)
    ws_bytes = 0
    if n_splits > 1:
        need = decode_workspace_floats(n_seqs, n_heads, D, n_splits)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.is_contiguous()
              and workspace.numel() >= need, f"attention_decode_rel: the workspace must hold {need} float32")
        ws_bytes = workspace.numel() * 4
    _check(_lib().da_attn_decode_rel(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table), block_table.shape[1],
                                     _ptr(seq_lens), n_seqs, n_heads, Hkv, D, page, float(scale), int(window or 0),
                                     bias_ptr, n_dist, float(temp_coef), int(temp_every), _ptr(out), out.stride(0),
                                     int(n_splits), _ptr(workspace) if n_splits > 1 else None, ws_bytes, _stream()))
    return out


def attention_prefill_rel(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor, q_start: torch.Tensor,
                          seq_lens: torch.Tensor, seq0: int, n_seqs: int, max_query_len: int, n_heads: int, scale: float,
                          window: Optional[int], dist_bias: Optional[torch.Tensor], temp_coef: float, temp_every: int,
                          out: torch.Tensor, form: int = 0) -> torch.Tensor:
    """``attention_prefill`` with a bias by distance (up to ``PREFILL_REL_MAX_DIST`` entries a head) and a query
    temperature on the scores; head sizes up to ``PREFILL_REL_MAX_HEAD_DIM``."""
    Hkv, page, D = _attn_common(q, cache_slot, block_table, n_heads, out, "attention_prefill_rel")
    _need(q_start.dtype == torch.int32 and q_start.numel() >= seq0 + n_seqs + 1, "attention_prefill_rel: q_start must be int32 [S+1]")
    _need(seq_lens.dtype == torch.int32 and seq_lens.numel() >= seq0 + n_seqs, "attention_prefill_rel: seq_lens must be int32 [S]")
    _need(block_table.shape[0] >= seq0 + n_seqs, "attention_prefill_rel: block table has fewer rows than sequences")
    _need(q.shape[0] == out.shape[0], "attention_prefill_rel: q and out differ in rows")
    bias_ptr, n_dist = _rel_bias_args(dist_bias, n_heads, "attention_prefill_rel")
    _dev(dist_bias)
    _check(_lib().da_attn_prefill_rel(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table), block_table.shape[1],
                                      _ptr(q_start), _ptr(seq_lens), seq0, n_seqs, max_query_len, n_heads, Hkv, D, page,
                                      float(scale), int(window or 0), bias_ptr, n_dist, float(temp_coef), int(temp_every),
                                      _ptr(out), out.stride(0), form, _stream()))
    return out


def attention_window(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor, q_start: torch.Tensor,
                     seq_lens: torch.Tensor, seq0: int, n_seqs: int, max_query_len: int, n_heads: int, n_kv_heads: int,
                     head_dim: int, v_head_dim: int, page: int, scale: float, window: Optional[int], keep_first: int,
                     softcap: float, out: torch.Tensor, form: int = 0, sink: Optional[torch.Tensor] = None,
                     gate_col: int = -1) -> torch.Tensor:
    """Attention of the sequences ``seq0 .. seq0 + n_seqs - 1`` of a step on the matrix cores, in bfloat16, with keys and
    values of their own sizes, a cap on the scores and, with a window, ``keep_first`` first keys that stay visible.
    ``form``: 0 leaves the workgroup's row blocks to the kernel's rule; 1, 2 or 4 fixes them."""
    _dev(q, cache_slot, block_table, q_start, seq_lens, out, sink)
    _rows_2d(q, "q"); _rows_2d(out, "out")
    gate_ptr, gate_ld = _sink_gate_args(sink, gate_col, n_heads, n_heads * head_dim, n_heads * v_head_dim, q, "attention_window")
    _need(q.dtype == cache_slot.dtype == out.dtype == torch.bfloat16, "attention_window: q, cache and out must be bfloat16")
    _need(cache_slot.is_contiguous() and cache_page_elems(cache_slot) == n_kv_heads * page * (head_dim + v_head_dim),
          "attention_window: a page of the cache slot does not hold Hkv * page * (D + Dv) entries")
    _need((q.shape[1] == n_heads * head_dim or gate_col >= 0) and out.shape[1] == n_heads * v_head_dim and out.shape[0] == q.shape[0],
          "attention_window: q must be [N, Hq*D] and out [N, Hq*Dv]")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
          and block_table.shape[0] >= seq0 + n_seqs, "attention_window: block_table must be contiguous int32 [S, max_blocks]")
    _need(q_start.dtype == torch.int32 and q_start.numel() >= seq0 + n_seqs + 1 and seq_lens.dtype == torch.int32
          and seq_lens.numel() >= seq0 + n_seqs, "attention_window: q_start must be int32 [S+1] and seq_lens int32 [S]")
    _check(_lib().da_attn_window(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(block_table), block_table.shape[1],
                                 _ptr(q_start), _ptr(seq_lens), seq0, n_seqs, max_query_len, n_heads, n_kv_heads, head_dim,
                                 v_head_dim, page, float(scale), int(window or 0), int(keep_first if window else 0),
                                 float(softcap), _ptr(sink), gate_ptr, gate_ld, _ptr(out),
                                 out.stride(0), int(form), _stream()))
    return out


def attention_window_takes(head_dim: int, v_head_dim: int, page: int) -> bool:
    return bool(_lib().da_attn_window_takes(head_dim, v_head_dim, page))


def paged_attention_rel(ctx, q: torch.Tensor, cache_slot: torch.Tensor, group: int, n_heads: int, n_kv_heads: int,
                        head_dim: int, v_head_dim: int, scale: float, window: Optional[int],
                        dist_bias: Optional[torch.Tensor], temp_coef: float, temp_every: int,
                        out: torch.Tensor, softcap: float = 0.0, keep_first: int = 0,
                        sink: Optional[torch.Tensor] = None, gate_col: int = -1) -> torch.Tensor:
    """Attention of every row of the step with a bias by distance, a query temperature, values of their own
    size, a cap on the scores, first keys that a window keeps, a term without a key in the softmax's denominator
    (``sink``) and a logistic gate on the result (``gate_col``: where the gate lies in q's rows), each optional; the last two go with the matrix-core
    kernel for windows or the plain one.  In bfloat16, with keys and values of one size that is a multiple of 16 up to 128 and a
    bias row that fits the prefill kernel's LDS copy, the one-token sequences go to the decode kernel and the
    portions to the prefill kernel (their forms with these extras); a cap, kept first keys and values of another size
    go to the matrix-core kernel for those (head sizes up to 128, no bias table, no temperature); 32-bit, the reference
    mode and every other shape use the plain kernel for all rows."""
    bt = ctx.block_tables[group]
    page = cache_slot.shape[3] if cache_slot.dim() == 5 else ctx.cache.page_size
    D, nd = head_dim, ctx.n_decode
    el = cache_slot.element_size()
    lens, starts = ctx.seq_lens_host, ctx.q_start_host        # for the profiler's cost model only

    def cost(first, last):
        if not KernelProfiler.enabled or not lens:
            return 0, 0
        keys = pairs = rows = 0
        span = (window + keep_first) if window else 0
        for s_ in range(first, last):
            t = starts[s_ + 1] - starts[s_]
            n = lens[s_]
            keys += min(n, span + t) if span else n
            rows += t
            if span:
                pairs += sum(min(n - t + i + 1, span) for i in range(t))
            else:
                pairs += sum(n - t + i + 1 for i in range(t)) if t > 1 else n
        return (keys * n_kv_heads * (D + v_head_dim) * el + rows * n_heads * (D + v_head_dim) * el,
                2 * pairs * n_heads * (D + v_head_dim))

    tuned = (_MODE == "tuned" and q.dtype == torch.bfloat16 and v_head_dim == D and D % 16 == 0
             and softcap == 0.0 and not (window and keep_first) and sink is None and gate_col < 0
             and D <= PREFILL_REL_MAX_HEAD_DIM and cache_slot.dim() == 5 and q.stride(0) % 8 == 0
             and q.data_ptr() % 16 == 0 and (dist_bias is None or dist_bias.shape[1] <= PREFILL_REL_MAX_DIST))
    if tuned:
        if nd:
            n_splits = decode_splits(nd, n_heads, bt.shape[1], page)
            ws = None
            if n_splits > 1:
                ws = ctx.buf("decode_partial", 1, decode_workspace_floats(nd, n_heads, D, n_splits), torch.float32)
            with _timed("attention_decode", *cost(0, nd)):
                attention_decode_rel(q, cache_slot, bt, ctx.seq_lens, nd, n_heads, scale, window, dist_bias, temp_coef,
                                     temp_every, out, n_splits, ws)
        if ctx.n_seqs > nd:
            with _timed("attention_prefill", *cost(nd, ctx.n_seqs)):
                attention_prefill_rel(q, cache_slot, bt, ctx.q_start, ctx.seq_lens, nd, ctx.n_seqs - nd,
                                      ctx.max_query_len, n_heads, scale, window, dist_bias, temp_coef, temp_every, out)
        return out
    if (_MODE == "tuned" and q.dtype == torch.bfloat16 and dist_bias is None and temp_every == 0
            and attention_window_takes(D, v_head_dim, page) and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0):
        # decode rows (four key phases a row) and portions (row blocks by the longest portion) in a launch each
        if nd:
            with _timed("attention_window_decode", *cost(0, nd)):
                attention_window(q, cache_slot, bt, ctx.q_start, ctx.seq_lens, 0, nd, 1, n_heads, n_kv_heads, D,
                                 v_head_dim, page, scale, window, keep_first, softcap, out, sink=sink, gate_col=gate_col)
        if ctx.n_seqs > nd:
            with _timed("attention_window", *cost(nd, ctx.n_seqs)):
                attention_window(q, cache_slot, bt, ctx.q_start, ctx.seq_lens, nd, ctx.n_seqs - nd, ctx.max_query_len,
                                 n_heads, n_kv_heads, D, v_head_dim, page, scale, window, keep_first, softcap, out,
                                 sink=sink, gate_col=gate_col)
        return out
    with _timed("attention_plain", *cost(0, ctx.n_seqs), "fp32" if q.dtype == torch.float32 else "bf16"):
        return attention_rel_ref(q, cache_slot, bt, ctx.seq_of_token, ctx.positions, n_heads, n_kv_heads, head_dim,
                                 v_head_dim, page, scale, window, dist_bias, temp_coef, temp_every, out, softcap, keep_first,
                                 sink=sink, gate_col=gate_col)


def gated_linear(ctx, h: torch.Tensor, gate_up: torch.Tensor, mid: torch.Tensor, act: str, limit: float = 0.0) -> torch.Tensor:
    """mid = act(h @ gate.T) * (h @ up.T) with gate | up as one matrix [2 inner, width]."""
    N, inner = mid.shape
    gu = ctx.buf("ff_gate_up", N, 2 * inner, h.dtype)
    linear(h, gate_up, None, gu)
    return gated_act(gu, mid, act, limit)


def moe_top(z: torch.Tensor, bias: Optional[torch.Tensor], top: int, mode: str, renorm: bool, ids: torch.Tensor,
            weights: torch.Tensor) -> None:
    """Every row's ``top`` largest entries of z + bias (32-bit router logits; the lower index wins a tie): ids[n, k]
    and weights[n, k] in descending order.  ``mode`` "logistic": weights logistic(z) (``renorm``: divided by their
    sum); "softmax": the softmax over the chosen logits only."""
    _dev(z, bias, ids, weights)
    _rows_2d(z, "z")
    N, E = z.shape
    _need(z.dtype == torch.float32, "moe_top: router logits must be float32")
    _need(1 <= top <= E, f"moe_top: top {top} of {E}")
    _need(bias is None or (bias.is_contiguous() and bias.numel() == E), "moe_top: the bias has one entry an expert")
    _need(mode in ("logistic", "softmax"), f"moe_top: unknown mode {mode!r}")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and ids.numel() >= N * top and weights.dtype == torch.float32
          and weights.is_contiguous() and weights.numel() >= N * top, "moe_top: ids int32 and weights float32, [N, top]")
    with _timed("moe_top", N * E * 4 + N * top * 8, N * E * top, "fp32"):
        _check(_lib().da_moe_top(_ptr(z), z.stride(0), _ptr(bias), _dt(bias) if bias is not None else 0, N, E, top,
                                 1 if mode == "softmax" else 0, int(renorm), _ptr(ids), _ptr(weights), _stream()))


def _moe_mfma_ok(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> bool:
    return (_MODE == "tuned" and h.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 and h.shape[1] % 8 == 0
            and h.stride(0) % 8 == 0 and down.shape[2] % 8 == 0 and h.data_ptr() % 16 == 0
            and gate_up.data_ptr() % 16 == 0 and down.data_ptr() % 16 == 0)


def moe_top_logistic(z: torch.Tensor, top: int, renorm: bool, ids: torch.Tensor, weights: torch.Tensor) -> None:
    """Every row's ``top`` largest entries of z (32-bit router logits): ids[n, k] and weights[n, k] =
    logistic(z[n, ids[n, k]]) in descending order (the lower index wins a tie); ``renorm``: divided by their sum."""
    _dev(z, ids, weights)
    _rows_2d(z, "z")
    N, E = z.shape
    _need(z.dtype == torch.float32, "moe_top_logistic: router logits must be float32")
    _need(1 <= top <= E, f"moe_top_logistic: top {top} of {E}")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and ids.numel() >= N * top and weights.dtype == torch.float32
          and weights.is_contiguous() and weights.numel() >= N * top, "moe_top_logistic: ids int32 and weights float32, [N, top]")
    with _timed("moe_top", N * E * 4 + N * top * 8, N * E * top, "fp32"):
        _check(_lib().da_moe_top_logistic(_ptr(z), z.stride(0), N, E, top, int(renorm), _ptr(ids), _ptr(weights), _stream()))


def experts_forward(ctx, h: torch.Tensor, table: Optional[torch.Tensor], gate_up: torch.Tensor, down: torch.Tensor,
                    n_experts: int, top: int, weight: float, act: str, x: torch.Tensor, accumulate: bool,
                    ids: Optional[torch.Tensor] = None, pair_weights: Optional[torch.Tensor] = None,
                    gated: bool = True, weight_input: bool = False, limit: float = 0.0) -> torch.Tensor:
    """x (+)= sum_k weight_k * expert_k(h) (or, with ``weight_input``, sum_k expert_k(weight_k * h)): route, two
    grouped products, combine.  The experts of a row come from ``table[token, k]`` or from ``ids[n, k]``; the
    weights are ``pair_weights[n, k]`` or the one ``weight``.  ``gated``: the first matrix of an expert is gate | up
    ([2 inner, width]) and its middle is act(gate h) * (up h); else it is [inner, width] and the middle is act(up h).
    bfloat16 steps run the grouped products on the matrix cores; 32-bit and the reference mode use the plain ones."""
    N, width = h.shape
    inner = down.shape[2]
    first_rows = (2 if gated else 1) * inner
    mfma = _moe_mfma_ok(h, gate_up, down)
    # Many rows an expert (prompt portions): the rows are gathered expert by expert and go through the block
    # tiles of the dense products, a matrix per group of 128 rows.  Few (decoding): tiles of 32 rows that
    # stream each expert's weights once.  The choice reads the step's shape only.
    block = mfma and N * top >= 64 * n_experts and inner % 8 == 0
    tile = MOE_TILE_ROWS_BLOCK if block else (MOE_TILE_ROWS_MFMA if mfma else MOE_TILE_ROWS)
    tiles, rows = moe_slot_space(N, top, n_experts, tile)
    ints = ctx.buf("moe_route", N * top + rows + tiles, 1, torch.int32).view(-1)
    slot_of_pair, row_of_slot, tile_expert = ints[:N * top], ints[N * top:N * top + rows], ints[N * top + rows:]
    _need(not weight_input or pair_weights is not None, "experts: weights on the input need a weight a pair")
    # a pair's weight where its slot is: the first product scales its rows with it
    slot_scale = ctx.buf("moe_slot_scale", rows, 1, torch.float32).view(-1) if weight_input else None
    if ids is None:
        moe_route(ctx.tokens, table, None, N, top, n_experts, tile, slot_of_pair, row_of_slot, tile_expert)
    else:
        moe_route(None, None, ids, N, top, n_experts, tile, slot_of_pair, row_of_slot, tile_expert,
                  pair_weights if weight_input else None, slot_scale)
    mid = ctx.buf("moe_mid", rows, inner, h.dtype)
    pair_out = ctx.buf("moe_out", rows, width, torch.float32)
    _need(gate_up.is_contiguous() and down.is_contiguous() and tuple(gate_up.shape) == (n_experts, first_rows, width)
          and tuple(down.shape) == (n_experts, width, inner), "experts: stacked weights of the wrong shape")
    _dev(h, gate_up, down)
    if not (act in ACTIVATIONS):
        raise KernelError(f"experts: unknown activation {act!r}")
    if block:
        hs = ctx.buf("moe_rows", rows, width, h.dtype)
        with _timed("experts_gather", 2 * N * top * width * 2, 0):
            _check(_lib().da_moe_gather(_ptr(h), h.stride(0), _ptr(row_of_slot), _ptr(hs), rows, width, _stream(),
                                        _ptr(slot_scale)))
        if gated:
            gu = ctx.buf("moe_gate_up", rows, 2 * inner, h.dtype)
            with _timed("experts_gate_up", N * top * (width + 2 * inner) * 2 + _nbytes(gate_up), 4 * N * top * inner * width):
                _check(_lib().da_gemm_bf16_grouped(_ptr(hs), hs.stride(0), _ptr(gate_up), width, 2 * inner * width,
                                                   _ptr(tile_expert), tile, _ptr(gu), BF16, gu.stride(0), rows, 2 * inner, width,
                                                   _stream(), 0))
            gated_act(gu, mid, act, limit)
        else:                      # the activation rides in the product's epilogue
            with _timed("experts_up", N * top * (width + inner) * 2 + _nbytes(gate_up), 2 * N * top * inner * width):
                _check(_lib().da_gemm_bf16_grouped(_ptr(hs), hs.stride(0), _ptr(gate_up), width, inner * width,
                                                   _ptr(tile_expert), tile, _ptr(mid), BF16, mid.stride(0), rows, inner, width,
                                                   _stream(), ACTIVATIONS[act]))
        with _timed("experts_down", N * top * (inner * 2 + width * 4) + _nbytes(down), 2 * N * top * inner * width):
            _check(_lib().da_gemm_bf16_grouped(_ptr(mid), mid.stride(0), _ptr(down), inner, width * inner,
                                               _ptr(tile_expert), tile, _ptr(pair_out), F32, pair_out.stride(0), rows, width,
                                               inner, _stream(), 0))
    elif mfma:
        # every expert's weights once (decode: what the step must move), the pairs' rows in and out
        nb = N * top * (width * 2 + inner * 2) + min(n_experts, N * top) * first_rows * width * 2
        if gated:
            with _timed("experts_gated", nb, 4 * N * top * inner * width):
                _check(_lib().da_moe_gated_mfma(_ptr(h), h.stride(0), _ptr(row_of_slot), _ptr(tile_expert), _ptr(gate_up),
                                                _ptr(mid), mid.stride(0), tiles, width, inner, ACTIVATIONS[act], float(limit),
                                                _stream()))
        else:
            with _timed("experts_up", nb, 2 * N * top * inner * width):
                _check(_lib().da_moe_up_mfma(_ptr(h), h.stride(0), _ptr(row_of_slot), _ptr(tile_expert), _ptr(gate_up),
                                             _ptr(slot_scale), _ptr(mid), mid.stride(0), tiles, width, inner,
                                             ACTIVATIONS[act], _stream()))
        nb = N * top * (inner * 2 + width * 4) + min(n_experts, N * top) * inner * width * 2
        with _timed("experts_down", nb, 2 * N * top * inner * width):
            _check(_lib().da_moe_down_mfma(_ptr(mid), mid.stride(0), _ptr(row_of_slot), _ptr(tile_expert), _ptr(down),
                                           _ptr(pair_out), pair_out.stride(0), tiles, inner, width, _stream()))
    else:
        if gated:
            moe_gated_ref(h, row_of_slot, tile_expert, gate_up, mid, tiles, act, limit)
        else:
            _moe_common(h, row_of_slot, tile_expert, gate_up, tiles, MOE_TILE_ROWS, "moe_up")
            with _timed("moe_up_plain", _nbytes(h, gate_up, mid), 2 * tiles * MOE_TILE_ROWS * inner * width,
                        "fp32" if h.dtype == torch.float32 else "bf16"):
                _check(_lib().da_moe_up_ref(_ptr(h), h.stride(0), _dt(h), _ptr(row_of_slot), _ptr(tile_expert), _ptr(gate_up),
                                            _ptr(slot_scale), _ptr(mid), mid.stride(0), tiles, width, inner, ACTIVATIONS[act],
                                            _stream()))
        moe_down_ref(mid, row_of_slot, tile_expert, down, pair_out, tiles)
    if weight_input:               # the weights already sit in the rows
        return moe_combine(pair_out, slot_of_pair, None, 1.0, top, x, accumulate)
    return moe_combine(pair_out, slot_of_pair, pair_weights, weight, top, x, accumulate)


# ------------------------------------------------------------------------------- rotation, latent attention
LATENT_MAX_ROW = 1024        # entries of a latent cache row that the attention kernels take (csrc/attn_latent.hip)
CONV_MAX_TAPS = 16           # taps of a short filter (csrc/ssm.hip)
SCAN_MAX_STATE = 1024        # state entries a channel of the scan


def linear_heads(a: torch.Tensor, a_head_stride: int, a_off: int, w: torch.Tensor, out: torch.Tensor,
                 out_head_stride: int, out_off: int) -> torch.Tensor:
    """A product per head: out[:, h * out_head_stride + out_off : .. + n] = a[:, h * a_head_stride + a_off : .. + k]
    @ w[h].T for the stack w [heads, n, k]; the heads' pieces lie side by side in the rows of a and out."""
    _rows_2d(a, "a"); _rows_2d(out, "out")
    H, n, k = w.shape
    M = a.shape[0]
    _need(a.shape[1] >= (H - 1) * a_head_stride + a_off + k and out.shape[1] >= (H - 1) * out_head_stride + out_off + n
          and out.shape[0] == M, "linear_heads: the heads leave the rows")
    if (_MODE == "tuned" and a.dtype == w.dtype == out.dtype == torch.bfloat16 and w.is_contiguous()
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and bool(_lib().da_gemm_heads_takes(a.stride(0), a_head_stride, a_off, k))):
        _dev(a, w, out)
        with _timed("product_heads", _nbytes(w) + M * H * (n + k) * 2, 2 * M * H * n * k):
            _check(_lib().da_gemm_heads(_ptr(a), a.stride(0), a_head_stride, a_off, _ptr(w), _ptr(out), out.stride(0),
                                        out_head_stride, out_off, M, H, n, k, _stream()))
        return out
    for h in range(H):
        linear(a[:, h * a_head_stride + a_off:h * a_head_stride + a_off + k], w[h], None,
               out[:, h * out_head_stride + out_off:h * out_head_stride + out_off + n])
    return out


def rotary(src: torch.Tensor, dst: torch.Tensor, positions: torch.Tensor, speeds: torch.Tensor, n_heads: int,
           src_head_stride: int, dst_head_stride: int, width: int, dims: int, interleaved: bool = True,
           magnitude: float = 1.0) -> torch.Tensor:
    """dst[n, h, :width] = src[n, h, :width] with the first ``dims`` entries of every head turned in pairs by the angle
    positions[n] * speeds[i] (float64 [dims / 2]); pairs are (2i, 2i + 1) when ``interleaved``, else (i, i + dims/2).
    Heads start ``*_head_stride`` entries apart in a row; src and dst may be views into wider rows."""
    _dev(src, dst, positions, speeds)
    _rows_2d(src, "src"); _rows_2d(dst, "dst")
    N = src.shape[0]
    _need(dst.shape[0] == N and src.dtype == dst.dtype, "rotary: src and dst differ in rows or dtype")
    _need(positions.dtype == torch.int32 and positions.numel() >= N, "rotary: positions must be int32 [N]")
    _need(speeds.dtype == torch.float64 and speeds.is_contiguous() and speeds.numel() >= dims // 2,
          "rotary: speeds must be float64 [dims / 2]")
    _need(src.shape[1] >= (n_heads - 1) * src_head_stride + width and dst.shape[1] >= (n_heads - 1) * dst_head_stride + width,
          "rotary: the heads leave the row")
    with _timed("rotary", 2 * N * n_heads * width * src.element_size(), 3 * N * n_heads * dims, "fp32"):
        _check(_lib().da_rotary(_ptr(src), src.stride(0), src_head_stride, _ptr(dst), dst.stride(0), dst_head_stride,
                                _dt(src), _ptr(positions), _ptr(speeds), N, n_heads, width, dims, int(interleaved),
                                float(magnitude), _stream()))
    return dst


def latent_partial_floats(n_seqs: int, max_query_len: int, n_heads: int, v_dim: int, n_splits: int) -> int:
    """Entries of the 32-bit scratch that the matrix-core latent attention needs to share keys out (blocks of 64 rows)."""
    return n_seqs * (-(-max_query_len * n_heads // 64)) * 64 * n_splits * (v_dim + 2)


def latent_cache_row(cache_slot: torch.Tensor, page: int) -> int:
    """Entries of a row of a latent cache slot [pages, page * D]."""
    return cache_slot[0].numel() // page


def latent_prepare(down: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, q_gain: Optional[torch.Tensor],
                   kv_gain: torch.Tensor, eps: float, positions: torch.Tensor, slot_map: Optional[torch.Tensor],
                   speeds: torch.Tensor, dims: int, interleaved: bool, cq: Optional[torch.Tensor],
                   cache_slot: torch.Tensor, page: int, magnitude: float = 1.0) -> None:
    """From rows [ query latent (q_rank) | latent (kv_rank) | key piece (rot_dim) ] of ``down``: cq = rms(query
    latent) * q_gain; the cache row slot_map[n] = [ rms(latent) * kv_gain | the key piece turned by the position ]."""
    _dev(down, q_gain, kv_gain, positions, slot_map, speeds, cq, cache_slot)
    _rows_2d(down, "down")
    N = down.shape[0]
    _need(down.shape[1] >= q_rank + kv_rank + rot_dim, "latent_prepare: rows shorter than the three pieces")
    _need(cache_slot.is_contiguous() and latent_cache_row(cache_slot, page) == kv_rank + rot_dim,
          "latent_prepare: a row of the cache slot does not hold latent + key piece")
    _need(kv_gain.numel() == kv_rank and (q_rank == 0 or (q_gain is not None and q_gain.numel() == q_rank and cq is not None)),
          "latent_prepare: gains differ from the ranks")
    if cq is not None:
        _rows_2d(cq, "cq")
        _need(cq.shape[0] >= N and cq.shape[1] >= q_rank and cq.dtype == cache_slot.dtype, "latent_prepare: cq [N, q_rank] of the cache's dtype")
    _need(positions.dtype == torch.int32 and positions.numel() >= N and (slot_map is None or (slot_map.dtype == torch.int32 and slot_map.numel() >= N)),
          "latent_prepare: positions and slot_map must be int32 [N]")
    _need(speeds.dtype == torch.float64 and speeds.is_contiguous() and speeds.numel() >= dims // 2, "latent_prepare: speeds float64 [dims / 2]")
    with _timed("latent_prepare", N * (q_rank + kv_rank + rot_dim) * (down.element_size() + cache_slot.element_size()), 6 * N * (q_rank + kv_rank + rot_dim), "fp32"):
        _check(_lib().da_latent_prepare(_ptr(down), _dt(down), down.stride(0), q_rank, kv_rank, rot_dim, _ptr(q_gain),
                                        _dt(q_gain) if q_gain is not None else 0, _ptr(kv_gain), _dt(kv_gain), float(eps),
                                        _ptr(positions), _ptr(slot_map), _ptr(speeds), dims, int(interleaved), float(magnitude), _ptr(cq),
                                        cq.stride(0) if cq is not None else 0, _ptr(cache_slot), _dt(cache_slot), page, N,
                                        _stream()))


def attention_latent_ref(q: torch.Tensor, cache_slot: torch.Tensor, block_table: torch.Tensor, seq_of_token: torch.Tensor,
                         positions: torch.Tensor, n_heads: int, row_dim: int, v_dim: int, page: int, scale: float,
                         window: Optional[int], out: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Plain attention over a latent cache: q [N, Hq * row_dim] (the key maps folded in), out [N, Hq * v_dim] = the
    weighted sums of the rows' first v_dim entries.  ``sink`` (float32 [Hq]): exp(sink[h]) joins the denominator."""
    _dev(q, cache_slot, block_table, seq_of_token, positions, out, sink)
    _sink_gate_args(sink, -1, n_heads, 0, 0, q, "attention_latent")
    _rows_2d(q, "q"); _rows_2d(out, "out")
    N = q.shape[0]
    _need(cache_slot.is_contiguous() and latent_cache_row(cache_slot, page) == row_dim, "attention_latent: the cache rows differ from q's")
    _need(q.shape[1] == n_heads * row_dim and out.shape[1] == n_heads * v_dim and out.shape[0] == N and v_dim <= row_dim,
          "attention_latent: q must be [N, Hq*D] and out [N, Hq*Dv]")
    _need(q.dtype == cache_slot.dtype == out.dtype, "attention_latent: q, cache and out must share a dtype")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "attention_latent: block_table must be contiguous int32 [S, max_blocks]")
    _need(seq_of_token.dtype == torch.int32 and positions.dtype == torch.int32 and seq_of_token.numel() >= N
          and positions.numel() >= N, "attention_latent: ids must be int32, one a row")
    _check(_lib().da_attn_latent_ref(_ptr(q), q.stride(0), _ptr(cache_slot), _dt(q), _ptr(block_table), block_table.shape[1],
                                     _ptr(seq_of_token), _ptr(positions), N, n_heads, row_dim, v_dim, page, float(scale),
                                     int(window or 0), _ptr(sink), _ptr(out), out.stride(0), _stream()))
    return out


def paged_attention_latent(ctx, q: torch.Tensor, cache_slot: torch.Tensor, group: int, n_heads: int, row_dim: int,
                           v_dim: int, scale: float, window: Optional[int], out: torch.Tensor,
                           sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of every row of the step over its sequence's latent rows (``sink``: see ``attention_latent_ref``)."""
    bt = ctx.block_tables[group]
    page = ctx.cache.page_size
    el = cache_slot.element_size()
    lens, starts = ctx.seq_lens_host, ctx.q_start_host        # for the profiler's cost model only

    def cost(first=0, last=None):
        if not KernelProfiler.enabled or not lens:
            return 0, 0
        keys = pairs = rows = 0
        for s_ in range(first, ctx.n_seqs if last is None else last):
            t = starts[s_ + 1] - starts[s_]
            n = lens[s_]
            keys += min(n, window + t) if window else n
            rows += t
            if window:
                pairs += sum(min(n - t + i + 1, window) for i in range(t))
            else:
                pairs += sum(n - t + i + 1 for i in range(t)) if t > 1 else n
        return keys * row_dim * el + rows * n_heads * (row_dim + v_dim) * el, 2 * pairs * n_heads * (row_dim + v_dim)

    if (_MODE == "tuned" and q.dtype == torch.bfloat16 and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0
            and bool(_lib().da_attn_latent_mfma_takes(row_dim, v_dim))):
        # prompt portions and decoded tokens alike: the query rows of a workgroup are (token, head) pairs
        _dev(q, cache_slot, bt, out, sink)
        _rows_2d(q, "q"); _rows_2d(out, "out")
        _sink_gate_args(sink, -1, n_heads, 0, 0, q, "attention_latent")
        _need(cache_slot.is_contiguous() and cache_slot.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
              and latent_cache_row(cache_slot, page) == row_dim, "attention_latent: a bfloat16 cache of rows like q's")
        _need(q.shape[1] == n_heads * row_dim and out.shape[1] == n_heads * v_dim and out.shape[0] == q.shape[0],
              "attention_latent: q must be [N, Hq*D] and out [N, Hq*Dv]")
        _need(bt.dtype == torch.int32 and bt.dim() == 2 and bt.is_contiguous() and bt.shape[0] >= ctx.n_seqs,
              "attention_latent: block_table must be contiguous int32 [S, max_blocks]")
        nd = ctx.n_decode

        def go(seq0, n_seqs, max_q, n_splits, ws):
            _check(_lib().da_attn_latent_mfma(_ptr(q), q.stride(0), _ptr(cache_slot), _ptr(bt), bt.shape[1], _ptr(ctx.q_start),
                                              _ptr(ctx.seq_lens), seq0, n_seqs, max_q, n_heads, row_dim, v_dim, page,
                                              float(scale), int(window or 0), _ptr(out), out.stride(0), n_splits, _ptr(ws),
                                              0 if ws is None else ws.numel(), _ptr(sink), _stream()))
        if nd:                 # one-token sequences: the keys of a token's heads shared out over workgroups
            n_splits = int(_lib().da_attn_latent_splits(nd, n_heads, bt.shape[1], page))
            ws = None
            if n_splits > 1:
                ws = ctx.buf("latent_partial", 1, latent_partial_floats(nd, 1, n_heads, v_dim, n_splits), torch.float32)
            with _timed("attention_latent_decode", *cost(0, nd)):
                go(0, nd, 1, n_splits, ws)
        if ctx.n_seqs > nd:
            with _timed("attention_latent", *cost(nd, ctx.n_seqs)):
                go(nd, ctx.n_seqs - nd, ctx.max_query_len, 1, None)
        return out
    with _timed("attention_latent_plain", *cost(), "fp32" if q.dtype == torch.float32 else "bf16"):
        return attention_latent_ref(q, cache_slot, bt, ctx.seq_of_token, ctx.positions, n_heads, row_dim, v_dim, page,
                                    scale, window, out, sink=sink)


# ------------------------------------------------------------------------------- retention
RETENTION_MAX_DIM = 256      # key entries a head of the retention kernel (csrc/retention.hip)
RETENTION_CHUNK = 128        # tokens of a chunk when a long portion's walk is cut up
RETENTION_CHUNK_FROM = 256   # portions from this length on are cut up (bfloat16 serving only)


def retention(ctx, qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, decay: torch.Tensor, k_scale: float,
              state: torch.Tensor, o: torch.Tensor, n_heads: int, head_dim: int, v_head_dim: int,
              write: bool = True, chunk: Optional[int] = None) -> torch.Tensor:
    """Per head S <- decay[h] S + k v^T, o = S^T q over every sequence of the step, token by token (csrc/retention.hip).
    ``chunk``: tokens of the chunks that long portions are walked in, side by side (0: every portion in one piece; None:
    ``RETENTION_CHUNK`` in bfloat16 serving when the step's longest portion has ``RETENTION_CHUNK_FROM`` rows, else 0).
    ``qkv`` [N, ...] holds the turned q and k (H * D entries each, from columns ``q_off`` and ``k_off``) and v (H * Dv
    from ``v_off``) in the step's dtype; k is multiplied by ``k_scale``; ``decay`` float32 [H]; ``state`` [slots, >= H * Dv
    * D] 32-bit is read at each portion's start and, with ``write``, written at its end; ``o`` [N, H * Dv] 32-bit."""
    _dev(qkv, decay, state, o)
    _rows_2d(qkv, "qkv"); _rows_2d(o, "o")
    N = qkv.shape[0]
    H, D, Dv = n_heads, head_dim, v_head_dim
    ld = _state_args(state, "retention")
    _need(1 <= D <= RETENTION_MAX_DIM, f"retention: a key size of {D} is outside 1..{RETENTION_MAX_DIM}")
    _need(min(q_off, k_off, v_off) >= 0 and max(q_off, k_off) + H * D <= qkv.shape[1] and v_off + H * Dv <= qkv.shape[1],
          "retention: q, k and v leave the row")
    _need(o.dtype == torch.float32 and o.shape[0] == N and o.shape[1] >= H * Dv, "retention: o must be float32 [N, H * Dv]")
    _need(decay.dtype == torch.float32 and decay.is_contiguous() and decay.numel() == H, "retention: decay must be float32 [H]")
    _need(ld >= H * Dv * D, "retention: the state row is too short")
    _need(ctx.q_start.numel() >= ctx.n_seqs + 1 and ctx.state_slots.numel() >= ctx.n_seqs, "retention: the step's arrays are too short")
    longest = int(getattr(ctx, "max_query_len", 0) or 0)
    if chunk is None:
        chunk = RETENTION_CHUNK if (_MODE == "tuned" and qkv.dtype == torch.bfloat16 and longest >= RETENTION_CHUNK_FROM) else 0
    n_chunks, ends = 1, None
    if chunk:
        _need(chunk % 16 == 0 and longest > 0, "retention: chunks are multiples of 16 tokens and need the longest portion's length")
        n_chunks = -(-longest // chunk)
        ends = ctx.buf("retention_ends", ctx.n_seqs * n_chunks, H * Dv * D, torch.float32)
    nb = N * ((2 * H * D + H * Dv) * qkv.element_size() + H * Dv * 4) + 2 * ctx.n_seqs * H * Dv * D * 4
    with _timed("retention", nb, 4 * N * H * D * Dv, "fp32"):
        _check(_lib().da_retention(_ptr(qkv), _dt(qkv), qkv.stride(0), int(q_off), int(k_off), int(v_off), _ptr(decay),
                                   float(k_scale), _ptr(state), ld, _ptr(ctx.state_slots), _ptr(ctx.q_start), _ptr(o),
                                   o.stride(0), ctx.n_seqs, H, D, Dv, int(bool(write)), int(chunk), n_chunks, _ptr(ends),
                                   0 if ends is None else ends.numel(), _stream()))
    return o


# ------------------------------------------------------------------------------- short filter and scan
def _state_args(state: torch.Tensor, name: str):
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous(), f"{name}: the state must be contiguous float32 [slots, row]")
    return state.stride(0)


def conv_causal(ctx, x: torch.Tensor, state: torch.Tensor, conv_off: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
                act: Optional[str], y: torch.Tensor) -> torch.Tensor:
    """y[n, c] = act(bias[c] + sum_k weight[c, k] * x[n - (K - 1 - k), c]) within each sequence of the step; rows before
    the step's portion are the K - 1 inputs that ``state[slot, conv_off:]`` keeps ([K - 1, C], oldest first)."""
    _dev(x, state, weight, bias, y)
    _rows_2d(x, "x"); _rows_2d(y, "y")
    N, C = y.shape
    K = weight.shape[1]
    ld = _state_args(state, "conv_causal")
    _need(x.shape[0] == N and x.shape[1] >= C and x.dtype == y.dtype, "conv_causal: x and y differ")
    _need(weight.is_contiguous() and tuple(weight.shape) == (C, K) and (bias is None or bias.numel() == C), "conv_causal: weight [C, K], bias [C]")
    _need(ld >= conv_off + (K - 1) * C, "conv_causal: the state row is too short")
    if not (act in ACTIVATIONS):
        raise KernelError(f"conv_causal: unknown activation {act!r}")
    with _timed("conv_causal", N * C * (x.element_size() * 2), 2 * N * C * K, "fp32"):
        _check(_lib().da_conv_causal(_ptr(x), _dt(x), x.stride(0), _ptr(state), ld, conv_off, _ptr(ctx.state_slots),
                                     _ptr(ctx.seq_of_token), _ptr(ctx.q_start), _ptr(weight), _dt(weight), _ptr(bias),
                                     _dt(bias) if bias is not None else 0, ACTIVATIONS[act], _ptr(y), y.stride(0), N, C, K,
                                     _stream()))
    return y


def conv_state_update(ctx, x: torch.Tensor, state: torch.Tensor, conv_off: int, channels: int, taps: int) -> None:
    """After the step, ``state[slot, conv_off:]`` holds each sequence's last taps - 1 inputs."""
    _dev(x, state)
    _rows_2d(x, "x")
    ld = _state_args(state, "conv_state_update")
    _need(x.shape[1] >= channels and ld >= conv_off + (taps - 1) * channels, "conv_state_update: sizes differ")
    _check(_lib().da_conv_state_update(_ptr(x), _dt(x), x.stride(0), _ptr(state), ld, conv_off, _ptr(ctx.state_slots),
                                       _ptr(ctx.q_start), ctx.n_seqs, channels, taps, _stream()))


SCAN_CHUNK = 32               # tokens of a chunk when a long portion's scan is cut up
SCAN_CHUNK_FROM = 128         # portions from this length on are cut up


def scan_rates(a_log: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """What ``selective_scan`` takes for A = -exp(A_log), in 32-bit: for bfloat16 rows A log2(e), so that a decay
    exp(dt A) is one exp2 of the hardware; for 32-bit rows A itself (the kernel then calls the library's expf)."""
    a = -torch.exp(a_log.to(torch.float32))
    return (a * 1.4426950408889634 if dtype == torch.bfloat16 else a).contiguous()


def selective_scan(ctx, x: torch.Tensor, raw_dt: torch.Tensor, bc: torch.Tensor, b_off: int, c_off: int, z: torch.Tensor,
                   a2: torch.Tensor, d: Optional[torch.Tensor], state: torch.Tensor, y: torch.Tensor, n_state: int) -> torch.Tensor:
    """The scan of a selective state-space mixer over every sequence of the step (see csrc/ssm.hip), ``a2`` from
    ``scan_rates``; the state
    [slots, >= inner * n_state] is read at each portion's start and written at its end.  Steps whose longest portion
    has ``SCAN_CHUNK_FROM`` tokens or more are cut into chunks of ``SCAN_CHUNK`` that run side by side (bfloat16 rows;
    the 32-bit path walks every portion in order, as the recurrence is written)."""
    _dev(x, raw_dt, bc, z, a2, d, state, y)
    for t_, nm in ((x, "x"), (raw_dt, "raw_dt"), (bc, "bc"), (z, "z"), (y, "y")):
        _rows_2d(t_, nm)
    N, inner = y.shape
    ld = _state_args(state, "selective_scan")
    _need(x.shape[0] == N and raw_dt.shape[0] == N and bc.shape[0] == N and z.shape[0] == N, "selective_scan: rows differ")
    _need(raw_dt.dtype == torch.float32 and x.dtype == y.dtype == bc.dtype == z.dtype, "selective_scan: step sizes in float32, the rest of one dtype")
    _need(a2.is_contiguous() and a2.dtype == torch.float32 and tuple(a2.shape) == (inner, n_state) and (d is None or d.numel() == inner),
          "selective_scan: rates float32 [inner, state], D [inner]")
    chunk = max_chunks = 0
    cs = cd = None
    if ctx.max_query_len >= SCAN_CHUNK_FROM and x.dtype == torch.bfloat16:
        chunk = SCAN_CHUNK
        max_chunks = -(-ctx.max_query_len // chunk)
        cs = ctx.buf("scan_chunk_state", ctx.n_seqs * max_chunks, inner * n_state, torch.float32)
        cd = ctx.buf("scan_chunk_dt", ctx.n_seqs * max_chunks, inner, torch.float32)
    with _timed("selective_scan", N * inner * (x.element_size() * 3 + 4) + N * 2 * n_state * x.element_size(),
                N * inner * n_state * 6 * (2 if chunk else 1), "fp32"):
        _check(_lib().da_selective_scan(_ptr(x), _dt(x), x.stride(0), _ptr(raw_dt), raw_dt.stride(0), _ptr(bc), bc.stride(0),
                                        b_off, c_off, _ptr(z), z.stride(0), _ptr(a2), _ptr(d),
                                        _dt(d) if d is not None else 0, _ptr(state), ld, _ptr(ctx.state_slots), _ptr(ctx.q_start),
                                        _ptr(y), y.stride(0), ctx.n_seqs, inner, n_state, chunk, max_chunks, _ptr(cs), _ptr(cd),
                                        _stream()))
    return y


# ------------------------------------------------------------------------------- gated delta rule, attention extras
DELTA_MAX_DIM = 256          # key entries a head of the delta rule (csrc/delta.hip)
PREPARE_MAX_ROT = 256        # turned entries a head that ``attn_prepare`` takes (csrc/attn_prepare.hip)


def attn_prepare(raw: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int,
                 q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float, whole: bool,
                 positions: torch.Tensor, speeds: Optional[torch.Tensor], dims: int, interleaved: bool, q_out: torch.Tensor,
                 cache_slot: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], page: int,
                 values_are_keys: bool = False, pass_cols: int = 0, magnitude: float = 1.0) -> torch.Tensor:
    """From the 32-bit rows of a q | k | v product: queries and keys normalised (``whole``: one root mean square
    over all of a token's query entries and one over all its key entries, gains of those lengths; else head by
    head with gains of ``head_dim`` entries; no gains: no norm), their first ``dims`` entries turned by the
    position (``speeds`` float64 [dims / 2]; pairs (2i, 2i + 1) when ``interleaved``, else (i, i + dims / 2)),
    the queries stored in ``q_out`` and keys and values in their cache rows ``slot_map`` (a page of the slot
    holds Hkv * page * D keys, then Hkv * Dv * page values).  ``values_are_keys``: the rows hold q | k only, and a key
    before its turn is also the value.  ``pass_cols``: so many columns behind q | k | v go over into ``q_out`` behind the
    queries, converted.  ``magnitude`` multiplies sine and cosine."""
    _dev(raw, q_gain, k_gain, positions, speeds, q_out, cache_slot, slot_map)
    _rows_2d(raw, "raw"); _rows_2d(q_out, "q_out")
    N = raw.shape[0]
    q_cols, k_cols, v_cols = n_heads * head_dim, n_kv_heads * head_dim, 0 if values_are_keys else n_kv_heads * v_head_dim
    _need(not values_are_keys or v_head_dim == head_dim, "attn_prepare: values that are the keys have the keys' size")
    _need(raw.dtype == torch.float32 and pass_cols >= 0 and raw.shape[1] >= q_cols + k_cols + v_cols + pass_cols,
          "attn_prepare: raw must be float32 [N, q | k | v | what passes]")
    _need(q_out.shape[0] == N and q_out.shape[1] >= q_cols + pass_cols, "attn_prepare: q_out must be [N, Hq * D + what passes]")
    _need((q_gain is None) == (k_gain is None), "attn_prepare: a norm needs both gains")
    if q_gain is not None:
        nq, nk = (q_cols, k_cols) if whole else (head_dim, head_dim)
        _need(q_gain.is_contiguous() and k_gain.is_contiguous() and q_gain.numel() == nq and k_gain.numel() == nk,
              f"attn_prepare: gains of {nq} and {nk} entries are needed")
    _need(dims % 2 == 0 and 0 <= dims <= min(head_dim, PREPARE_MAX_ROT), f"attn_prepare: {dims} turned entries of {head_dim}")
    if dims:
        _need(positions.dtype == torch.int32 and positions.numel() >= N, "attn_prepare: positions must be int32 [N]")
        _need(speeds is not None and speeds.dtype == torch.float64 and speeds.is_contiguous() and speeds.numel() >= dims // 2,
              "attn_prepare: speeds must be float64 [dims / 2]")
    if cache_slot is not None:
        _need(slot_map is not None and slot_map.dtype == torch.int32 and slot_map.numel() >= N, "attn_prepare: slot_map must be int32 [N]")
        _need(cache_slot.is_contiguous() and cache_page_elems(cache_slot) == n_kv_heads * page * (head_dim + v_head_dim),
              "attn_prepare: a page of the cache slot does not hold Hkv * page * (D + Dv) entries")
        _need(cache_slot.dtype == q_out.dtype, "attn_prepare: cache and queries differ in dtype")
    with _timed("attn_prepare", N * (q_cols + k_cols + v_cols) * (4 + q_out.element_size()), 8 * N * (q_cols + k_cols), "fp32"):
        _check(_lib().da_attn_prepare(_ptr(raw), raw.stride(0), n_heads, n_kv_heads, head_dim, v_head_dim, _ptr(q_gain),
                                      _dt(q_gain) if q_gain is not None else 0, _ptr(k_gain),
                                      _dt(k_gain) if k_gain is not None else 0, float(eps), int(bool(whole)), _ptr(positions),
                                      _ptr(speeds) if dims else None, int(dims), int(bool(interleaved)), _ptr(q_out),
                                      _dt(q_out), q_out.stride(0), _ptr(cache_slot),
                                      _ptr(slot_map) if cache_slot is not None else None, int(page), N,
                                      int(bool(values_are_keys)), int(pass_cols), float(magnitude), _stream()))
    return q_out


def delta_rule(ctx, qkv: torch.Tensor, k_off: int, v_off: int, beta_raw: torch.Tensor, decay_raw: torch.Tensor,
               dt_bias: torch.Tensor, rate: torch.Tensor, state: torch.Tensor, o: torch.Tensor, n_heads: int,
               n_kv_heads: int, head_dim: int, v_head_dim: int, channel_decay: bool, unit_eps: float,
               write: bool = True, decay_off: int = 0) -> torch.Tensor:
    """The gated delta rule over every sequence of the step (see csrc/delta.hip).  ``qkv`` [N, q | k | v] after the
    filters; ``beta_raw`` [N, H] and ``decay_raw`` [N, H] (or [N, H * D] with ``channel_decay``; from column
    ``decay_off`` on, so that both may be the rows of one product) are 32-bit sums before their functions; ``rate`` = exp(A_log) [H]; ``state`` [slots, >= H * Dv * D] is read at each portion's
    start and, with ``write``, written at its end; ``o`` [N, H * Dv] 32-bit."""
    _dev(qkv, beta_raw, decay_raw, dt_bias, rate, state, o)
    for t_, nm in ((qkv, "qkv"), (beta_raw, "beta_raw"), (decay_raw, "decay_raw"), (o, "o")):
        _rows_2d(t_, nm)
    N = qkv.shape[0]
    H, G, D, Dv = n_heads, n_kv_heads, head_dim, v_head_dim
    ld = _state_args(state, "delta_rule")
    n_decay = H * D if channel_decay else H
    _need(H % G == 0 and 1 <= D <= DELTA_MAX_DIM, f"delta_rule: {H} heads on {G} key heads of {D} entries")
    _need(k_off >= G * D and v_off >= k_off + G * D and qkv.shape[1] >= v_off + H * Dv, "delta_rule: q, k and v leave the row")
    _need(beta_raw.shape[0] == N and decay_raw.shape[0] == N and o.shape[0] == N, "delta_rule: rows differ")
    _need(beta_raw.dtype == decay_raw.dtype == o.dtype == torch.float32 and beta_raw.shape[1] >= H
          and decay_raw.shape[1] >= decay_off + n_decay and o.shape[1] >= H * Dv, "delta_rule: beta, decay and o must be float32 of H, H (* D) and H * Dv columns")
    _need(dt_bias.dtype == rate.dtype == torch.float32 and dt_bias.is_contiguous() and rate.is_contiguous()
          and dt_bias.numel() == n_decay and rate.numel() == H, "delta_rule: dt_bias and rate must be float32")
    _need(ld >= H * Dv * D, "delta_rule: the state row is too short")
    _need(ctx.q_start.numel() >= ctx.n_seqs + 1 and ctx.state_slots.numel() >= ctx.n_seqs, "delta_rule: the step's arrays are too short")
    nb = N * ((2 * G * D + H * Dv) * qkv.element_size() + (H + n_decay + H * Dv) * 4) + 2 * ctx.n_seqs * H * Dv * D * 4
    with _timed("delta_rule", nb, 8 * N * H * D * Dv, "fp32"):
        _check(_lib().da_delta_rule(_ptr(qkv), _dt(qkv), qkv.stride(0), k_off, v_off, _ptr(beta_raw), beta_raw.stride(0),
                                    _ptr(decay_raw), decay_raw.stride(0), int(decay_off), _ptr(dt_bias), _ptr(rate), _ptr(state), ld,
                                    _ptr(ctx.state_slots), _ptr(ctx.q_start), _ptr(o), o.stride(0), ctx.n_seqs, H, G, D, Dv,
                                    int(bool(channel_decay)), float(unit_eps), int(bool(write)),
                                    int(getattr(ctx, "max_query_len", 0) or 0), _stream()))
    return o


def delta_gate_norm(o: torch.Tensor, gate: torch.Tensor, gain: torch.Tensor, eps: float, act: str, n_heads: int,
                    v_head_dim: int, y: torch.Tensor) -> torch.Tensor:
    """y[n, h, :] = o[n, h, :] / sqrt(mean(o[n, h, :]^2) + eps) * gain * act(gate[n, h, :]); ``act``: "silu" or
    "sigmoid"; o 32-bit, gate and y in the step's dtype."""
    _dev(o, gate, gain, y)
    for t_, nm in ((o, "o"), (gate, "gate"), (y, "y")):
        _rows_2d(t_, nm)
    N, cols = o.shape[0], n_heads * v_head_dim
    _need(o.dtype == torch.float32 and gate.dtype == y.dtype and gate.shape[0] == N and y.shape[0] == N
          and o.shape[1] >= cols and gate.shape[1] >= cols and y.shape[1] >= cols, "delta_gate_norm: o float32, gate and y of one dtype, [N, H * Dv]")
    _need(gain.is_contiguous() and gain.numel() == v_head_dim, "delta_gate_norm: the gain has one entry a value channel")
    if act not in ("silu", "sigmoid"):
        raise KernelError(f"delta_gate_norm: unknown gate {act!r}")
    with _timed("delta_gate_norm", N * cols * (4 + 2 * y.element_size()), 8 * N * cols, "fp32"):
        _check(_lib().da_delta_gate_norm(_ptr(o), o.stride(0), _ptr(gate), _dt(gate), gate.stride(0), _ptr(gain), _dt(gain),
                                         float(eps), ACTIVATIONS["silu"] if act == "silu" else 0, _ptr(y), y.stride(0), N,
                                         n_heads, v_head_dim, _stream()))
    return y
