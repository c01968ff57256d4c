"""Causal self-attention over the paged cache, as a mixer.

Fused projection to q | k | v (+ bias), optional position encoding of q and k, write of the
new k and v rows into the cache slot, attention of every row over its sequence's pages, and
the output projection (+ bias) added into the residual stream.

Optional extras, each a record of the spec with its constants: values of a per-head size of their own
(``v_head_dim``), a learned bias by the distance between query and key (``distance_bias``, a table of
buckets that the mixer writes out once as a table by distance), a query temperature that grows with
the position (``query_temperature``), a root-mean-square norm of queries and keys before the rotation
(``qk_norm``: over a token's whole projection or head by head), a cap on the scores (``score_softcap``:
cap * tanh(score / cap)), and first keys of a sequence that a window never leaves behind (``keep_first``:
position i sees j <= i when i - j < window or j < keep_first), values that are the keys before their rotation
(``values_are_keys``: the projection has no value rows; the kernel that turns the keys also keeps them unturned as
values), a term without key or value in the softmax's denominator (``sink``: exp(0), or exp of a learned number per
head), and a logistic gate of one more projection of the input on the heads' results (``out_gate``: its rows are stacked
behind q | k | v in the same product).
Reference: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:226-420
(projections :266-291, cache write :315-336, scores/softmax/weighted sum :458-532, output
projection :385-408); the residual add is TransformerBlock.java:176.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import (KVNeed, Mixer, StepContext, build_position, register_mixer, to_matrix, to_vector)


def distance_bucket(n: int, n_buckets: int, max_distance: int) -> int:
    """The row of a bias table of ``n_buckets`` rows that the distance ``n`` >= 0 uses: one row a distance below
    half the rows, then rows shared in steps that grow like a logarithm up to ``max_distance``."""
    half = n_buckets // 2
    if n < half:
        return n
    return min(n_buckets - 1, half + int(math.floor(math.log(n / half) / math.log(max_distance / half) * (n_buckets - half))))


def bias_by_distance(table: torch.Tensor, max_distance: int) -> torch.Tensor:
    """A bucket table [n_buckets, heads] written out by distance: float32 [heads, max_distance + 1] on the CPU;
    every distance from ``max_distance`` on uses the last column (it lies in the last bucket)."""
    n_buckets = table.shape[0]
    if n_buckets < 2 or max_distance <= n_buckets // 2:
        raise ValueError(f"a bias table of {n_buckets} rows with a largest distance of {max_distance}")
    rows = torch.tensor([distance_bucket(n, n_buckets, max_distance) for n in range(max_distance + 1)], dtype=torch.long)
    return table.detach().to("cpu", torch.float32)[rows].t().contiguous()


class CausalSelfAttention(Mixer):
    graph_safe = True
    can_store = True          # with ``ctx.part_accumulate`` off the output projection stores instead of adding

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        self.n_heads, self.n_kv_heads, self.head_dim = spec.n_heads, spec.n_kv_heads, spec.head_dim
        if self.n_heads % self.n_kv_heads != 0:
            raise ValueError(f"{self.n_heads} query heads are not a multiple of {self.n_kv_heads} key heads")
        # Any head size up to 256 runs: multiples of 16 on the matrix-core attention kernels in bfloat16,
        # the others (and everything in 32-bit) on the plain attention kernel.
        if not (1 <= self.head_dim <= ops.MAX_HEAD_DIM):
            raise ValueError(f"head size {self.head_dim} is outside 1..{ops.MAX_HEAD_DIM}")
        self.v_head_dim = int(getattr(spec, "v_head_dim", None) or self.head_dim)
        if not (1 <= self.v_head_dim <= ops.MAX_HEAD_DIM):
            raise ValueError(f"value head size {self.v_head_dim} is outside 1..{ops.MAX_HEAD_DIM}")
        self.q_cols = self.n_heads * self.head_dim
        self.kv_cols = self.n_kv_heads * self.head_dim
        self.v_cols = self.n_kv_heads * self.v_head_dim
        self.o_cols = self.n_heads * self.v_head_dim
        self.values_are_keys = bool(getattr(spec, "values_are_keys", False))
        self.qkv_cols = self.q_cols + self.kv_cols + (0 if self.values_are_keys else self.v_cols)
        self.out_gate = getattr(spec, "out_gate", None)
        if self.out_gate not in (None, "sigmoid"):
            raise ValueError(f"an output gate is 'sigmoid' or None, not {self.out_gate!r}")
        if self.values_are_keys and self.v_head_dim != self.head_dim:
            raise ValueError(f"values that are the keys have the keys' size {self.head_dim}, not {self.v_head_dim}")
        self.gate_cols = self.o_cols if self.out_gate else 0
        self.proj_cols = self.qkv_cols + self.gate_cols            # the projection's rows: q | k | v | gate
        # Where the attention kernel finds the gate in the rows that hold its queries: behind q | k | v where the
        # product's rows are those rows, right behind the queries where a kernel of its own makes them ready.
        self.gate_off = self.qkv_cols
        self.scale = float(spec.scale)
        self.window = spec.window
        self.qkv_weight = to_matrix(params["qkv_weight"], dtype, device)
        self.out_weight = to_matrix(params["out_weight"], dtype, device)
        self.qkv_bias = to_vector(params.get("qkv_bias"), dtype, device) if spec.qkv_bias else None
        self.out_bias = to_vector(params.get("out_bias"), dtype, device) if spec.out_bias else None
        if tuple(self.qkv_weight.shape) != (self.proj_cols, spec.width):
            raise ValueError(f"qkv weight is {list(self.qkv_weight.shape)}, expected {[self.proj_cols, spec.width]}")
        sink = getattr(spec, "sink", None)
        if sink not in (None, "zero", "learned"):
            raise ValueError(f"a sink is 'zero', 'learned' or None, not {sink!r}")
        self.sink = None                              # 32-bit, one a query head
        if sink == "zero":
            self.sink = torch.zeros(self.n_heads, dtype=torch.float32, device=device)
        elif sink == "learned":
            self.sink = params["sink"].to(device=device, dtype=torch.float32).contiguous()
            if self.sink.numel() != self.n_heads:
                raise ValueError(f"the sink has {self.sink.numel()} entries for {self.n_heads} heads")
        if tuple(self.out_weight.shape) != (spec.width, self.o_cols):
            raise ValueError(f"output weight is {list(self.out_weight.shape)}, expected {[spec.width, self.o_cols]}")
        # the extras: a table by distance [heads, max_distance + 1] (32-bit) and the temperature's constants
        self.dist_bias = None
        db = getattr(spec, "distance_bias", None)
        if db is not None:
            table = params["distance_bias"]
            if table.dim() != 2 or table.shape[1] != self.n_heads or (db.n_buckets and table.shape[0] != db.n_buckets):
                raise ValueError(f"distance-bias table is {list(table.shape)}, expected "
                                 f"{[db.n_buckets or 'rows', self.n_heads]}")
            self.dist_bias = bias_by_distance(table, db.max_distance).to(device)
        qt = getattr(spec, "query_temperature", None)
        self.temp_coef, self.temp_every = (float(qt.coef), int(qt.every)) if qt is not None else (0.0, 0)
        if qt is not None and self.temp_every <= 0:
            raise ValueError(f"query temperature period {self.temp_every} must be positive")
        # a cap on the scores, first keys that a window keeps, and the norm of queries and keys
        self.softcap = float(getattr(spec, "score_softcap", 0.0) or 0.0)
        self.keep_first = int(getattr(spec, "keep_first", 0) or 0) if self.window else 0
        if self.softcap < 0.0 or self.keep_first < 0:
            raise ValueError(f"score cap {self.softcap} and kept first keys {self.keep_first} must not be negative")
        qn = getattr(spec, "qk_norm", None)
        self.qk_norm = qn
        if qn is not None:
            nq, nk = (self.q_cols, self.kv_cols) if qn.whole else (self.head_dim, self.head_dim)
            self.q_gain = to_vector(params["q_norm"], dtype, device)
            self.k_gain = to_vector(params["k_norm"], dtype, device)
            if self.q_gain.numel() != nq or self.k_gain.numel() != nk:
                raise ValueError(f"query and key gains have {self.q_gain.numel()} and {self.k_gain.numel()} entries, "
                                 f"expected {nq} and {nk}")
        self.extras = (self.dist_bias is not None or self.temp_every > 0 or self.v_head_dim != self.head_dim
                       or self.softcap > 0.0 or self.keep_first > 0 or self.sink is not None or self.out_gate is not None)
        self.position = None
        if spec.position is not None and spec.position.kind != "none":
            self.position = build_position(spec.position, params.get("position", {}), dtype, device)

    def cache_need(self):
        return KVNeed(self.n_kv_heads, self.head_dim, self.window,
                      None if self.v_head_dim == self.head_dim else self.v_head_dim, keep_first=self.keep_first)

    def _epilogue_write(self) -> bool:
        """Whether the q|k|v product may write keys and values to the cache itself (its epilogue assumes
        keys and values of one size)."""
        return (self.position is None and self.v_head_dim == self.head_dim and self.qk_norm is None
                and self.out_gate is None and not self.values_are_keys)

    normed_into = True

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor, call, into=None) -> bool:
        """Small steps: the norm in front (LayerNorm or a root-mean-square norm), the q|k|v projection and the
        cache write in one kernel.  The result joins ``into`` (the stream ``x`` itself when None)."""
        N = x.shape[0]
        ln = norm.fusable_params()
        rms = getattr(norm, "rms_params", lambda: None)() if ln is None else None
        if (ln is None and rms is None) or not ops.can_fuse_ln(N, x, self.qkv_weight):
            return False
        slot = ctx.cache.kv[call.cache]
        group = ctx.group_of(call.cache)
        if self._prepared():
            # the norm and the one product in one kernel, its 32-bit sums made ready by the next
            raw = ctx.buf("qkv_raw", N, self.proj_cols, torch.float32)
            if ln is not None:
                ops.linear_ln(x, None, N, ln[0], ln[1], ln[2], self.qkv_weight, self.qkv_bias, raw)
            else:
                ops.linear_rms(x, None, N, rms[0], rms[1], rms[2], self.qkv_weight, self.qkv_bias, raw)
            self._attend(ctx, self._prepare(ctx, raw, slot, group, call), x if into is None else into, slot, group, call,
                         gate_off=self.q_cols)
            return True
        if not self._epilogue_write():
            # the norm and the one product in one kernel; the turn of q and k and the cache write follow
            qkv = ctx.buf("qkv", N, self.proj_cols, ctx.dtype)
            if ln is not None:
                ops.linear_ln(x, None, N, ln[0], ln[1], ln[2], self.qkv_weight, self.qkv_bias, qkv)
            else:
                ops.linear_rms(x, None, N, rms[0], rms[1], rms[2], self.qkv_weight, self.qkv_bias, qkv)
            self._turn_and_keep(ctx, qkv, slot, group, call)
            self._attend(ctx, qkv, x if into is None else into, slot, group, call)
            return True
        qkv = ctx.buf("qkv", N, self.qkv_cols, ctx.dtype)
        kv = dict(kv_cache=slot if call.write else None, slot_map=ctx.slot_maps[group] if call.write else None,
                  q_cols=self.q_cols)
        if ln is not None:
            gain, bias, eps = ln
            ops.linear_ln(x, None, N, gain, bias, eps, self.qkv_weight, self.qkv_bias, qkv, **kv)
        else:
            gain, offset, eps = rms
            ops.linear_rms(x, None, N, gain, offset, eps, self.qkv_weight, self.qkv_bias, qkv, **kv)
        self._attend(ctx, qkv, x if into is None else into, slot, group, call)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        N = h.shape[0]
        qkv = ctx.buf("qkv", N, self.proj_cols, ctx.dtype)
        slot = ctx.cache.kv[call.cache]
        group = ctx.group_of(call.cache)
        if self._epilogue_write() and call.write:
            # the new keys and values go to the cache in the projection's epilogue
            ops.linear(h, self.qkv_weight, self.qkv_bias, qkv, kv_cache=slot, slot_map=ctx.slot_maps[group],
                       q_cols=self.q_cols)
        elif self._prepared():
            # one kernel works on the product's unrounded 32-bit sums: it normalises queries and keys (if the design
            # has that), turns them by the position, stores the queries (and the gate behind them) and writes keys and
            # values to the cache
            raw = ctx.buf("qkv_raw", N, self.proj_cols, torch.float32)
            ops.linear(h, self.qkv_weight, self.qkv_bias, raw)
            self._attend(ctx, self._prepare(ctx, raw, slot, group, call), x, slot, group, call, gate_off=self.q_cols)
            return
        else:
            ops.linear(h, self.qkv_weight, self.qkv_bias, qkv)
            self._turn_and_keep(ctx, qkv, slot, group, call)
        self._attend(ctx, qkv, x, slot, group, call)

    def _prepared(self) -> bool:
        """Whether queries, keys and values go through ``ops.attn_prepare`` (a norm of queries and keys, or values
        that are the keys; a rotation or no position encoding)."""
        if self.qk_norm is None and not self.values_are_keys:
            return False
        if self.position is not None and not hasattr(self.position, "speeds"):
            raise ValueError("queries and keys with a norm, or keys that are values, take a rotation or no position encoding")
        return True

    def _prepare(self, ctx: StepContext, raw: torch.Tensor, slot: torch.Tensor, group: int, call) -> torch.Tensor:
        """[queries | gate] in the compute dtype from the product's 32-bit rows; keys and values into the cache."""
        rot = self.position
        norm = self.qk_norm
        q = ctx.buf("q_ready", raw.shape[0], self.q_cols + self.gate_cols, ctx.dtype)
        ops.attn_prepare(raw, self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim,
                         None if norm is None else self.q_gain, None if norm is None else self.k_gain,
                         0.0 if norm is None else norm.eps, True if norm is None else norm.whole, ctx.positions,
                         None if rot is None else rot.speeds, 0 if rot is None else rot.dims,
                         True if rot is None else rot.interleaved, q,
                         slot if call.write else None, ctx.slot_maps[group] if call.write else None,
                         ctx.cache.page_size, values_are_keys=self.values_are_keys, pass_cols=self.gate_cols,
                         magnitude=1.0 if rot is None else getattr(rot, "magnitude", 1.0))
        return q

    def _turn_and_keep(self, ctx: StepContext, qkv: torch.Tensor, slot: torch.Tensor, group: int, call) -> None:
        """The position encoding of q and k in place, then keys and values into the cache."""
        if self.position is not None:
            self.position.apply_qk(ctx, qkv, self.n_heads, self.n_kv_heads, self.head_dim)
        if call.write and self.v_head_dim == self.head_dim:
            ops.kv_write(qkv, self.q_cols, self.q_cols + self.kv_cols, slot, ctx.slot_maps[group],
                         self.n_kv_heads, self.head_dim)
        elif call.write:
            ops.kv_write_split(qkv, self.q_cols, self.q_cols + self.kv_cols, slot, ctx.slot_maps[group],
                               self.n_kv_heads, self.head_dim, self.v_head_dim, ctx.cache.page_size)

    def _attend(self, ctx: StepContext, qkv: torch.Tensor, x: torch.Tensor, slot: torch.Tensor, group: int,
                call, gate_off=None) -> None:
        """``qkv``: rows that start with the queries; with a gate it lies in the same rows from ``gate_off`` on."""
        N = qkv.shape[0]
        gate_off = self.gate_off if gate_off is None else gate_off
        o = ctx.buf("attn_out", N, self.o_cols, ctx.dtype)
        if self.extras:
            # with a gate, q is the whole rows: queries first, the gate from ``gate_off`` on
            ops.paged_attention_rel(ctx, qkv if self.out_gate else qkv[:, :self.q_cols], slot, group, self.n_heads, self.n_kv_heads, self.head_dim,
                                    self.v_head_dim, self.scale, self.window, self.dist_bias, self.temp_coef,
                                    self.temp_every, o, softcap=self.softcap, keep_first=self.keep_first, sink=self.sink,
                                    gate_col=gate_off if self.out_gate else -1)
        else:
            ops.paged_attention(ctx, qkv[:, :self.q_cols], slot, group, self.n_heads, self.scale, self.window, o)
        if ctx.debug_hook is not None:      # the reference's stage names (CausalSelfAttention.java:299-301,384)
            ctx.emit(call.layer, "query_projection", qkv[:, :self.q_cols])
            if qkv.shape[1] >= self.q_cols + self.kv_cols + self.v_cols and not self._prepared():
                ctx.emit(call.layer, "key_projection", qkv[:, self.q_cols:self.q_cols + self.kv_cols])
                ctx.emit(call.layer, "value_projection", qkv[:, self.q_cols + self.kv_cols:self.qkv_cols])
            ctx.emit(call.layer, "attention_value", o)
            # the output projection before its bias (CausalSelfAttention.java:406), worked out once more for the hook
            ctx.emit(call.layer, "attention_output",
                     ops.linear(o, self.out_weight, None, ctx.buf("attn_proj_debug", N, x.shape[1], torch.float32)))
        ops.linear(o, self.out_weight, self.out_bias, x, accumulate=ctx.part_accumulate)


register_mixer("attention", CausalSelfAttention)
