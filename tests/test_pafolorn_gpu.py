"""Pafolorn on the engine against the plain implementation (tests/plain_pafolorn.py): each mechanism alone through its
kernels and parts (the gated delta rule with either decay, its read-out norm and gate, the norm and turn of queries
and keys, attention with a capped score over a window that keeps first tokens, parallel mixers, layer scale), then
whole models through the step function (whole prompts, decoding token by token, portions down to two tokens, mixed
batches over a small pool whose pages and state slots come back and go out again), and greedy generation through the
engine's entry point and scheduler.  Sizes differ from test to test; where random numbers would hide a fault (a key at
a window's edge, a kept first token, something written to the state long ago) the inputs are made so that it shows."""
import json
from types import SimpleNamespace

from deliverance_amd.config.specs import LayerCall

import numpy as np
import pytest
import torch

import helpers
import plain_pafolorn as P
from helpers import quick
from pafolorn_models import CONFIG_F, CONFIG_G, CONFIG_H, attention, channel_layer, delta, make_model, parallel_layer

pytestmark = pytest.mark.gpu
DEV = helpers.DEVICE
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def bf16(a):
    """What bfloat16 keeps of an array (as float64)."""
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def dev(a, dtype=torch.int32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def host(t):
    return t.double().cpu().numpy()


class Pages:
    """Pages of a hand-made cache, handed out in a shuffled order and taken back."""

    def __init__(self, n_pages, seed=1):
        self.free = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
        self.tables = {}

    def grow(self, seq, total, page):
        t = self.tables.setdefault(seq, [])
        while len(t) * page < total:
            t.append(self.free.pop())
        return t

    def end(self, seq):
        self.free = self.tables.pop(seq) + self.free        # the next request gets these first


def step_ctx(dtype, seqs, lens_new, past, pages, page=16, slots=None):
    """A step context by hand: sequences ``seqs`` with ``past`` cached positions bring ``lens_new`` tokens each (one-token
    sequences first, as the step function orders them)."""
    from deliverance_amd.parts import Arena, StepContext
    S = len(seqs)
    total = [p + n for p, n in zip(past, lens_new)]
    tables = [pages.grow(s, t, page) for s, t in zip(seqs, total)]
    bt = torch.full((S, max(len(t) for t in tables)), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    ctx = StepContext()
    ctx.device, ctx.dtype = torch.device(DEV), DTYPES[dtype]
    ctx.n_seqs, ctx.n_tokens = S, sum(lens_new)
    ctx.n_decode = sum(1 for n in lens_new if n == 1)
    pos, seq_of, rows, q_start = [], [], [], [0]
    for s in range(S):
        for i in range(lens_new[s]):
            p_ = past[s] + i
            pos.append(p_); seq_of.append(s); rows.append(int(bt[s, p_ // page]) * page + p_ % page)
        q_start.append(len(pos))
    ctx.positions, ctx.seq_of_token, ctx.q_start, ctx.seq_lens = dev(pos), dev(seq_of), dev(q_start), dev(total)
    ctx.tokens = dev([0] * len(pos))
    ctx.q_start_host, ctx.seq_lens_host = q_start, total
    ctx.max_query_len, ctx.max_seq_len = max(lens_new), max(total)
    ctx.block_tables, ctx.slot_maps = [bt.to(DEV)], [dev(rows)]
    ctx.state_slots = dev(slots if slots is not None else list(range(S)))
    ctx.state_slots_host = list(slots) if slots is not None else list(range(S))
    ctx._arena = Arena(DEV)
    ctx.cache = SimpleNamespace(page_size=page, group_of_slot={0: 0, 1: 0}, kv={}, state={})
    return ctx


class PartRunner:
    """Sequences of inputs go through a mixer part in steps of any cut, over hand-made pages and state slots; every
    step's rows are compared with the plain result over the whole sequences."""

    def __init__(self, part, dtype, width, seqs, want, slot_of, tol, n_slots=5, page=16, n_caches=1):
        self.part, self.dtype, self.width, self.seqs, self.want, self.slot_of = part, dtype, width, seqs, want, slot_of
        self.page, self.tol = page, tol
        self.scale = max(np.abs(w).max() for w in want)
        self.done = [0] * len(seqs)
        needs = part.cache_need()
        needs = list(needs) if isinstance(needs, (tuple, list)) else [needs]
        self.pages = Pages(sum(-(-len(s) // page) for s in seqs) + 3)
        n_pages = len(self.pages.free)
        self.kv, self.state = {}, {}
        for c, need in enumerate(needs):
            if hasattr(need, "elems"):
                self.state[c] = torch.full((n_slots, need.elems), float("nan"), dtype=torch.float32, device=DEV)
            else:
                D, Dv, G = need.head_dim, need.v_head_dim or need.head_dim, need.n_kv_heads
                shape = (n_pages, 2, G, page, D) if D == Dv else (n_pages, G * page * (D + Dv))
                self.kv[c] = torch.full(shape, float("nan"), dtype=DTYPES[dtype], device=DEV)

    def step(self, takes):
        order = sorted(takes, key=lambda s: (takes[s] != 1, s))
        for s in order:
            if self.done[s] == 0:
                for st in self.state.values():
                    st[self.slot_of[s]].zero_()          # what the engine does when a request is opened
        ctx = step_ctx(self.dtype, order, [takes[s] for s in order], [self.done[s] for s in order], self.pages, self.page,
                       slots=[self.slot_of[s] for s in order])
        ctx.cache.kv, ctx.cache.state = self.kv, self.state
        h = np.concatenate([self.seqs[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        x = torch.zeros(len(h), self.width, dtype=torch.float32, device=DEV)
        self.part.forward(ctx, dev(h, DTYPES[self.dtype]), x, LayerCall(0, 0, True))
        ref = np.concatenate([self.want[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        err = np.abs(host(x) - ref).max(axis=1)
        assert err.max() <= self.tol * self.scale, f"step {takes}: row {int(np.argmax(err))} is off by {err.max():.3e} of {self.scale:.3e}"
        for s in order:
            self.done[s] += takes[s]

    def end(self, s):
        self.pages.end(s)


# ------------------------------------------------------------------------------------------ the gated delta rule
def delta_weights(rng, E, m, channel):
    H, G, D, Dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    W = {"q": rng.normal(size=(G * D, E)) * 0.3, "k": rng.normal(size=(G * D, E)) * 0.3, "v": rng.normal(size=(H * Dv, E)) * 0.3,
         "q.conv": rng.normal(size=(G * D, K)) * 0.5, "k.conv": rng.normal(size=(G * D, K)) * 0.5,
         "v.conv": rng.normal(size=(H * Dv, K)) * 0.5, "b": rng.normal(size=(H, E)) * 0.3, "A_log": rng.normal(size=H) * 0.5,
         "norm": 1 + rng.normal(size=Dv) * 0.2, "o": rng.normal(size=(E, H * Dv)) * 0.2}
    if channel:
        W.update({"a1": rng.normal(size=(m["a_rank"], E)) * 0.3, "a2": rng.normal(size=(H * D, m["a_rank"])) * 0.5,
                  "g1": rng.normal(size=(m["g_rank"], E)) * 0.3, "g2": rng.normal(size=(H * Dv, m["g_rank"])) * 0.5,
                  "dt_bias": rng.normal(size=H * D) * 0.5})
    else:
        W.update({"a": rng.normal(size=(H, E)) * 0.3, "g": rng.normal(size=(H * Dv, E)) * 0.3, "dt_bias": rng.normal(size=H) * 0.5})
    return {k: bf16(v) for k, v in W.items()}


def delta_part(W, E, m, channel, dtype, eps=1e-5):
    from deliverance_amd.config.specs import DeltaRuleSpec
    from deliverance_amd.parts import build_mixer
    t = lambda k: torch.tensor(W[k], dtype=torch.float32).to(torch.bfloat16)
    p = {"q_weight": t("q"), "k_weight": t("k"), "v_weight": t("v"), "q_conv": t("q.conv"), "k_conv": t("k.conv"),
         "v_conv": t("v.conv"), "beta_weight": t("b"), "a_log": t("A_log"), "out_norm": t("norm"), "dt_bias": t("dt_bias"),
         "out_weight": t("o")}
    if channel:
        p.update({"decay_down": t("a1"), "decay_up": t("a2"), "gate_down": t("g1"), "gate_up": t("g2")})
    else:
        p.update({"decay_weight": t("a"), "gate_weight": t("g")})
    spec = DeltaRuleSpec("delta_rule", E, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], eps,
                         decay="channel" if channel else "head", decay_rank=-1 if channel else 0,
                         gate="sigmoid" if channel else "silu", gate_rank=-1 if channel else 0)
    return build_mixer(spec, p, DTYPES[dtype], DEV)


DELTA_SIZES = [quick(delta(4, 2, 16, 32, 4), False), (delta(3, 1, 20, 12, 2, a_rank=5, g_rank=3), True),
               quick(delta(1, 1, 8, 48, 1, a_rank=1, g_rank=1), True), (delta(2, 2, 72, 24, 5), False),
               (delta(6, 2, 32, 16, 3, a_rank=8, g_rank=12), True), (delta(2, 1, 130, 17, 3), False)]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m,channel", DELTA_SIZES)
def test_delta_rule_part_any_cut_and_slots_used_again(m, channel, dtype):
    """Four sequences in portions of every size (shorter than the filter, one token, long ones), their states in slots
    that are not in order; a new sequence takes a slot that was used."""
    rng = np.random.default_rng(9)
    E = 40
    W = delta_weights(rng, E, m, channel)
    part = delta_part(W, E, m, channel, dtype)
    seqs = [bf16(rng.normal(size=(n, E))) for n in (61, 23, 9, 30)]
    want = [P.delta_mixer(W, "", m, s, 1e-5, channel) for s in seqs]
    r = PartRunner(part, dtype, E, seqs, want, {0: 3, 1: 0, 2: 4, 3: 0}, 3e-5 if dtype == "float32" else 4e-2)
    r.step({0: 2, 1: 1})              # shorter than the filter
    r.step({0: 1, 1: 2, 2: 9})
    r.step({0: 25, 1: 20})
    r.step({0: 1, 3: 22})             # a decoded token beside a portion; slot 0 again, from zero
    r.step({0: 32, 3: 8})
    assert r.done == [61, 23, 9, 30]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("channel", [False, True])
@pytest.mark.parametrize("cuts", [(400,), quick((1, 2, 250, 1, 1, 145)), tuple([3] + [1] * 397)])
def test_delta_rule_keeps_what_was_written_long_ago(dtype, channel, cuts):
    """One head whose decay stays close to 1 reads, at the last token, what the very first token wrote: the first
    token's key comes back as the last token's query, every key in between is at a right angle to it.  The other head
    decays fast and must have forgotten.  Through a whole prompt, portions, and four hundred decoded tokens."""
    from deliverance_amd.kernels import ops
    T, H, D, Dv = sum(cuts), 2, 24, 20
    rng = np.random.default_rng(4)
    first = np.zeros(D); first[0] = 1.0
    k = np.concatenate([np.zeros((T, 1)), rng.normal(size=(T, D - 1))], axis=1)
    k[0] = first * 3.0
    q = rng.normal(size=(T, D)); q[-1] = first * 2.0
    v = rng.normal(size=(T, H, Dv)); v[0] = 5.0
    q, k, v = bf16(q), bf16(k), bf16(v)
    beta_raw = np.full((T, H), 6.0)                               # beta close to 1
    cols = H * D if channel else H
    a_raw = np.zeros((T, cols)); dt_bias = np.zeros(cols)
    a_log = np.array([-12.0, 1.0])                                 # decays of 1 - 4e-6 and of 0.15 a token
    rate = np.exp(a_log)
    step = np.logaddexp(0.0, a_raw + dt_bias).reshape(T, H, -1)
    decay = np.exp(-rate[None, :, None] * step) * np.ones((1, 1, D))
    want = np.zeros((T, H, Dv))
    qn, kn = P.unit_length(q) * D ** -0.5, P.unit_length(k)
    for h in range(H):
        want[:, h], _ = P.delta_recurrence(qn, kn, v[:, h], 1 / (1 + np.exp(-beta_raw[:, h])), decay[:, h])
    assert np.abs(want[-1, 0]).min() > 0.5 and np.abs(want[-1, 1]).max() < 1e-6      # remembered, forgotten
    qkv = dev(np.concatenate([q, k, v.reshape(T, -1)], axis=1), DTYPES[dtype])
    state = torch.full((2, H * Dv * D), float("nan"), dtype=torch.float32, device=DEV)
    state[1].zero_()
    got, done = np.zeros((T, H * Dv)), 0
    pages = Pages(T // 16 + 4)
    for n in cuts:
        ctx = step_ctx(dtype, ["s"], [n], [done], pages, slots=[1])
        o = torch.empty(n, H * Dv, dtype=torch.float32, device=DEV)
        ops.delta_rule(ctx, qkv[done:done + n], D, 2 * D, dev(beta_raw[done:done + n], torch.float32),
                       dev(a_raw[done:done + n], torch.float32), dev(dt_bias, torch.float32), dev(rate, torch.float32),
                       state, o, H, 1, D, Dv, channel, 1e-6, write=True, decay_off=0)
        got[done:done + n] = host(o)
        done += n
    tol = 2e-5 if dtype == "float32" else 2e-3           # the kernel's own arithmetic is 32-bit in either mode
    assert np.abs(got - want.reshape(T, -1)).max() <= tol * np.abs(want).max()
    assert torch.isnan(state[0]).all()


def test_delta_rule_without_write_leaves_the_state():
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(5)
    H, G, D, Dv, N = 4, 2, 12, 10, 7
    qkv = dev(rng.normal(size=(N, 2 * G * D + H * Dv)), torch.float32)
    state = dev(rng.normal(size=(3, H * Dv * D + 5)), torch.float32)
    before = state.clone()
    ctx = step_ctx("float32", ["s"], [N], [0], Pages(4), slots=[2])
    o = torch.empty(N, H * Dv, dtype=torch.float32, device=DEV)
    raw = dev(rng.normal(size=(N, 2 * H)), torch.float32)
    ops.delta_rule(ctx, qkv, G * D, 2 * G * D, raw, raw, dev(np.zeros(H), torch.float32), dev(np.ones(H), torch.float32),
                   state, o, H, G, D, Dv, False, 1e-6, write=False, decay_off=H)
    assert torch.equal(state, before) and bool(torch.isfinite(o).all())
    # a sequence without a slot starts from zeros and keeps nothing
    ctx.state_slots = dev([-1])
    o2 = torch.empty_like(o)
    ops.delta_rule(ctx, qkv, G * D, 2 * G * D, raw, raw, dev(np.zeros(H), torch.float32), dev(np.ones(H), torch.float32),
                   state, o2, H, G, D, Dv, False, 1e-6, write=True, decay_off=H)
    assert torch.equal(state, before)
    state[2].zero_()
    ctx.state_slots = dev([2])
    ops.delta_rule(ctx, qkv, G * D, 2 * G * D, raw, raw, dev(np.zeros(H), torch.float32), dev(np.ones(H), torch.float32),
                   state, o, H, G, D, Dv, False, 1e-6, write=True, decay_off=H)
    assert torch.equal(o, o2) and float(state[2, H * Dv * D:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,Dv,act", [(3, 20, "silu"), (1, 64, "sigmoid"), (5, 130, "silu"), (2, 1, "sigmoid")])
def test_read_out_norm_and_gate(dtype, H, Dv, act):
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(H * Dv)
    N = 6
    o = rng.normal(size=(N, H, Dv)).astype(np.float32).astype(np.float64)
    o[1] *= 1e-3                                                   # small rows: eps matters
    gate, gain = bf16(rng.normal(size=(N, H, Dv)) * 2), bf16(1 + rng.normal(size=Dv) * 0.3)
    y = torch.empty(N, H * Dv, dtype=DTYPES[dtype], device=DEV)
    ops.delta_gate_norm(dev(o.reshape(N, -1), torch.float32), dev(gate.reshape(N, -1), DTYPES[dtype]),
                        dev(gain, DTYPES[dtype]), 1e-5, act, H, Dv, y)
    want = P.unit_rms(o, 1e-5) * gain * (P.swish(gate) if act == "silu" else P.logistic(gate))
    assert np.abs(host(y).reshape(N, H, Dv) - want).max() <= (3e-6 if dtype == "float32" else 2.0 ** -7) * np.abs(want).max()


# ------------------------------------------------------------------------------------------ queries and keys
@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("H,G,D,Dv,dims", [quick(4, 2, 32, 16, 16), (3, 1, 12, 20, 12), (2, 2, 24, 8, 6), (1, 1, 16, 16, 0), (6, 3, 48, 96, 48)])
def test_norm_and_turn_of_queries_and_keys(dtype, H, G, D, Dv, dims):
    """The norm over a token's whole query and key projections, the turn of the first entries of every head by the
    position (entry i with entry i + dims / 2), and the rows that reach the cache."""
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(D + dims)
    N, page, base, eps = 11, 4, 500.0, 1e-5
    raw = rng.normal(size=(N, H * D + G * D + G * Dv)).astype(np.float32).astype(np.float64)
    raw[2] *= 1e-3
    qg, kg = bf16(1 + rng.normal(size=H * D) * 0.2), bf16(1 + rng.normal(size=G * D) * 0.2)
    places = [0, 1, 2, 3, 700, 701, 5, 6, 40000, 8, 9]
    q = P.turn_halves((P.unit_rms(raw[:, :H * D], eps) * qg).reshape(N, H, D), places, dims, base)
    k = P.turn_halves((P.unit_rms(raw[:, H * D:H * D + G * D], eps) * kg).reshape(N, G, D), places, dims, base)
    v = raw[:, H * D + G * D:].reshape(N, G, Dv)
    q_out = torch.empty(N, H * D, dtype=DTYPES[dtype], device=DEV)
    cache = torch.zeros(4, G * page * (D + Dv), dtype=DTYPES[dtype], device=DEV)
    rows = [13, 2, 7, 0, 5, 4, 15, 10, 9, 8, 1]
    speeds = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64, device=DEV) if dims else None
    ops.attn_prepare(dev(raw, torch.float32), H, G, D, Dv, dev(qg, DTYPES[dtype]), dev(kg, DTYPES[dtype]), eps, True,
                     dev(places), speeds, dims, False, q_out, cache, dev(rows), page)
    tol = 4e-6 if dtype == "float32" else 2.0 ** -7
    assert np.abs(host(q_out).reshape(N, H, D) - q).max() <= tol * np.abs(q).max()
    c = host(cache)
    for n, r in enumerate(rows):
        pg, i = divmod(r, page)
        for g in range(G):
            keys = c[pg, (g * page + i) * D:(g * page + i + 1) * D]
            vals = c[pg, G * page * D + g * Dv * page:G * page * D + (g + 1) * Dv * page].reshape(Dv, page)[:, i]
            assert np.abs(keys - k[n, g]).max() <= tol * np.abs(k).max()
            assert np.abs(vals - v[n, g]).max() <= tol * np.abs(v).max()


# ------------------------------------------------------------------------------------------ attention
def attention_weights(rng, E, m):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    W = {"q": rng.normal(size=(H * D, E)) * 0.3, "k": rng.normal(size=(G * D, E)) * 0.3, "v": rng.normal(size=(G * Dv, E)) * 0.3,
         "q.norm": 1 + rng.normal(size=H * D) * 0.2, "k.norm": 1 + rng.normal(size=G * D) * 0.2,
         "o": rng.normal(size=(E, H * Dv)) * 0.2}
    return {k: bf16(v) for k, v in W.items()}


def attention_part(W, E, m, dtype, eps=1e-5):
    from deliverance_amd.config.specs import AttentionSpec, QKNormSpec, RotarySpec
    from deliverance_amd.parts import build_mixer
    t = lambda a: torch.tensor(a, dtype=torch.float32).to(torch.bfloat16)
    spec = AttentionSpec("attention", E, m["heads"], m["kv_heads"], m["dim"], m["scale"], qkv_bias=False, out_bias=False,
                         window=m["mask"]["size"], position=RotarySpec("rotary", m["rot"]["dims"], m["rot"]["base"], interleaved=False)
                         if m["rot"]["dims"] else None, v_head_dim=m["vdim"], qk_norm=QKNormSpec(eps, True),
                         score_softcap=m.get("softcap") or 0.0, keep_first=m["mask"]["keep_first"])
    return build_mixer(spec, {"qkv_weight": t(np.concatenate([W["q"], W["k"], W["v"]])), "out_weight": t(W["o"]),
                              "q_norm": t(W["q.norm"]), "k_norm": t(W["k.norm"])}, DTYPES[dtype], DEV)


ATTENTION_SIZES = [quick(attention(4, 2, 32, 16, 0.18, 24, 5, 10000.0, 16, softcap=30.0)), attention(3, 1, 12, 20, 0.3, 17, 0, 500.0, 12),
                   attention(2, 2, 24, 8, 0.2, 33, 40, 250000.0, 6, softcap=5.0), attention(1, 1, 16, 16, 0.25, 1, 3, 100.0, 0),
                   quick(attention(6, 3, 16, 16, 0.4, 9, 2, 10000.0, 16, softcap=50.0)), attention(2, 1, 64, 64, 0.1, 70, 1, 1e6, 32)]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", ATTENTION_SIZES)
def test_attention_part_prompt_portions_and_decoding(m, dtype):
    """Three sequences through the part in portions and single tokens that pass the window and the kept first tokens;
    a fourth takes the pages that the second gave back."""
    rng = np.random.default_rng(m["dim"] + m["mask"]["size"])
    E = 40
    W = attention_weights(rng, E, m)
    part = attention_part(W, E, m, dtype)
    seqs = [bf16(rng.normal(size=(n, E))) for n in (90, 21, 50, 37)]
    want = [P.window_attention(W, "", m, s, 1e-5) for s in seqs]
    r = PartRunner(part, dtype, E, seqs, want, {0: 0, 1: 1, 2: 2, 3: 1}, 3e-5 if dtype == "float32" else 3e-2)
    r.step({0: 2, 1: 1, 2: 47})
    r.step({0: 1, 1: 20, 2: 1})
    r.end(1)
    r.step({0: 60, 2: 1, 3: 3})
    r.step({2: 1, 0: 1, 3: 34})
    for _ in range(26):
        r.step({0: 1})
    assert r.done == [90, 21, 50, 37]


def edge_case(window, keep, T, where, E, m, rng):
    """Inputs of one sequence in which the last query is the key at ``where`` (the weights make a head's query the
    negative of its group's key, and the last input is the negative of the marked one): that pair's score stands out
    if the key is seen."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    W = attention_weights(rng, E, m)
    W["q"] = -np.concatenate([W["k"][(i // (H // G)) * D:(i // (H // G) + 1) * D] for i in range(H)])
    W["q.norm"], W["k.norm"] = np.ones(H * D), np.ones(G * D)
    h = rng.normal(size=(T, E)) * 0.5
    mark = rng.normal(size=E)
    h[where] = mark * 3
    h[T - 1] = -mark * 3                 # its query is the marked key; its own key points the other way
    W["v"] = bf16(W["v"] * 0.1)
    return W, bf16(h)


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("tail", [quick(0), 1, 37])
@pytest.mark.parametrize("case", ["window_in", "window_out", "first_in", "first_out", "page_in", "far_out", "self"])
def test_attention_sees_one_key_at_every_edge(dtype, tail, case):
    """The last query looks for one key: just inside and just outside the window, the last kept first token and the
    one behind it, a key at a page's border inside the window, one far back; as the last row of a prompt's portion
    (tail 0) or decoded alone after 1 or 37 single tokens (the window passes over decoded tokens)."""
    window, keep, T = 35, 6, 131
    where = {"window_in": T - window, "window_out": T - window - 1, "first_in": keep - 1, "first_out": keep,
             "page_in": 112, "far_out": 48, "self": T - 1}[case]
    seen = case in ("window_in", "first_in", "page_in", "self")
    m = attention(4, 2, 32, 48, 0.9, window, keep, 10000.0, 4, softcap=40.0)
    rng = np.random.default_rng(where)
    E = 48
    W, h = edge_case(window, keep, T, where, E, m, rng)
    want, weights = P.window_attention(W, "", m, h, 1e-5, with_weights=True)
    if case != "self":
        assert (weights[:, T - 1, where].min() > 0.7) if seen else (weights[:, T - 1, where].max() == 0.0)
    part = attention_part(W, E, m, dtype)
    r = PartRunner(part, dtype, E, [h], [want], {0: 0}, 3e-5 if dtype == "float32" else 3e-2)
    if tail == 0:
        r.step({0: 100}); r.step({0: T - 100})
    else:
        r.step({0: 7}); r.step({0: T - tail - 7})
        for _ in range(tail):
            r.step({0: 1})
    assert r.done == [T]


WINDOW_KERNEL_SIZES = [quick(4, 2, 64, 64, 100, 4, 30.0), (2, 1, 128, 128, 300, 70, 0.0), (3, 3, 48, 24, 0, 0, 20.0),
                       (2, 2, 8, 100, 33, 1, 0.0), (8, 2, 32, 64, 64, 64, 10.0), (2, 1, 40, 72, 7, 0, 3.0)]


@pytest.mark.parametrize("page", [16, quick(64)])
@pytest.mark.parametrize("H,G,D,Dv,window,keep,cap", WINDOW_KERNEL_SIZES)
def test_window_attention_kernel_against_sums_written_out(H, G, D, Dv, window, keep, cap, page):
    """The matrix-core kernel alone: single rows behind long pasts and portions of 2 to 300 rows (one, two and four row
    blocks a workgroup, the last one part-filled) behind pasts of 0 to 500 keys; pages handed out in a shuffled order;
    pages that neither a window nor the kept first keys reach are gone from the table and hold NaN."""
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(H * 1000 + D + window)
    scale = 0.7 / np.sqrt(D)
    decode = [(1, 0), (1, 37), (1, 500), (1, window + keep if window else 64)]
    portions = [(2, 0), (33, 5), (64, 130), (65, 0), (300, 200), (31, 470)]
    if helpers.SIMT:                                   # (the simulated kernels: the same forms, fewer keys)
        decode = [(1, 0), (1, 37), (1, window + keep + 9 if window else 64)]
        portions = [(2, 0), (33, 5), (40, 130), (65, 0), (31, 170)]
    n_pages = sum(-(-(T + past) // page) for T, past in decode + portions) + 1
    order = list(rng.permutation(n_pages - 1) + 1)                      # page 0 belongs to nobody and holds NaN
    elems = G * page * (D + Dv)
    cache = np.full((n_pages, elems), np.nan)
    max_blocks = max(-(-(T + past) // page) for T, past in decode + portions) + 2
    tables, qs, wants = [], [], []
    for T, past in decode + portions:
        L = T + past
        K, V = bf16(rng.normal(size=(L, G, D))), bf16(rng.normal(size=(L, G, Dv)))
        q = bf16(rng.normal(size=(T, H, D)) * 1.5)
        lo_all = max(0, past - window + 1) if window else 0             # the first key that any row's window reaches
        row = np.full(max_blocks, -1, dtype=np.int64)
        for b in range(-(-L // page)):
            first, last = b * page, min(L, (b + 1) * page) - 1
            if last < lo_all and first >= keep:
                continue                                                # nobody sees this page: it is gone
            pg = order.pop()
            row[b] = pg
            for j in range(first, last + 1):
                r = j - first
                for g in range(G):
                    cache[pg, (g * page + r) * D:(g * page + r + 1) * D] = K[j, g]
                    cache[pg, G * page * D + g * Dv * page:G * page * D + (g + 1) * Dv * page].reshape(Dv, page)[:, r] = V[j, g]
        # what was left of a page behind a sequence's end is anything: keep the NaN there
        tables.append(row)
        qs.append(q.reshape(T, H * D))
        o = np.zeros((T, H, Dv))
        for i in range(T):
            p_ = past + i
            js = np.array([j for j in range(p_ + 1) if not window or p_ - j < window or j < keep])
            for h in range(H):
                g = h // (H // G)
                sc = (K[js, g] @ q[i, h]) * scale
                if cap:
                    sc = cap * np.tanh(sc / cap)
                w = np.exp(sc - sc.max())
                o[i, h] = (w / w.sum()) @ V[js, g]
        wants.append(o.reshape(T, H * Dv))
    q_all = dev(np.concatenate(qs), torch.bfloat16)
    lens = [T + past for T, past in decode + portions]
    starts = np.concatenate([[0], np.cumsum([T for T, _ in decode + portions])])
    out = torch.full((q_all.shape[0], H * Dv), float("nan"), dtype=torch.bfloat16, device=DEV)
    cache_t, bt = dev(cache, torch.bfloat16), dev(np.stack(tables))
    nd = len(decode)
    ops.attention_window(q_all, cache_t, bt, dev(starts), dev(lens), 0, nd, 1, H, G, D, Dv, page, scale, window, keep, cap, out)
    want = np.concatenate(wants)
    for form in (0, 4, 2, 1):                              # the rule's choice, then every number of row blocks
        out[starts[nd]:] = float("nan")
        ops.attention_window(q_all, cache_t, bt, dev(starts), dev(lens), nd, len(portions), max(T for T, _ in portions), H, G, D,
                             Dv, page, scale, window, keep, cap, out, form=form)
        got = host(out)
        assert np.isfinite(got).all(), form
        assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max(), form


# ------------------------------------------------------------------------------------------ parallel mixers, layer scale
@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_parallel_mixers_add_with_their_constants(dtype):
    from deliverance_amd.config.specs import ParallelMixerSpec
    from deliverance_amd.parts import build_mixer
    rng = np.random.default_rng(12)
    E = 40
    ma, md = attention(4, 2, 16, 32, 0.2, 20, 3, 1000.0, 8, softcap=20.0), delta(4, 2, 16, 24, 3)
    Wa, Wd = attention_weights(rng, E, ma), delta_weights(rng, E, md, False)
    a, d = attention_part(Wa, E, ma, dtype), delta_part(Wd, E, md, False, dtype)
    t = lambda x: torch.tensor(x, dtype=torch.float32).to(torch.bfloat16)
    pa = {"qkv_weight": t(np.concatenate([Wa["q"], Wa["k"], Wa["v"]])), "out_weight": t(Wa["o"]), "q_norm": t(Wa["q.norm"]), "k_norm": t(Wa["k.norm"])}
    pd = {"q_weight": t(Wd["q"]), "k_weight": t(Wd["k"]), "v_weight": t(Wd["v"]), "q_conv": t(Wd["q.conv"]), "k_conv": t(Wd["k.conv"]),
          "v_conv": t(Wd["v.conv"]), "beta_weight": t(Wd["b"]), "a_log": t(Wd["A_log"]), "out_norm": t(Wd["norm"]),
          "dt_bias": t(Wd["dt_bias"]), "out_weight": t(Wd["o"]), "decay_weight": t(Wd["a"]), "gate_weight": t(Wd["g"])}
    part = build_mixer(ParallelMixerSpec("parallel", (a.spec, d.spec), (1.3, -0.6)), {"branches": [pa, pd]}, DTYPES[dtype], DEV)
    seqs = [bf16(rng.normal(size=(n, E))) for n in (45, 12)]
    want = [1.3 * P.window_attention(Wa, "", ma, s, 1e-5) - 0.6 * P.delta_mixer(Wd, "", md, s, 1e-5, False) for s in seqs]
    r = PartRunner(part, dtype, E, seqs, want, {0: 2, 1: 0}, 3e-5 if dtype == "float32" else 3e-2)
    r.step({0: 30, 1: 1}); r.step({0: 1, 1: 11}); r.step({0: 14})
    # asked to store (a norm follows): what the target held does not count
    ctx = step_ctx(dtype, ["z"], [4], [0], Pages(3), slots=[4])
    ctx.cache.kv, ctx.cache.state = r.kv, r.state
    r.state[1][4].zero_()
    ctx.part_accumulate = False
    x = torch.full((4, E), 1e6, dtype=torch.float32, device=DEV)
    part.forward(ctx, dev(seqs[0][:4], DTYPES[dtype]), x, LayerCall(0, 0, True))
    assert np.abs(host(x) - want[0][:4]).max() <= (3e-5 if dtype == "float32" else 3e-2) * r.scale


def test_layer_scale_joins_the_stream():
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(6)
    src, scale, x = rng.normal(size=(7, 50)), rng.normal(size=50), rng.normal(size=(7, 50))
    got = ops.scale_add_rows(dev(src, torch.float32), dev(scale, torch.float32), dev(x, torch.float32), 0.5)
    assert np.abs(host(got) - (x + 0.5 * scale * src)).max() <= 1e-6


# ------------------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def fmodels(tmp_path_factory):
    return {"F": make_model(tmp_path_factory.mktemp("pf"), CONFIG_F, 21), "G": make_model(tmp_path_factory.mktemp("pg"), CONFIG_G, 22),
            "H": make_model(tmp_path_factory.mktemp("ph"), CONFIG_H, 23)}


def check(model, got, requests, dtype, what=""):
    """32-bit: every logit within 3e-5 of the largest plain logit.  bfloat16: the rms error within 2^-5 of the logits'
    root mean square, the largest error of a position within a fifth of it, but for one position in fifty (or one)
    that may take three times as much (measured: rms 1 to 2 %, positions up to 12 %, a rare one 34 %.  Every part's
    result is normalised before it joins the stream, so a part's relative rounding error enters in full, and these
    models are narrow; a position whose mixer result or key happens to be small takes more, in 32-bit too)."""
    for rid, ids in requests:
        ref = model.plain_logits(ids)
        out = got[rid].astype(np.float64)
        assert out.shape == ref.shape, f"{what} {rid}: shape {out.shape} vs {ref.shape}"
        err = np.abs(out - ref)
        rms = float(np.sqrt((ref ** 2).mean()))
        by_position = err.max(axis=1)
        if dtype == "float32":
            bound = 3e-5 * np.abs(ref).max()
            assert by_position.max() <= bound, f"{what} {rid}: max error {err.max():.3e} > {bound:.3e}, first at position {int(np.argmax(by_position > bound))}"
            continue
        over = np.flatnonzero(by_position > 0.2 * rms)
        assert len(over) <= max(1, len(ids) // 50) and by_position.max() <= 0.6 * rms, \
            f"{what} {rid}: positions {over.tolist()[:8]} are off by up to {by_position.max() / rms:.3f} of the rms"
        assert float(np.sqrt((err ** 2).mean())) <= 2.0 ** -5 * rms, f"{what} {rid}: rms error"


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_stream_after_every_layer(fmodels, dtype):
    m = fmodels["F"]
    ids = m.prompt(40, salt=9)
    _, after = P.forward(m.plain_cfg, m.W, ids, with_layers=True)
    s = helpers.trace_session(m.folder, dtype, 64)
    got = []
    s.runner.debug_hook = lambda layer, stage, t: got.append(t.double().cpu().numpy()) if stage == "layer_output" else None
    helpers.replay(s, helpers.trace_whole("r", ids))
    s.runner.debug_hook = None
    assert len(got) == len(after)
    for i, (a, b) in enumerate(zip(got, after)):
        assert np.abs(a - b).max() <= (2e-5 if dtype == "float32" else 3e-2) * np.abs(b).max(), f"after layer {i}"


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("F"), "G", "H"])
def test_whole_prompts_and_first_tokens(fmodels, name, dtype):
    m = fmodels[name]
    reqs = [("one", m.prompt(1)), ("two", m.prompt(2)), ("three", m.prompt(3)), ("long", m.prompt(120))]
    s = helpers.trace_session(m.folder, dtype, 256)
    for rid, ids in reqs:
        check(m, helpers.replay(s, helpers.trace_whole(rid, ids)), [(rid, ids)], dtype, "whole")
    s.cache.manager.check()


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["F", quick("G"), "H"])
def test_prefill_against_token_by_token_decoding(fmodels, name, dtype):
    """All but the last 60 tokens at once, the rest one by one: they cross page borders and the windows pass over
    decoded tokens; then a request decoded from its first token on."""
    m = fmodels[name]
    ids = m.prompt(95, salt=1)
    s = helpers.trace_session(m.folder, dtype, 128)
    check(m, helpers.replay(s, helpers.trace_bulk_then_single("r", ids, tail=60)), [("r", ids)], dtype, "decode")
    ids2 = m.prompt(50, salt=2)
    check(m, helpers.replay(s, helpers.trace_bulk_then_single("q", ids2, tail=49)), [("q", ids2)], dtype, "decode from 1")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("F"), "G", "H"])
@pytest.mark.parametrize("sizes", [(7, 2, 13, 3, 5, 2), quick((2, 2, 31, 1, 16, 33, 2))])
def test_portions_of_any_size(fmodels, name, dtype, sizes):
    m = fmodels[name]
    ids = m.prompt(97, salt=3)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True)
    check(m, helpers.replay(s, helpers.trace_portions("r", ids, sizes)), [("r", ids)], dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["F", "G", quick("H")])
def test_mixed_batches_over_a_small_pool(fmodels, name, dtype):
    """Seven unequal requests, four live at a time, over a pool that holds just what is live and four state slots: pages
    and slots come back and go out again (freed pages are filled with NaN).  Then requests alone: what a request gets
    must not depend on its neighbours beyond rounding."""
    m = fmodels[name]
    reqs = [(f"r{i}", m.prompt(n, salt=10 + i)) for i, n in enumerate((40, 3, 71, 18, 64, 1, 33))]
    steps = helpers.trace_mixed(reqs, seed=5, max_live=4)
    s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True)
    got = helpers.replay(s, steps)
    check(m, got, reqs, dtype, "mixed")
    s.cache.manager.check()
    alone = helpers.trace_session(m.folder, dtype, 128)
    for rid, ids in reqs[:3]:
        one = helpers.replay(alone, helpers.trace_whole(rid, ids))[rid]
        scale = float(np.sqrt((one.astype(np.float64) ** 2).mean()))
        assert np.abs(one.astype(np.float64) - got[rid]).max() <= (2e-5 if dtype == "float32" else 0.1) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(fmodels, dtype):
    """Two hundred tokens one by one beside a neighbour that comes and goes."""
    m = fmodels["F"]
    ids, other = m.prompt(210, salt=20), m.prompt(60, salt=21)
    helpers.skip_in_simulation_if(True)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:10], "want": list(range(10))}], "end": []}]
    for i in range(10, len(ids)):
        entries = [{"id": "a", "tokens": [ids[i]], "want": [0]}]
        j = i - 50
        if 0 <= j < len(other):
            entries.append({"id": "b", "tokens": [other[j]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["b"] if j == len(other) - 1 else []})
    steps[-1]["end"].append("a")
    s = helpers.trace_session(m.folder, dtype, 320, poison_freed=True)
    check(m, helpers.replay(s, steps), [("a", ids), ("b", other)], dtype, "long decode")


def test_low_ranks_come_from_the_tensors(tmp_path):
    """A config.json that does not name the low ranks of the channel-wise decay and gate: the shapes say them."""
    m = make_model(tmp_path / "m", CONFIG_G, 31)
    cfg = json.load(open(f"{m.folder}/config.json"))
    for L in cfg["layers"]:
        L["mixer"].pop("a_rank", None); L["mixer"].pop("g_rank", None)
    json.dump(cfg, open(f"{m.folder}/config.json", "w"))
    ids = m.prompt(30)
    s = helpers.trace_session(m.folder, "float32", 64)
    check(m, helpers.replay(s, helpers.trace_whole("w", ids)), [("w", ids)], "float32", "ranks by shape")


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["F", "G"])
def test_greedy_generation_through_the_engine(fmodels, name, dtype):
    """The engine's own entry point and scheduler: several prompts at once over a pool that forces portions, with
    recorded decode steps and steps launched ahead, against the plain model's greedy choice."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = fmodels[name]
    prompts = [m.prompt(n, salt=30 + n) for n in (5, 33, 70, 2)]
    model = AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=512, max_num_seqs=3,
                                                 max_batch_tokens=48, max_chunk=32)
    outs = model.generate(prompts, GeneratorParameters(max_tokens=24, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.finish_reason == "length" and len(out.generated_tokens) == 24
        if dtype == "float32":
            assert out.generated_tokens == P.greedy_generate(m.plain_cfg, m.W, prompt, 24)
        else:
            ids = list(prompt)
            for t in out.generated_tokens:            # bfloat16 may flip a near-tie, nothing more
                row = m.plain_logits(ids)[-1]
                assert row[t] >= row.max() - 0.2 * float(np.sqrt((row ** 2).mean()))
                ids.append(t)


# ------------------------------------------------------------------------------------------ random configurations
def random_config(seed):
    """Sizes drawn at random: widths and head sizes that are no multiple of 8 or 16, one key head for several value
    heads, filters of one tap, windows shorter than the kept first tokens, layers in any order."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = pick(40, 50, 64, 100, 72, 36)

    def a_delta(channel):
        G = pick(1, 2, 3)
        d = delta(G * pick(1, 2, 3), G, pick(8, 16, 24, 33, 64, 96, 130), pick(8, 12, 32, 40, 72), pick(1, 2, 3, 4, 6))
        if channel:
            d["a_rank"], d["g_rank"] = pick(1, 4, 9), pick(2, 8, 16)
        return d

    layers = []
    for _ in range(int(rng.integers(1, 5))):
        ff = pick(None, 24, 40, 100)
        if pick(True, False):
            layers.append(channel_layer(a_delta(True), ff=ff))
        else:
            G = pick(1, 2, 3)
            D = pick(8, 16, 24, 32, 64, 48, 128)
            att = attention(G * pick(1, 2, 4), G, D, pick(D, D, 8, 40, 128), float(pick(0.1, D ** -0.5, 0.3)), pick(1, 7, 16, 30, 64),
                            pick(0, 0, 1, 4, 20), float(pick(100.0, 10000.0, 1e6)), pick(0, D // 2 // 2 * 2, D),
                            softcap=pick(None, 5.0, 30.0))
            layers.append(parallel_layer(att, a_delta(False), float(pick(1.0, 0.7, 1.4)), float(pick(1.0, 0.5, 1.1)), ff=ff))
    return {"architecture": "Pafolorn", "vocab": pick(50, 130, 257), "width": width, "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))},
            "logit_scale": float(pick(0.25, 1.0, 3.0)), "layers": layers}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(24))
def test_random_configurations(tmp_path, seed, dtype):
    m = make_model(tmp_path / "m", random_config(seed), 100 + seed)
    ids = m.prompt(75, salt=seed)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True)
    check(m, helpers.replay(s, helpers.trace_whole("w", ids)), [("w", ids)], dtype, f"seed {seed} whole")
    check(m, helpers.replay(s, helpers.trace_portions("p", ids, (5, 2, 17, 1, 1, 9, 33, 1, 1, 1))), [("p", ids)], dtype, f"seed {seed} portions")
