"""Salivik on the engine against the plain implementation (tests/plain_salivik.py): each mechanism alone through
its kernels and parts, then whole models through the step function (whole prompts, decoding token by token,
portions down to two tokens, mixed batches over a small pool whose pages and state slots come back and go out
again), and greedy generation through the engine's entry point and scheduler.  Sizes differ from test to test;
where random numbers would hide a fault (one far key among hundreds, a window's edge, the term without a key in a
softmax) the inputs are made so that it shows.  In bfloat16 two experts of nearly equal logits may be ranked the
other way round: the engine reports its choices through the layer debug hook and the plain model follows them
where they are as good as its own."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_salivik as P
from helpers import quick
from salivik_models import CONFIG_S, CONFIG_T, CONFIG_U, att, config, dense, lat, layer, make_model, moe, replay_routed, ret, rot

pytestmark = pytest.mark.gpu
DEV = helpers.DEVICE
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
SLACK = {"float32": 1e-4, "bfloat16": 0.06}      # how far below the plain model's last choice an engine's choice may lie


def bf16(a):
    """What bfloat16 keeps of an array (as float64)."""
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def dev(a, dtype=torch.int32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def host(t):
    return t.double().cpu().numpy()


def tb(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16)


# ------------------------------------------------------------------------------------------ rotation
@pytest.mark.parametrize("scaling", [None, (4.0, 64, 8.0, 1.0), quick((3.0, 512, 24.0, 2.0)), (1.0, 32, 4.0, 2.0), (8.0, 16, 1.0, 0.5)])
@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_rotation_of_halves_with_ramped_speeds(dtype, scaling):
    """Entry i is paired with entry i + dims / 2; with a scaling the slow pairs turn slower and all turned pairs grow.
    Heads at a stride inside wider rows, only the first entries turned, positions up to the thousands."""
    from deliverance_amd.config.specs import RampedSpeedsSpec, RotarySpec
    from deliverance_amd.parts import build_position
    rng = np.random.default_rng(4)
    N, H, width, dims, base = 7, 3, 20, 16, 300.0
    places = [0, 1, 2, 1000, 4097, 65000, 3]
    src = bf16(rng.normal(size=(N, 5 + H * 24)))
    spec = RotarySpec("rotary", dims, base, False, None if scaling is None else RampedSpeedsSpec(*scaling))
    turner = build_position(spec, {}, DTYPES[dtype], DEV)
    ctx = SimpleNamespace(positions=dev(places))
    s = dev(src, DTYPES[dtype])
    out = torch.zeros(N, H * width + 3, dtype=DTYPES[dtype], device=DEV)
    turner.apply(ctx, s[:, 5:], out[:, 3:], H, 24, width, width)
    v = src[:, 5:].reshape(N, H, 24)[:, :, :width]
    want = P.turn_halves(v, places, rot(base, dims, scaling))
    if scaling is not None and scaling[0] != 1.0:
        plain = P.turn_halves(v, places, rot(base, dims))
        assert np.abs(plain - want).max() > 0.05, "the scaling changes nothing: the test would not see it"
    tol = 2e-6 if dtype == "float32" else 2.0 ** -7
    got = host(out[:, 3:]).reshape(N, H, width)
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    assert float(out[:, :3].abs().max()) == 0.0


# ------------------------------------------------------------------------------------------ feed-forwards
def run_ff(spec, params, dtype, h):
    from deliverance_amd.parts import Arena, StepContext, build_feed_forward
    part = build_feed_forward(spec, params, DTYPES[dtype], DEV)
    ctx = StepContext()
    ctx.device, ctx.dtype, ctx.n_tokens = torch.device(DEV), DTYPES[dtype], h.shape[0]
    ctx.tokens = dev([0] * h.shape[0])
    ctx._arena = Arena(DEV)
    x = torch.zeros(h.shape[0], h.shape[1], dtype=torch.float32, device=DEV)
    part.forward(ctx, dev(h, DTYPES[dtype]), x)
    return host(x), part


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("rows,width,inner,limit", [quick(5, 64, 40, 0.5), (70, 48, 104, 2.0), (3, 36, 20, 1.0), (300, 64, 96, 0.25)])
def test_capped_gated_feed_forward(dtype, rows, width, inner, limit):
    """Sums on both sides of the limit and of its negative: the gate is capped from above only, the other half on
    both sides, and 1 is added to it."""
    from deliverance_amd.config.specs import GatedFeedForwardSpec
    helpers.skip_in_simulation_if(rows > 100)
    rng = np.random.default_rng(rows)
    W = {"gate": bf16(rng.normal(size=(inner, width)) * 0.3), "up": bf16(rng.normal(size=(inner, width)) * 0.3),
         "down": bf16(rng.normal(size=(width, inner)) * 0.2)}
    h = bf16(rng.normal(size=(rows, width)))
    g, u = h @ W["gate"].T, h @ W["up"].T
    assert (g > limit).any() and (g < -limit).any() and (u > limit).any() and (u < -limit).any()
    want = P.capped_gated(W, "", h, limit)
    got, _ = run_ff(GatedFeedForwardSpec("gated", width, inner, "glu_capped", limit=limit),
                    {"gate_up_weight": torch.cat([tb(W["gate"]), tb(W["up"])]), "down_weight": tb(W["down"])}, dtype, h)
    assert np.abs(got - want).max() <= (2e-6 if dtype == "float32" else 2e-2) * np.abs(want).max()


@pytest.mark.parametrize("experts,top", [(10, 4), quick(5, 1), (3, 3), (1, 1), (40, 7)])
def test_router_takes_the_largest_logits_and_weighs_them_among_themselves(experts, top):
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(experts)
    N = 37
    z = rng.normal(size=(N, experts)).astype(np.float32)
    b = rng.normal(size=experts).astype(np.float32)
    z[3, :] = 0.25                                          # every logit the same but for the bias
    if experts > 2:
        z[5, 0], z[5, 2] = 7.0 - b[0], 7.0 - b[2]           # a tie: the lower index comes first
        assert np.float32(z[5, 0] + b[0]) == np.float32(z[5, 2] + b[2])
    ids = torch.zeros(N, top, dtype=torch.int32, device=DEV)
    w = torch.zeros(N, top, dtype=torch.float32, device=DEV)
    ops.moe_top(dev(z, torch.float32), dev(b, torch.float32), top, "softmax", False, ids, w)
    want_ids, want_w = P.router_choice((z + b).astype(np.float64), top)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.abs(host(w) - want_w).max() <= 1e-6
    assert np.abs(host(w).sum(-1) - 1.0).max() <= 1e-6


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("rows,shape", [quick(9, (4, 2, 32, 1.25, (48, 2.0))), (150, (4, 2, 32, 1.25, (48, 2.0))),
                                        (20, (3, 3, 20, 0.7, None)), (6, (1, 1, 40, 3.0, None)), (33, (10, 3, 24, 1.25, (8, 0.4)))])
def test_routed_feed_forward_part(dtype, rows, shape):
    """Few rows (the grouped kernels that stream an expert's weights) and many (rows gathered by expert), with and
    without a shared expert whose limit differs from the experts'."""
    from deliverance_amd.config.specs import ExpertsFeedForwardSpec
    helpers.skip_in_simulation_if(rows > 100)
    n, top, ff, limit, shared = shape
    width = 64
    rng = np.random.default_rng(rows + n)
    W = {"router": bf16(rng.normal(size=(n, width)) * 0.5), "router.b": bf16(rng.normal(size=n) * 0.5)}
    for j in range(n):
        W.update({f"e{j}.gate": bf16(rng.normal(size=(ff, width)) * 0.3), f"e{j}.up": bf16(rng.normal(size=(ff, width)) * 0.3),
                  f"e{j}.down": bf16(rng.normal(size=(width, ff)) * 0.2)})
    if shared:
        W.update({"shared.gate": bf16(rng.normal(size=(shared[0], width)) * 0.3), "shared.up": bf16(rng.normal(size=(shared[0], width)) * 0.3),
                  "shared.down": bf16(rng.normal(size=(width, shared[0])) * 0.2)})
    f = moe(n, top, ff, limit, shared)
    h = bf16(rng.normal(size=(rows, width)))
    spec = ExpertsFeedForwardSpec("experts", width, ff, n, top, "glu_capped", router="softmax_top", gated=True, limit=limit,
                                  shared_inner=shared[0] if shared else 0, shared_activation="glu_capped", shared_gated=True,
                                  shared_limit=shared[1] if shared else 0.0, router_bias=True)
    params = {"gate_up_weight": torch.stack([torch.cat([tb(W[f"e{j}.gate"]), tb(W[f"e{j}.up"])]) for j in range(n)]),
              "down_weight": torch.stack([tb(W[f"e{j}.down"]) for j in range(n)]), "router_weight": tb(W["router"]),
              "router_bias": tb(W["router.b"])}
    if shared:
        params.update({"shared_gate_up_weight": torch.cat([tb(W["shared.gate"]), tb(W["shared.up"])]), "shared_down_weight": tb(W["shared.down"])})
    from deliverance_amd.parts import Arena, StepContext, build_feed_forward
    part = build_feed_forward(spec, params, DTYPES[dtype], DEV)
    ctx = StepContext()
    ctx.device, ctx.dtype, ctx.n_tokens, ctx._arena = torch.device(DEV), DTYPES[dtype], rows, Arena(DEV)
    ctx.tokens = dev([0] * rows)
    ctx.debug_hook = lambda *a: None                        # so that the part keeps its choice
    x = torch.zeros(rows, width, dtype=torch.float32, device=DEV)
    part.forward(ctx, dev(h, DTYPES[dtype]), x)
    chosen = {t: [int(e) for e in row] for t, row in enumerate(part.last_choice.cpu().numpy())}
    want = P.routed_ff(W, "", f, h, routes=chosen, slack=SLACK[dtype])
    assert np.abs(host(x) - want).max() <= (3e-6 if dtype == "float32" else 2e-2) * np.abs(want).max()


# ------------------------------------------------------------------------------------------ mixers alone
class MixerBench:
    """One mixer part with weights of its own, fed with rows h of whole sequences in steps of any cut; its additions
    to the stream are compared with the plain mixer over the whole sequences.  Pages are handed out in a shuffled
    order and start as NaN; state slots are given in any order."""

    def __init__(self, dtype, kind, m, width, seqs, page=16, seed=0, make=None, slots=None):
        from deliverance_amd.config.specs import AttentionSpec, LatentAttentionSpec, RampedSpeedsSpec, RetentionSpec, RotarySpec
        from deliverance_amd.parts import KVNeed, build_mixer
        rng = np.random.default_rng(seed)
        self.eps = 1e-5
        sc = m["rot"].get("scaling")
        turn = RotarySpec("rotary", m["rot"]["dims"], m["rot"]["base"], False,
                          None if not sc else RampedSpeedsSpec(sc["factor"], sc["original"], sc["fast"], sc["slow"]))
        nrm = lambda *shape, s=0.2: rng.normal(size=shape) * s
        if kind == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            W = {"mix.q": nrm(H * D, width), "mix.k": nrm(G * D, width), "mix.g": nrm(H * D, width, s=0.5), "mix.o": nrm(width, H * D)}
            spec = AttentionSpec("attention", width, H, G, D, m["scale"], qkv_bias=False, out_bias=False, window=m["mask"]["size"],
                                 position=turn, values_are_keys=True, sink="zero", out_gate="sigmoid")
            names = lambda t: {"qkv_weight": torch.cat([t("mix.q"), t("mix.k"), t("mix.g")]), "out_weight": t("mix.o")}
            plain = lambda h: P.attention(self.W, "", m, h)
        elif kind == "retention":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            W = {"mix.q": nrm(H * D, width), "mix.k": nrm(H * D, width), "mix.v": nrm(H * Dv, width), "mix.g": nrm(H * Dv, width, s=0.5),
                 "mix.o": nrm(width, H * Dv)}
            spec = RetentionSpec("retention", width, H, D, Dv, tuple(m["decay"]), self.eps, turn)
            names = lambda t: {"q_weight": t("mix.q"), "k_weight": t("mix.k"), "v_weight": t("mix.v"), "gate_weight": t("mix.g"),
                               "out_weight": t("mix.o")}
            plain = lambda h: P.retention(self.W, "", m, h, self.eps)
        else:
            H, dn, dr, dv, rq, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            W = {"mix.dq": nrm(rq, width), "mix.dq.norm": 1 + nrm(rq, s=0.1), "mix.uq": nrm(H * (dn + dr), rq, s=0.3),
                 "mix.dkv": nrm(r + dr, width), "mix.dkv.norm": 1 + nrm(r, s=0.1), "mix.uk": nrm(H * dn, r, s=0.3),
                 "mix.uv": nrm(H * dv, r, s=0.3), "mix.sink": nrm(H, s=1.0), "mix.o": nrm(width, H * dv)}
            spec = LatentAttentionSpec("latent_attention", width, H, dn, dr, dv, rq, r, m["scale"], self.eps, turn,
                                       window=m["mask"]["size"], sink=True)
            names = lambda t: {"q_down_weight": t("mix.dq"), "q_norm_weight": t("mix.dq.norm"), "q_up_weight": t("mix.uq"),
                               "kv_down_weight": t("mix.dkv"), "kv_norm_weight": t("mix.dkv.norm"), "k_up_weight": t("mix.uk"),
                               "v_up_weight": t("mix.uv"), "sink": t("mix.sink"), "out_weight": t("mix.o")}
            plain = lambda h: P.latent_attention(self.W, "", m, h, self.eps)
        if make is not None:
            make(W)
        self.W = {k: bf16(v) for k, v in W.items()}
        self.width, self.dtype, self.page = width, dtype, page
        self.part = build_mixer(spec, names(lambda k: tb(self.W[k])), DTYPES[dtype], DEV)
        self.seqs = [bf16(s) for s in seqs]                       # h of every sequence, [T, width]
        self.want = [plain(s) for s in self.seqs]
        need = self.part.cache_need()
        self.kv = self.state = None
        n_pages = sum(-(-len(s) // page) for s in seqs) + 3
        perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(7)).tolist()
        self.tables = [[perm.pop() for _ in range(-(-len(s) // page))] for s in seqs]
        if isinstance(need, KVNeed) and need.values_in_keys:
            self.kv = torch.full((n_pages, page * need.head_dim), float("nan"), dtype=DTYPES[dtype], device=DEV)
        elif isinstance(need, KVNeed):
            self.kv = torch.full((n_pages, 2, need.n_kv_heads, page, need.head_dim), float("nan"), dtype=DTYPES[dtype], device=DEV)
        else:
            self.slots = list(slots) if slots is not None else list(range(len(seqs)))[::-1]
            self.state = torch.zeros(max(self.slots) + 2, need.elems, dtype=torch.float32, device=DEV)
        self.done = [0] * len(seqs)

    def step(self, takes):
        """takes: {sequence: number of next tokens}; returns the largest error of the step relative to the largest
        value of the plain result."""
        from deliverance_amd.parts import Arena, StepContext
        order = sorted(takes, key=lambda s: (takes[s] != 1, s))
        ctx = StepContext()
        ctx.device, ctx.dtype = torch.device(DEV), DTYPES[self.dtype]
        lens = [takes[s] for s in order]
        total = [self.done[s] + takes[s] for s in order]
        ctx.n_seqs, ctx.n_tokens, ctx.n_decode = len(order), sum(lens), sum(1 for n in lens if n == 1)
        mb = max(len(self.tables[s]) for s in order)
        bt = torch.full((len(order), mb), -1, dtype=torch.int32)
        pos, seq_of, rows, q_start = [], [], [], [0]
        for i, s in enumerate(order):
            bt[i, :len(self.tables[s])] = torch.tensor(self.tables[s], dtype=torch.int32)
            for p in range(self.done[s], total[i]):
                pos.append(p); seq_of.append(i); rows.append(self.tables[s][p // self.page] * self.page + p % self.page)
            q_start.append(len(pos))
        ctx.positions, ctx.seq_of_token, ctx.q_start, ctx.seq_lens = dev(pos), dev(seq_of), dev(q_start), dev(total)
        ctx.tokens = dev([0] * len(pos))
        ctx.q_start_host, ctx.seq_lens_host = q_start, total
        ctx.max_query_len, ctx.max_seq_len = max(lens), max(total)
        ctx.block_tables, ctx.slot_maps = [bt.to(DEV)], [dev(rows)]
        slots = [self.slots[s] for s in order] if self.state is not None else list(range(len(order)))
        ctx.state_slots, ctx.state_slots_host = dev(slots), slots
        ctx._arena = Arena(DEV)
        ctx.cache = SimpleNamespace(page_size=self.page, group_of_slot={0: 0}, kv={0: self.kv}, state={0: self.state})
        h = np.concatenate([self.seqs[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        x = torch.zeros(len(h), self.width, dtype=torch.float32, device=DEV)
        self.part.forward(ctx, dev(h, DTYPES[self.dtype]), x, SimpleNamespace(layer=0, cache=0, write=True))
        want = np.concatenate([self.want[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        for s in order:
            self.done[s] += takes[s]
        scale = max(np.abs(w).max() for w in self.want)
        return np.abs(host(x) - want).max() / scale


def walk(b, tol):
    """Three sequences of 70, 33 and 1 tokens in portions, decoded tokens and both at once."""
    assert b.step({0: 33, 1: 2}) <= tol                  # portions; the second ends inside a page
    assert b.step({0: 1, 1: 1, 2: 1}) <= tol             # decoding beside a first token
    assert b.step({0: 30, 1: 14}) <= tol                 # across a tile of 32 keys and page borders
    assert b.step({0: 1, 1: 1}) <= tol
    assert b.step({0: 5, 1: 15}) <= tol
    assert b.done == [70, 33, 1]


MIX = lambda d: d["mixer"]
ATTENTIONS = [quick(MIX(att(4, 2, 16, 0.25, 40, 10000.0, 8))),       # matrix cores; the window ends inside the prompts
              MIX(att(3, 1, 12, 0.3, 500, 500.0, 6)),               # a head size the matrix-core kernel leaves to the plain one
              MIX(att(2, 2, 64, 0.125, 17, 1e6, 64)),               # every entry turns; a window shorter than two pages
              quick(MIX(att(6, 3, 32, 0.2, 1, 10000.0, 0)))]        # a token sees itself only; nothing turns
RETENTIONS = [quick(MIX(ret(2, 16, 24, (0.9, 1.0), 10000.0, 16))),
              MIX(ret(3, 20, 12, (0.0, 0.5, 0.999), 100.0, 20)),    # rows that do not fill the lanes; a decay of 0
              quick(MIX(ret(1, 64, 40, (0.9375,), 1e6, 32))),      # columns that do not fill the last block
              MIX(ret(2, 136, 8, (0.9990234375, 0.25), 500.0, 0))]  # nine rows a lane; nothing turns
LATENTS = [quick(MIX(lat(2, 16, 8, 24, 24, 40, 0.2, 24, 10000.0, (4.0, 64, 8.0, 1.0)))),
           MIX(lat(3, 8, 12, 20, 18, 27, 0.3, 300, 500.0)),          # rows of 39 entries: the plain kernel
           quick(MIX(lat(5, 32, 32, 16, 48, 160, 0.1, 33, 10000.0, (3.0, 512, 24.0, 2.0)))),
           MIX(lat(1, 16, 16, 16, 16, 16, 0.25, 2, 100.0))]          # a window of two keys


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", ATTENTIONS)
def test_attention_part_prompt_portions_and_decoding(m, dtype):
    rng = np.random.default_rng(5)
    walk(MixerBench(dtype, "attention", m, 64, [rng.normal(size=(n, 64)) for n in (70, 33, 1)]), 2e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", RETENTIONS)
def test_retention_part_prompt_portions_and_decoding(m, dtype):
    """The state rows are handed out in any order.  (A decay of 0 leaves a head with the last token alone, whose
    read-out norm then divides by |q . k|: whole models keep away from it, since rounding decides the sign of a
    product near zero.)"""
    rng = np.random.default_rng(6)
    helpers.skip_in_simulation_if(m["dim"] > 100 and dtype == "float32")
    b = MixerBench(dtype, "retention", m, 48, [rng.normal(size=(n, 48)) for n in (70, 33, 1)], slots=[3, 0, 2])
    walk(b, 2e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", LATENTS)
def test_latent_attention_part_prompt_portions_and_decoding(m, dtype):
    rng = np.random.default_rng(7)
    helpers.skip_in_simulation_if(m["kv_rank"] > 100 and dtype == "float32")
    walk(MixerBench(dtype, "latent_attention", m, 64, [rng.normal(size=(n, 64)) for n in (70, 33, 1)]), 2e-5 if dtype == "float32" else 3e-2)


def marked_attention(W):
    """Input channel 0 makes a large key, channel 1 a large query: the one pair of marked tokens has a score far
    above all others."""
    W["mix.q"] *= 0.1
    W["mix.k"] *= 0.1
    W["mix.k"][:, 0] = 1.0
    W["mix.q"][:, 1] = 1.0


def marked_latent(W, r):
    W["mix.uq"] *= 0.05
    W["mix.dkv"][r:, 0] = 3.0           # the marked token's key piece is large in every entry
    W["mix.dq"][0, 1] = 8.0             # the asking token's query latent is large in entry 0 ...
    W["mix.uq"][:, 0] = np.where(np.arange(W["mix.uq"].shape[0]) % 32 >= 16, 2.0, 0.0)   # ... which feeds the rotated query entries


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("window,back", [quick(56, 55), (56, 56), (24, 23), quick(24, 24), (16, 15), (16, 16), (33, 32), (33, 33),
                                         (300, 250), (300, 1)])
def test_a_key_just_inside_and_just_outside_the_window(kind, window, back, dtype):
    """The last query matches the key ``back`` tokens before it far better than any other.  With back < window the
    output is that token's value; with back == window the key is no longer seen, and what is left are small scores
    beside the term without a key.  A window that is one token off, or a key read from a page that was given back,
    shows as an error of the order of the output; in a prompt and in decoding, at page borders and inside pages."""
    T, width = 261, 32
    rng = np.random.default_rng(window + back)
    h = rng.normal(size=(T, width)) * 0.1
    h[T - 1 - back, 0] = 6.0
    h[T - 1, 1] = 6.0
    if kind == "attention":
        m = MIX(att(2, 1, 16, 1.0, window, 10000.0, 0))
        make = marked_attention
    else:
        m = MIX(lat(2, 16, 16, 16, 16, 32, 1.0, window, 10000.0))
        m["rot"]["dims"] = 0                     # nothing turns: the key piece is matched as it is
        make = lambda W: marked_latent(W, 32)
    tol = 2e-5 if dtype == "float32" else 3e-2
    for decode in (False, True):
        b = MixerBench(dtype, kind, m, width, [h], seed=1, make=make)
        if decode:
            assert b.step({0: T - 1}) < 1.0
            err = b.step({0: 1})
        else:
            err = b.step({0: T})
        assert err <= tol, f"decode={decode}: {err}"
    # the test sees what it is meant to see: the far key decides the plain result at the last position
    other = dict(m, mask={"size": back if back < window else back + 1})
    plain = P.attention if kind == "attention" else (lambda W, p, mm, hh: P.latent_attention(W, p, mm, hh, 1e-5))
    a, c = plain(b.W, "", m, b.seqs[0])[-1], plain(b.W, "", other, b.seqs[0])[-1]
    assert np.abs(a - c).max() > 0.2 * max(np.abs(a).max(), np.abs(c).max())


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_the_term_without_a_key_takes_its_share(kind, dtype):
    """All scores well below zero: most of the softmax's weight goes to the term that has no value, and the result is
    a fraction of the values' average.  Left out, or counted once a share of the keys, the result would be another."""
    T, width = 40, 32
    rng = np.random.default_rng(3)
    h = rng.normal(size=(T, width)) * 0.1
    h[:, 0] = 1.0
    h[:, 1] = -0.3
    if kind == "attention":
        m = MIX(att(2, 1, 16, 1.0, 64, 10000.0, 0))
        make = marked_attention
    else:
        m = MIX(lat(2, 16, 16, 16, 16, 32, 1.0 / 80, 64, 10000.0))      # (the query latent's norm makes its marked entry large)
        m["rot"]["dims"] = 0

        def make(W):
            marked_latent(W, 32)
            W["mix.sink"][:] = [0.5, -1.0]
    b = MixerBench(dtype, kind, m, width, [h], seed=2, make=make)
    plain = P.attention if kind == "attention" else (lambda W, p, mm, hh: P.latent_attention(W, p, mm, hh, 1e-5))
    keep, P.softmax_with_sink = P.softmax_with_sink, lambda s_, mask, sink: keep(s_, mask, np.full_like(sink, -1e9))
    try:
        without = plain(b.W, "", m, b.seqs[0])
    finally:
        P.softmax_with_sink = keep
    assert np.abs(without).max() > 2.0 * np.abs(b.want[0]).max(), "the term takes too little for the test to see it"
    assert b.step({0: T - 3}) <= (2e-5 if dtype == "float32" else 3e-2)
    for _ in range(3):
        assert b.step({0: 1}) <= (2e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_retention_remembers_the_first_token(dtype):
    """A head whose decay is 1 keeps the first token's key and value for good: after 300 tokens, cut into portions and
    decoded tokens, a query that matches that key alone reads that value; the head beside it has forgotten it."""
    T, width = 300, 32
    rng = np.random.default_rng(8)
    h = rng.normal(size=(T, width)) * 0.05
    h[0, 0] = 5.0
    h[T - 1, 1] = 5.0
    m = MIX(ret(2, 16, 16, (1.0, 0.9), 10000.0, 0))

    def make(W):
        W["mix.q"] *= 0.1
        W["mix.k"] *= 0.1
        W["mix.k"][:, 0] = 1.0
        W["mix.q"][:, 1] = 1.0
    b = MixerBench(dtype, "retention", m, width, [h], seed=3, make=make, slots=[1])
    tol = 2e-5 if dtype == "float32" else 3e-2
    for n in (150, 2, 100, 1, 1, 44, 1, 1):
        assert b.step({0: n}) <= tol
    assert b.done == [T]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("chunk", [16, quick(32), 48])
def test_retention_in_chunks_side_by_side(dtype, chunk):
    """Long portions are walked in chunks that run side by side, with a carry pass between them: the same results and
    the same kept states as the walk in one piece, by 32-bit rounding; portions that end inside a chunk, at a chunk's
    edge, and one-token sequences beside them; states that are kept and states that are not."""
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(chunk)
    H, D, Dv = 3, 20, 24
    lens = [70, 1, 33, 2 * chunk, 1]
    N, S = sum(lens), len(lens)
    cols = 2 * H * D + H * Dv
    qkv = dev(bf16(rng.normal(size=(N, cols + 5)) * 0.5), DTYPES[dtype])
    decay = dev([0.5, 0.9375, 1.0], torch.float32)
    q_start = np.concatenate([[0], np.cumsum(lens)])
    state0 = rng.normal(size=(S + 1, H * Dv * D + 3)).astype(np.float32)
    ctx = SimpleNamespace(q_start=dev(q_start), state_slots=dev([4, 1, -1, 0, 3]), n_seqs=S, max_query_len=max(lens),
                          buf=lambda name, r, c_, dt: torch.empty(r, c_, dtype=dt, device=DEV))
    outs = {}
    for write in (True, False):
        for ch in (0, chunk):
            st = dev(state0, torch.float32)
            o = torch.full((N, H * Dv), float("nan"), dtype=torch.float32, device=DEV)
            ops.retention(ctx, qkv, 2, 2 + H * D, 2 + 2 * H * D, decay, D ** -0.5, st, o, H, D, Dv, write=write, chunk=ch)
            outs[(write, ch)] = (host(o), host(st))
        a, b = outs[(write, 0)], outs[(write, chunk)]
        assert np.isfinite(b[0]).all()
        assert np.abs(a[0] - b[0]).max() <= 2e-6 * np.abs(a[0]).max()
        assert np.abs(a[1] - b[1]).max() <= 2e-6 * np.abs(a[1]).max()
        if not write:
            assert np.array_equal(b[1], state0.astype(np.float64))
    assert np.array_equal(outs[(True, chunk)][1][2], state0[2].astype(np.float64)), "a slot that no sequence has was written"
    # and the walk in one piece against the formula, from the given states
    x = host(qkv)[:, 2:2 + cols]
    want = np.zeros((N, H, Dv))
    slots = [4, 1, -1, 0, 3]
    for s_, (a0, a1) in enumerate(zip(q_start[:-1], q_start[1:])):
        for h_ in range(H):
            St = np.zeros((D, Dv)) if slots[s_] < 0 else state0[slots[s_], h_ * Dv * D:(h_ + 1) * Dv * D].reshape(Dv, D).T.astype(np.float64)
            for t in range(a0, a1):
                q, k = x[t, h_ * D:(h_ + 1) * D], x[t, H * D + h_ * D:H * D + (h_ + 1) * D] * D ** -0.5
                v = x[t, 2 * H * D + h_ * Dv:2 * H * D + (h_ + 1) * Dv]
                St = float(host(decay)[h_]) * St + np.outer(k, v)
                want[t, h_] = St.T @ q
    assert np.abs(outs[(True, 0)][0] - want.reshape(N, H * Dv)).max() <= 3e-6 * np.abs(want).max()


# ------------------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def smodels(tmp_path_factory):
    return {"S": make_model(tmp_path_factory.mktemp("ss"), CONFIG_S, 41), "T": make_model(tmp_path_factory.mktemp("st"), CONFIG_T, 42),
            "U": make_model(tmp_path_factory.mktemp("su"), CONFIG_U, 43)}


def check(model, got, routes, requests, dtype, what=""):
    """32-bit: every logit within 3e-5 of the largest plain logit.  bfloat16: the largest error within 5 % of the
    logits' root mean square and the rms error within 2^-6 of it; at a sequence's first position four times that: a
    retention head's state is then one token's k v^T, its read-out (q . k) v, and the norm behind it divides by
    |q . k|, which rounding moves by any factor where the product is near zero.  The plain model follows the engine's
    choice of experts where two logits are nearly equal, and fails where the engine's choice is not nearly as good as
    its own."""
    for rid, ids in requests:
        ref = model.plain_logits(ids, routes.get(rid, {}), SLACK[dtype])
        out = got[rid].astype(np.float64)
        assert out.shape == ref.shape, f"{what} {rid}: shape {out.shape} vs {ref.shape}"
        err = np.abs(out - ref)
        rms = float(np.sqrt((ref ** 2).mean()))
        bound = np.full(len(ids), 3e-5 * np.abs(ref).max() if dtype == "float32" else 5e-2 * rms)
        if dtype == "bfloat16":
            bound[0] *= 4.0
        over = err.max(axis=1) > bound
        first = int(np.argmax(over))
        assert not over.any(), f"{what} {rid} ({dtype}): max error {err[first].max():.3e} > {bound[first]:.3e}, first at position {first}"
        if dtype == "bfloat16" and len(ids) > 1:
            assert float(np.sqrt((err[1:] ** 2).mean())) <= 2.0 ** -6 * rms, f"{what} {rid}: rms error"


def run(model, session, steps, requests, dtype, what):
    got, routes = replay_routed(session, steps, model.cfg)
    check(model, got, routes, requests, dtype, what)
    return got


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("S"), "T", "U"])
def test_whole_prompts_and_first_tokens(smodels, name, dtype):
    m = smodels[name]
    reqs = [("one", m.prompt(1)), ("two", m.prompt(2)), ("three", m.prompt(3)), ("long", m.prompt(90))]
    s = helpers.trace_session(m.folder, dtype, 256, state_slots=2)
    for rid, ids in reqs:
        run(m, s, helpers.trace_whole(rid, ids), [(rid, ids)], dtype, "whole")
    s.cache.manager.check()


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["S", quick("T"), "U"])
def test_prefill_against_token_by_token_decoding(smodels, name, dtype):
    """All but the last 45 tokens at once, the rest one by one, across page borders, tiles of keys and the windows'
    edges; then a request that is decoded from its very first token on."""
    m = smodels[name]
    ids = m.prompt(75, salt=1)
    s = helpers.trace_session(m.folder, dtype, 128, state_slots=1)
    run(m, s, helpers.trace_bulk_then_single("r", ids, tail=45), [("r", ids)], dtype, "decode")
    ids2 = m.prompt(20, salt=2)
    run(m, s, helpers.trace_bulk_then_single("q", ids2, tail=19), [("q", ids2)], dtype, "decode from 1")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("S"), "T", "U"])
@pytest.mark.parametrize("sizes", [(7, 2, 13, 3, 5, 2), quick((2, 2, 31, 1, 16, 33, 2))])
def test_portions_of_any_size(smodels, name, dtype, sizes):
    m = smodels[name]
    ids = m.prompt(97, salt=3)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True, state_slots=1)
    run(m, s, helpers.trace_portions("r", ids, sizes), [("r", ids)], dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["S", "T", quick("U")])
def test_mixed_batches_over_a_small_pool(smodels, name, dtype):
    """Seven unequal requests, four live at a time, over a pool that holds just what is live and four state slots:
    pages and slots come back and go out again (freed pages are filled with NaN, windows give pages back while a
    request runs).  Then some of them alone: what a request gets must not depend on its neighbours beyond rounding."""
    m = smodels[name]
    reqs = [(f"r{i}", m.prompt(n, salt=10 + i)) for i, n in enumerate((40, 3, 71, 18, 64, 1, 33))]
    steps = helpers.trace_mixed(reqs, seed=5, max_live=4)
    s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True, state_slots=4)
    got = run(m, s, steps, reqs, dtype, "mixed")
    s.cache.manager.check()
    if dtype == "float32":
        alone = helpers.trace_session(m.folder, dtype, 128, state_slots=1)
        for rid, ids in reqs[:3]:
            one = helpers.replay(alone, helpers.trace_whole(rid, ids))[rid]
            scale = float(np.sqrt((one.astype(np.float64) ** 2).mean()))
            assert np.abs(one.astype(np.float64) - got[rid]).max() <= 2e-5 * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts(smodels, dtype):
    """Prompts of several hundred tokens at once and in long portions (the forms that kernels keep for long portions),
    beside a short one; then decoding goes on from what they left."""
    helpers.skip_in_simulation_if(True)
    m = smodels["S"]
    ids, other = m.prompt(700, salt=40), m.prompt(9, salt=41)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:300], "want": list(range(300))}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": other[:8], "want": list(range(8))},
                                     {"id": "a", "tokens": ids[300:690], "want": list(range(390))}], "end": []}]
    for i in range(690, 700):
        entries = [{"id": "a", "tokens": [ids[i]], "want": [0]}]
        if i == 690:
            entries.append({"id": "b", "tokens": [other[8]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["b"] if i == 690 else []})
    steps[-1]["end"].append("a")
    s = helpers.trace_session(m.folder, dtype, 832, poison_freed=True, state_slots=2)
    run(m, s, steps, [("a", ids), ("b", other)], dtype, "long prompts")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, dtype):
    """Three hundred tokens one by one beside a neighbour that comes and goes, in a model whose layers use all of their
    experts (nothing hangs on a choice), whose windows pass over decoded tokens and whose retention forgets slowly."""
    helpers.skip_in_simulation_if(True)
    cfg = config(90, 40, 1e-5,
                 [layer(ret(2, 8, 16, (0.99, 0.9990234375), 10000.0, 8), moe(2, 2, 24, 1.0, (8, 1.5))),
                  layer(lat(2, 8, 16, 8, 16, 24, 0.3, 100, 10000.0, (2.0, 128, 16.0, 1.0)), moe(3, 3, 16, 1.0)),
                  layer(att(2, 1, 16, 0.25, 50, 10000.0, 16), dense(24, 1.0))], loop=(0, 2, 2))
    m = make_model(tmp_path / "m", cfg, 31)
    ids, other = m.prompt(310, salt=20), m.prompt(60, salt=21)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:10], "want": list(range(10))}], "end": []}]
    for i in range(10, len(ids)):
        entries = [{"id": "a", "tokens": [ids[i]], "want": [0]}]
        j = i - 50
        if 0 <= j < len(other):
            entries.append({"id": "b", "tokens": [other[j]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["b"] if j == len(other) - 1 else []})
    steps[-1]["end"].append("a")
    s = helpers.trace_session(m.folder, dtype, 448, poison_freed=True, state_slots=2)
    got = helpers.replay(s, steps)
    check(m, got, {}, [("a", ids), ("b", other)], dtype, "long decode")


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["S", "T"])
def test_greedy_generation_through_the_engine(smodels, name, dtype):
    """The engine's own entry point and scheduler: several prompts at once over a pool that forces portions, with
    recorded decode steps and steps launched ahead.  Every generated token must be (nearly) the best under the plain
    model given the tokens before it."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = smodels[name]
    prompts = [m.prompt(n, salt=30 + n) for n in (5, 33, 70, 2)]
    model = AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=512, max_num_seqs=3,
                                                 max_batch_tokens=48, max_chunk=32)
    outs = model.generate(prompts, GeneratorParameters(max_tokens=24, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.finish_reason == "length" and len(out.generated_tokens) == 24
        ids = list(prompt) + list(out.generated_tokens)
        ref = m.plain_logits(ids)
        for k, t in enumerate(out.generated_tokens):
            row = ref[len(prompt) + k - 1]
            slack = 1e-3 if dtype == "float32" else 2 * 5e-2 * float(np.sqrt((row ** 2).mean()))
            assert row[t] >= row.max() - slack


# ------------------------------------------------------------------------------------------ random configurations
def random_config(seed):
    """Sizes drawn at random, among them what the kernels take only on their plain paths (widths and ranks that are no
    multiple of 8, head sizes that the matrix-core attention does not take), one expert, as many experts a token as
    there are, windows of one key and longer than the prompt, loops anywhere."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = pick(40, 50, 64, 100, 72, 36)
    layers = []
    for i in range(int(rng.integers(1, 5))):
        n = pick(1, 2, 5, 9)
        mlp = pick(None, "moe", "moe", "dense")
        if mlp == "moe":
            mlp = moe(n, pick(1, n, max(1, n // 2)), pick(8, 20, 32), float(pick(0.5, 1.0, 7.0)), pick(None, (8, 1.5), (24, 0.3)))
        elif mlp == "dense":
            mlp = dense(pick(16, 40, 100), float(pick(0.5, 1.0, 7.0)))
        kind = pick("attention", "retention", "latent_attention")
        if kind == "attention":
            g, d = pick(1, 2, 3), pick(8, 16, 20, 32, 64)
            mixer = att(g * pick(1, 2, 3), g, d, float(pick(0.1, 0.25, 0.4)), pick(1, 7, 16, 40, 1000), float(pick(100.0, 1e4, 1e6)), pick(0, 2, d // 2, d))
        elif kind == "retention":
            h, d = pick(1, 2, 5), pick(4, 16, 24, 40)
            mixer = ret(h, d, pick(4, 16, 24, 40), [float(pick(0.5, 0.9, 1.0, 0.998046875)) for _ in range(h)], float(pick(100.0, 1e4)), pick(0, 2, d // 2, d))
        else:
            dr = pick(2, 8, 16, 24)
            mixer = lat(pick(1, 2, 3, 6), pick(8, 16, 20, 32), dr, pick(8, 16, 40), pick(8, 12, 32), pick(8, 24, 30, 64),
                        float(pick(0.1, 0.25, 0.4)), pick(1, 7, 16, 40, 1000), float(pick(100.0, 1e4, 1e6)),
                        pick(None, (2.0, 64, 8.0, 1.0), (16.0, 32, 4.0, 0.5)))
        layers.append(layer(mixer, mlp))
    loop = None
    if rng.random() < 0.6:
        a = int(rng.integers(0, len(layers)))
        loop = (a, int(rng.integers(a + 1, len(layers) + 1)), pick(1, 2, 3))
    return config(pick(50, 130, 257), width, float(pick(1e-6, 1e-5, 1e-3)), layers, loop)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(14))
def test_random_configurations(tmp_path, seed, dtype):
    m = make_model(tmp_path / "m", random_config(seed), 100 + seed)
    ids = m.prompt(45, salt=seed)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True, state_slots=2)
    run(m, s, helpers.trace_whole("w", ids), [("w", ids)], dtype, f"seed {seed} whole")
    run(m, s, helpers.trace_portions("p", ids, (5, 2, 17, 1, 1, 9)), [("p", ids)], dtype, f"seed {seed} portions")
