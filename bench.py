#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens a second at a fixed batch, prefill of 2,048
tokens, and the decode step's fraction of the HBM roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model 124m|355m|1.5b] [--batch B]

A "step" is one decode step of the engine (scheduler decision, model step over the paged cache,
sampling on the device, tokens back on the host).  Weights are random (N(0, 0.02)), prompts are
seeded uniform-random token ids of 512 tokens, decoding is greedy and ignores end tokens.

The default run measures GPT-2 124M layer sizes (the headline `value`: batch 8; `points`: batch 1
and 64; `prefill`: one step of 2 x 1,024 tokens) and then, into the same line, GPT-2 1.5B layer
sizes (decode at batch 1, 8, 64 and the same prefill) and the mixed workload at GPT-2 355M layer
sizes (64 requests at once, prompt portions of 512 tokens beside the others' decoding), each with
its fraction of the roofline; `--no-extra` leaves those two out.  Prints ONE JSON line.

`--design virudra` measures another design beside GPT-2 at equal sizes instead (width, heads, head size, layers,
vocabulary, feed-forward parameters that a token uses): decode at batch 1, 8 and 64 and the prefill of 2 x 1,024
tokens for both, at the layer sizes of GPT-2 124M and 355M, one JSON line; with `--profile-stages` also both
models' kernel tables (stderr).  `--design pedatar` does the same for a third design beside Virudra (the closest
of the engine's models to it), `--design pafolorn` for a fourth beside Pedatar, and `--design salivik` for a fifth beside Pedatar.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# GPT-2 layer sizes (random weights; n_positions 1024, vocabulary 50257, tied head)
MODELS = {
    "124m": dict(n_layer=12, n_embd=768, n_head=12),
    "355m": dict(n_layer=24, n_embd=1024, n_head=16),
    "1.5b": dict(n_layer=48, n_embd=1600, n_head=25),
}
# MI355X published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
SETTLE_STEPS = 3        # decode steps before the warm-up: the first records the step's HIP graph


def model_config(name, n_layer=None, n_positions=1024):
    c = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", vocab_size=50257, n_positions=n_positions,
             layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=50256, eos_token_id=50256)
    c.update(MODELS[name])
    if n_layer is not None:
        c["n_layer"] = n_layer
    return c


def weight_bytes(c, el):
    E, I, V, L = c["n_embd"], 4 * c["n_embd"], c["vocab_size"], c["n_layer"]
    per_layer = (3 * E * E + E * E + 2 * E * I) * el + (3 * E + E + I + E + 4 * E) * el
    return L * per_layer + V * E * el + 2 * E * el          # blocks + head table (read once) + ln_f


def step_flops(c, seq_lens_new, past=0):
    """Matrix-product and attention flops of a step that brings ``seq_lens_new`` tokens per sequence."""
    E, I, V, L = c["n_embd"], 4 * c["n_embd"], c["vocab_size"], c["n_layer"]
    n = sum(seq_lens_new)
    gemm = 2 * n * (3 * E * E + E * E + 2 * E * I) * L + 2 * len(seq_lens_new) * E * V
    attn = 0
    for t in seq_lens_new:
        keys = sum(past + i + 1 for i in range(t))
        attn += 4 * keys * E * L
    return gemm + attn


def decode_roofline(cfg, el, batch, ctx_mean, seconds_per_step):
    """Bytes a decode step must read (every weight once, the live requests' cache) over its time."""
    kv_bytes_per_token = 2 * cfg["n_embd"] * el * cfg["n_layer"]
    step_bytes = weight_bytes(cfg, el) + batch * ctx_mean * kv_bytes_per_token
    return step_bytes / seconds_per_step / 1e9


def engine_from_folder(folder, dtype, seats, cfg, **kw):
    from deliverance_amd import AutoModelForCausalLM
    kw.setdefault("max_batch_tokens", max(2048, seats))
    kw.setdefault("max_chunk", 1024)
    kw.setdefault("page_size", 16)
    return AutoModelForCausalLM.from_pretrained(folder, dtype=dtype, max_num_seqs=max(seats, 2),
                                                max_cached_tokens=max(seats, 2) * cfg["n_positions"], **kw)


def engine_from_gpu_weights(cfg, dtype, seats, seed=0, **kw):
    """The same engine with its random weights drawn on the GPU (the tensors that the architecture
    declares, with the standard deviations it declares for them), for the models whose checkpoint would
    take longer to write to disk and read back than to measure."""
    import torch
    import deliverance_amd.models  # noqa: F401
    from deliverance_amd import EngineConfig
    from deliverance_amd.engine.engine import CausalLanguageModel
    from deliverance_amd.models.causal_lm import CausalLM
    from deliverance_amd.registry import ModelSupport
    arch = ModelSupport.detect(cfg)
    mc = arch.read_config(cfg)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    tensors = {}
    for d in arch.declare_tensors(mc):
        if d.optional:
            continue
        if d.init == "distinct_ints":                  # (a table of integers: drawn as the random-weights mode draws it)
            from deliverance_amd.weights.loader import draw_tensor
            tensors[d.name] = draw_tensor(d, seed).to("cuda:0")
            continue
        t = torch.randn(d.shape, generator=g, device="cuda:0", dtype=torch.float32) * d.std
        if d.init == "ones_plus_normal":
            t += 1.0
        tensors[d.name] = t.to(torch.bfloat16)
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    model = CausalLM(mc, arch.bind_tensors(mc, tensors), tdt, "cuda:0")
    del tensors
    kw.setdefault("max_batch_tokens", max(2048, seats))
    kw.setdefault("max_chunk", 1024)
    kw.setdefault("page_size", 16)
    pool = kw.pop("max_cached_tokens", max(seats, 2) * cfg["n_positions"])
    ec = EngineConfig(dtype=dtype, max_num_seqs=max(seats, 2), max_cached_tokens=pool, **kw)
    return CausalLanguageModel(model, ec)


def virudra_config(name, n_positions=1024):
    """A Virudra of GPT-2 ``name``'s sizes: as many layers, heads and key heads of the same head size, dense gated
    feed-forwards and mixtures of 8 experts (2 a token) in turn whose matrices that a token uses hold what GPT-2's
    two hold (3 x width x 8/3 width), a bias table of 32 rows up to a distance of 512, no loop."""
    g = MODELS[name]
    E, H = g["n_embd"], g["n_head"]
    D = E // H
    F = (8 * E // 3 + 63) // 64 * 64
    mixer = {"heads": H, "kv_heads": H, "dim": D, "vdim": D, "scale": D ** -0.5, "bias_max": 512, "bias_buckets": 32,
             "q_temp": {"coef": 0.1, "every": 256}}
    layers = [{"type": "attention", "mixer": mixer,
               "mlp": {"kind": "dense", "ff": F} if i % 2 == 0 else
                      {"kind": "moe", "expert": {"ff": F // 2}, "router": {"experts": 8, "top": 2}}}
              for i in range(g["n_layer"])]
    return {"architecture": "Virudra", "vocab": 50257, "width": E, "norm": {"eps": 1e-5}, "logit_softcap": 50.0,
            "layers": layers, "max_positions": n_positions,
            # what decode_run and prefill_run read
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": g["n_layer"], "n_embd": E, "ff": F}


def virudra_weight_bytes(c, el, batch):
    """What a decode step must read of the weights: every matrix once, of the experts as many as ``batch`` tokens
    can choose (2 each of 8)."""
    E, F, V = c["width"], c["ff"], c["vocab"]
    n = 0
    for L in c["layers"]:
        n += 4 * E * E
        n += 3 * E * F if L["mlp"]["kind"] == "dense" else min(8, 2 * batch) * 3 * E * (F // 2)
    return (n + V * E) * el


def virudra_step_flops(c, seq_lens_new):
    E, F, V = c["width"], c["ff"], c["vocab"]
    n = sum(seq_lens_new)
    gemm = 2 * n * (4 * E * E + 3 * E * F) * len(c["layers"]) + 2 * len(seq_lens_new) * E * V
    attn = sum(4 * sum(i + 1 for i in range(t)) * E * len(c["layers"]) for t in seq_lens_new)
    return gemm + attn


def pedatar_config(name, n_positions=1024):
    """A Pedatar of GPT-2 ``name``'s sizes: as many layers, latent attention and selective scans in turn.  Attention:
    GPT-2's heads with 64 query entries each (48 unrotated, 16 rotated) and values of 64, a query latent of half the
    width, a latent of a quarter of the width beside a key piece of 16.  Scan: twice the width of channels, 16 state
    entries, width / 16 step-size numbers, 4 taps.  Feed-forward: 8 experts of the width's size (2 a token) and a
    shared one of twice the width, which is what GPT-2's two matrices hold for a token."""
    g = MODELS[name]
    E, H = g["n_embd"], g["n_head"]
    att = {"heads": H, "dim": 48, "rot_dim": 16, "vdim": 64, "q_rank": E // 2, "kv_rank": E // 4, "scale": 64 ** -0.5,
           "rot": {"base": 10000.0, "dims": 16}}
    scan = {"inner": 2 * E, "state": 16, "dt_rank": E // 16, "conv": 4}
    mlp = {"kind": "moe", "expert": {"ff": E}, "router": {"experts": 8, "top": 2}, "shared": {"ff": 2 * E}}
    layers = [{"type": "latent_attention", "mixer": att, "mlp": mlp} if i % 2 == 0 else {"type": "mamba1", "mixer": scan, "mlp": mlp}
              for i in range(g["n_layer"])]
    return {"architecture": "Pedatar", "vocab": 50257, "width": E, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "layers": layers, "max_positions": n_positions,
            # what decode_run and prefill_run read
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": g["n_layer"], "n_embd": E}


def _pedatar_layer_params(c, L, experts_used):
    E = c["width"]
    m = L["mixer"]
    if L["type"] == "latent_attention":
        H, qd = m["heads"], m["dim"] + m["rot_dim"]
        n = E * (m["q_rank"] + m["kv_rank"] + m["rot_dim"]) + m["q_rank"] * H * qd + m["kv_rank"] * H * (m["dim"] + m["vdim"]) + H * m["vdim"] * E
    else:
        I = m["inner"]
        n = 2 * I * E + I * (m["dt_rank"] + 2 * m["state"]) + m["dt_rank"] * I + I * m["state"] + I * E
    f = L["mlp"]
    return n + 2 * E * (experts_used * f["expert"]["ff"] + f["shared"]["ff"]) + f["router"]["experts"] * E


def pedatar_step_bytes(c, el, batch, ctx_mean):
    """What a decode step must read: every matrix once (of the experts as many as ``batch`` tokens can choose), the
    live requests' latent rows, and the scans' states (read and written, 32-bit)."""
    n, extra = c["vocab"] * c["width"], 0
    for L in c["layers"]:
        f = L["mlp"]["router"]
        n += _pedatar_layer_params(c, L, min(f["experts"], f["top"] * batch))
        m = L["mixer"]
        if L["type"] == "latent_attention":
            extra += batch * ctx_mean * (m["kv_rank"] + m["rot_dim"]) * el
        else:
            extra += batch * 2 * 4 * m["inner"] * (m["state"] + m["conv"] - 1)
    return n * el + extra


def pedatar_step_flops(c, seq_lens_new):
    """Matrix-product flops of a step (the parameters a token uses, twice), the folded attention's two products over
    rows of latent + key piece and of latent entries, and the scan's six operations a state entry."""
    n = sum(seq_lens_new)
    fl = 2 * len(seq_lens_new) * c["width"] * c["vocab"]
    for L in c["layers"]:
        fl += 2 * n * _pedatar_layer_params(c, L, L["mlp"]["router"]["top"])
        m = L["mixer"]
        if L["type"] == "latent_attention":
            pairs = sum(sum(i + 1 for i in range(t)) for t in seq_lens_new)
            fl += 2 * pairs * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"])
        else:
            fl += 6 * n * m["inner"] * m["state"]
    return fl


def pafolorn_config(name, n_positions=1024):
    """A Pafolorn of GPT-2 ``name``'s sizes: as many layers, a delta rule with a decay per key channel and a parallel
    mixer in turn.  Delta rule alone: GPT-2's heads with 64 key and 64 value entries each, 4 taps, decay and gate
    through low ranks of width / 16 and width / 8.  Parallel: attention and a delta rule with half of GPT-2's heads
    each (64 entries, the first 32 rotated, a window of 512 keys that keeps the first 4, scores capped at 30).
    Feed-forwards of four times the width, which with the mixers is about what a GPT-2 layer holds."""
    g = MODELS[name]
    E, H = g["n_embd"], g["n_head"]
    alone = {"heads": H, "kv_heads": H, "dim": 64, "vdim": 64, "conv": 4, "a_rank": E // 16, "g_rank": E // 8}
    left = {"heads": H // 2, "kv_heads": H // 2, "dim": 64, "vdim": 64, "scale": 64 ** -0.5, "softcap": 30.0,
            "mask": {"size": 512, "keep_first": 4}, "rot": {"base": 10000.0, "dims": 32}}
    right = {"heads": H // 2, "kv_heads": H // 2, "dim": 64, "vdim": 64, "conv": 4}
    mlp = {"kind": "dense", "ff": 4 * E}
    layers = [{"type": "channel_delta", "mixer": alone, "mlp": mlp} if i % 2 == 0 else
              {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 0.5, "right_scale": 0.5}, "mlp": mlp}
              for i in range(g["n_layer"])]
    return {"architecture": "Pafolorn", "vocab": 50257, "width": E, "norm": {"eps": 1e-5}, "logit_scale": 0.25,
            "layers": layers, "max_positions": n_positions,
            # what decode_run and prefill_run read
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": g["n_layer"], "n_embd": E}


def _pafolorn_delta_params(E, m, channel):
    qk, v = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
    n = E * (2 * qk + v) + m["heads"] * E + v * E
    if channel:
        n += m["a_rank"] * (E + m["heads"] * m["dim"]) + m["g_rank"] * (E + v)
    else:
        n += m["heads"] * E + v * E
    return n


def _pafolorn_layer_params(c, L):
    E, m = c["width"], L["mixer"]
    if L["type"] == "channel_delta":
        n = _pafolorn_delta_params(E, m, True)
    else:
        a = m["left"]
        n = E * (a["heads"] * a["dim"] + a["kv_heads"] * (a["dim"] + a["vdim"])) + a["heads"] * a["vdim"] * E
        n += _pafolorn_delta_params(E, m["right"], False)
    return n + (2 * E * L["mlp"]["ff"] if L["mlp"] else 0)


def pafolorn_step_bytes(c, el, batch, ctx_mean):
    """What a decode step must read: every matrix once, the delta rules' states and filter inputs (read and written,
    32-bit), and the keys and values that the windows see."""
    n, extra = c["vocab"] * c["width"], 0
    for L in c["layers"]:
        n += _pafolorn_layer_params(c, L)
        d = L["mixer"] if L["type"] == "channel_delta" else L["mixer"]["right"]
        chans = 2 * d["kv_heads"] * d["dim"] + d["heads"] * d["vdim"]
        extra += batch * 2 * 4 * (d["heads"] * d["vdim"] * d["dim"] + (d["conv"] - 1) * chans)
        if L["type"] == "parallel":
            a = L["mixer"]["left"]
            seen = min(ctx_mean, a["mask"]["size"] + a["mask"]["keep_first"])
            extra += batch * seen * a["kv_heads"] * (a["dim"] + a["vdim"]) * el
    return n * el + extra


def pafolorn_step_flops(c, seq_lens_new):
    """Matrix-product flops of a step (the parameters a token uses, twice), the attention's two products over the
    keys that each row sees, and the delta rule's seven operations a state entry and token."""
    n = sum(seq_lens_new)
    fl = 2 * len(seq_lens_new) * c["width"] * c["vocab"]
    for L in c["layers"]:
        fl += 2 * n * _pafolorn_layer_params(c, L)
        d = L["mixer"] if L["type"] == "channel_delta" else L["mixer"]["right"]
        fl += 7 * n * d["heads"] * d["vdim"] * d["dim"]
        if L["type"] == "parallel":
            a = L["mixer"]["left"]
            w, kf = a["mask"]["size"], a["mask"]["keep_first"]
            pairs = sum(sum(min(i + 1, w + min(kf, max(i + 1 - w, 0))) for i in range(t)) for t in seq_lens_new)
            fl += 2 * pairs * a["heads"] * (a["dim"] + a["vdim"])
    return fl


def pafolorn_compare(args):
    """Decode and prefill of Pafolorn beside Pedatar (the closest of the engine's models: a state per request beside
    attention, root-mean-square norms, short filters) at the layer sizes of GPT-2 124M and 355M; one JSON line."""
    import numpy as np
    el, dkey = 2, "bf16"
    out = {"metric": "decode tok/s at batch 8 of Pafolorn at GPT-2 124M layer sizes (beside Pedatar at the same sizes: see points)",
           "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey, "steps": args.steps, "warmup": args.warmup,
           "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", "points": {}, "points_frac": {}}
    for size in ("124m", "355m"):
        for design in ("pedatar", "pafolorn"):
            rng = np.random.default_rng(0)
            cfg = pedatar_config(size) if design == "pedatar" else pafolorn_config(size)
            nbytes = pedatar_step_bytes if design == "pedatar" else pafolorn_step_bytes
            model = engine_from_gpu_weights(cfg, "bfloat16", 64, kernels=args.kernels)
            key = f"{design}_{size}"
            for b in (1, 8, 64):
                steps = min(args.steps, 128)
                d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
                out["points"][f"{key}_decode_b{b}"] = round(b * steps / d, 1)
                out["points_frac"][f"{key}_decode_b{b}"] = round(nbytes(cfg, el, b, cm) / (d / steps) / 1e9 / HBM_GBS, 4)
            fl = pedatar_step_flops(cfg, [1024, 1024]) if design == "pedatar" else pafolorn_step_flops(cfg, [1024, 1024])
            pf = prefill_run(model, cfg, rng, dkey, flops=fl)
            out["points"][f"{key}_prefill_2048"] = pf["value"]
            out["points_frac"][f"{key}_prefill_2048"] = pf["frac"]
            if args.profile_stages:
                print(f"==== {key}", file=sys.stderr)
                kernel_table(model, cfg, rng, args.batch, args.prompt_len)
            del model
    out["value"] = out["points"]["pafolorn_124m_decode_b8"]
    out["config"] = {"model": "pafolorn beside pedatar at gpt2-124m and gpt2-355m layer sizes", "global_batch": 8,
                     "prompt_len": args.prompt_len,
                     "pafolorn": "a delta rule with a decay per key channel (GPT-2's heads, 64 key and value entries, 4 taps, low "
                                 "ranks width / 16 and width / 8) and a parallel mixer (attention beside a delta rule, half of "
                                 "GPT-2's heads each, window 512 keeping the first 4, cap 30, 32 rotated entries) in turn; "
                                 "feed-forwards of 4 x width", "parallelism": "single-gpu"}
    print(json.dumps(out))
    return 0


def salivik_config(name, n_positions=1024):
    """A Salivik of GPT-2 ``name``'s sizes: as many layer runs, with latent attention, attention whose keys are its values
    and retention in turn.  Latent attention as in ``pedatar_config`` (GPT-2's heads, 48 + 16 query entries, values of 64,
    a query latent of half the width, a latent of a quarter of the width beside a key piece of 16) with a window of 512
    keys, a learned sink and ramped speeds.  Attention: GPT-2's heads of 64 entries on a quarter as many key heads, the
    first 32 entries rotated, a window of 512.  Retention: GPT-2's heads with 64 key and 64 value entries.  Feed-forward:
    8 capped gated experts of 2/3 of the width (2 a token) and a shared one of 4/3 of the width, which hold what
    Pedatar's ungated ones hold for a token.  The first three layers run twice (a loop), so the stored layers are three
    fewer than the runs."""
    g = MODELS[name]
    E, H = g["n_embd"], g["n_head"]
    lat = {"heads": H, "dim": 48, "rot_dim": 16, "vdim": 64, "q_rank": E // 2, "kv_rank": E // 4, "scale": 64 ** -0.5,
           "mask": {"size": 512}, "rot": {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "original": 256, "fast": 32.0, "slow": 1.0}}}
    att = {"heads": H, "kv_heads": H // 4, "dim": 64, "vdim": 64, "scale": 64 ** -0.5, "mask": {"size": 512},
           "rot": {"base": 10000.0, "dims": 32}}
    ret = {"heads": H, "dim": 64, "vdim": 64, "decay": [1.0 - 0.3 * 2.0 ** (-(i % 8)) for i in range(H)], "rot": {"base": 10000.0, "dims": 64}}
    f, fs = (2 * E // 3) // 8 * 8, (4 * E // 3) // 8 * 8
    mlp = {"kind": "moe", "expert": {"ff": f, "limit": 7.0}, "router": {"experts": 8, "top": 2}, "shared": {"ff": fs, "limit": 7.0}}
    kinds = (("latent_attention", lat), ("attention", att), ("retention", ret))
    layers = [{"type": kinds[i % 3][0], "mixer": kinds[i % 3][1], "mlp": mlp} for i in range(g["n_layer"] - 3)]
    return {"architecture": "Salivik", "vocab": 50257, "width": E, "norm": {"eps": 1e-5}, "layers": layers,
            "loop": {"start": 0, "stop": 3, "times": 2}, "max_positions": n_positions,
            # what decode_run and prefill_run read
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": g["n_layer"], "n_embd": E}


def _salivik_runs(c):
    lp = c["loop"]
    order = list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"] + list(range(lp["stop"], len(c["layers"])))
    return [c["layers"][i] for i in order]


def _salivik_layer_params(c, L, experts_used):
    E, m = c["width"], L["mixer"]
    if L["type"] == "latent_attention":
        H, qd = m["heads"], m["dim"] + m["rot_dim"]
        n = E * (m["q_rank"] + m["kv_rank"] + m["rot_dim"]) + m["q_rank"] * H * qd + m["kv_rank"] * H * (m["dim"] + m["vdim"]) + H * m["vdim"] * E
    elif L["type"] == "attention":
        n = E * m["dim"] * (3 * m["heads"] + m["kv_heads"])
    else:
        n = E * m["heads"] * (2 * m["dim"] + 3 * m["vdim"])
    f = L["mlp"]
    return n + 3 * E * (experts_used * f["expert"]["ff"] + f["shared"]["ff"]) + f["router"]["experts"] * E


def salivik_step_bytes(c, el, batch, ctx_mean):
    """What a decode step must read: every matrix of every run once (of the experts as many as ``batch`` tokens can
    choose; a looped layer's matrices are read again in its second pass), the keys that the windows see, and the
    retention states (read and written, 32-bit)."""
    n, extra = c["vocab"] * c["width"] + 2 * c["width"] ** 2 * c["loop"]["times"], 0
    for L in _salivik_runs(c):
        f = L["mlp"]["router"]
        n += _salivik_layer_params(c, L, min(f["experts"], f["top"] * batch))
        m = L["mixer"]
        if L["type"] == "latent_attention":
            extra += batch * min(ctx_mean, m["mask"]["size"]) * (m["kv_rank"] + m["rot_dim"]) * el
        elif L["type"] == "attention":
            extra += batch * min(ctx_mean, m["mask"]["size"]) * m["kv_heads"] * 2 * m["dim"] * el
        else:
            extra += batch * 2 * 4 * m["heads"] * m["dim"] * m["vdim"]
    return n * el + extra


def salivik_step_flops(c, seq_lens_new):
    """Matrix-product flops of a step (the parameters a token uses, twice), the attentions' two products over the keys
    that each row sees, and the retention's four operations a state entry and token."""
    n = sum(seq_lens_new)
    fl = 2 * len(seq_lens_new) * c["width"] * c["vocab"] + 2 * n * 2 * c["width"] ** 2 * c["loop"]["times"]
    for L in _salivik_runs(c):
        fl += 2 * n * _salivik_layer_params(c, L, L["mlp"]["router"]["top"])
        m = L["mixer"]
        if L["type"] == "retention":
            fl += 4 * n * m["heads"] * m["dim"] * m["vdim"]
            continue
        pairs = sum(sum(min(i + 1, m["mask"]["size"]) for i in range(t)) for t in seq_lens_new)
        if L["type"] == "latent_attention":
            fl += 2 * pairs * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"])
        else:
            fl += 2 * pairs * m["heads"] * 2 * m["dim"]
    return fl


def salivik_compare(args):
    """Decode and prefill of Salivik beside Pedatar (the closest of the engine's models: latent attention, a mixer with a
    state per request, routed experts beside a shared one, root-mean-square norms) at the layer sizes of GPT-2 124M and
    355M; one JSON line."""
    import numpy as np
    el, dkey = 2, "bf16"
    out = {"metric": "decode tok/s at batch 8 of Salivik at GPT-2 124M layer sizes (beside Pedatar at the same sizes: see points)",
           "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey, "steps": args.steps, "warmup": args.warmup,
           "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", "points": {}, "points_frac": {}}
    for size in ("124m", "355m"):
        for design in ("pedatar", "salivik"):
            rng = np.random.default_rng(0)
            cfg = pedatar_config(size) if design == "pedatar" else salivik_config(size)
            nbytes = pedatar_step_bytes if design == "pedatar" else salivik_step_bytes
            model = engine_from_gpu_weights(cfg, "bfloat16", 64, kernels=args.kernels)
            key = f"{design}_{size}"
            for b in (1, 8, 64):
                steps = min(args.steps, 128)
                d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
                out["points"][f"{key}_decode_b{b}"] = round(b * steps / d, 1)
                out["points_frac"][f"{key}_decode_b{b}"] = round(nbytes(cfg, el, b, cm) / (d / steps) / 1e9 / HBM_GBS, 4)
            fl = pedatar_step_flops(cfg, [1024, 1024]) if design == "pedatar" else salivik_step_flops(cfg, [1024, 1024])
            pf = prefill_run(model, cfg, rng, dkey, flops=fl)
            out["points"][f"{key}_prefill_2048"] = pf["value"]
            out["points_frac"][f"{key}_prefill_2048"] = pf["frac"]
            if args.profile_stages:
                print(f"==== {key}", file=sys.stderr)
                kernel_table(model, cfg, rng, args.batch, args.prompt_len)
            del model
    out["value"] = out["points"]["salivik_124m_decode_b8"]
    out["config"] = {"model": "salivik beside pedatar at gpt2-124m and gpt2-355m layer sizes", "global_batch": 8,
                     "prompt_len": args.prompt_len,
                     "salivik": "latent attention (as Pedatar's, with a window of 512, a sink and ramped speeds), attention "
                                "whose keys are its values (GPT-2's heads on a quarter as many key heads, window 512, sink, "
                                "output gate) and retention (GPT-2's heads, 64 x 64 states) in turn; 8 capped gated experts of "
                                "2/3 width (2 a token) beside a shared one of 4/3 width; the first three layers run twice",
                     "parallelism": "single-gpu"}
    print(json.dumps(out))
    return 0


def design_compare(args):
    """Decode and prefill of another design beside its like at equal sizes; one JSON line."""
    if args.design == "pedatar":
        return pedatar_compare(args)
    if args.design == "pafolorn":
        return pafolorn_compare(args)
    if args.design == "salivik":
        return salivik_compare(args)
    return virudra_compare(args)


def pedatar_compare(args):
    """Decode and prefill of Pedatar beside Virudra (the closest of the engine's models: root-mean-square norms, no
    position table, mixtures of experts) at the layer sizes of GPT-2 124M and 355M; one JSON line."""
    import numpy as np
    el, dkey = 2, "bf16"
    out = {"metric": "decode tok/s at batch 8 of Pedatar at GPT-2 124M layer sizes (beside Virudra at the same sizes: see points)",
           "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey, "steps": args.steps, "warmup": args.warmup,
           "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", "points": {}, "points_frac": {}}
    for size in ("124m", "355m"):
        for design in ("virudra", "pedatar"):
            rng = np.random.default_rng(0)
            cfg = virudra_config(size) if design == "virudra" else pedatar_config(size)
            model = engine_from_gpu_weights(cfg, "bfloat16", 64, kernels=args.kernels)
            key = f"{design}_{size}"
            for b in (1, 8, 64):
                steps = min(args.steps, 128)
                d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
                out["points"][f"{key}_decode_b{b}"] = round(b * steps / d, 1)
                if design == "virudra":
                    nb = virudra_weight_bytes(cfg, el, b) + b * cm * 2 * cfg["n_embd"] * el * cfg["n_layer"]
                else:
                    nb = pedatar_step_bytes(cfg, el, b, cm)
                out["points_frac"][f"{key}_decode_b{b}"] = round(nb / (d / steps) / 1e9 / HBM_GBS, 4)
            fl = virudra_step_flops(cfg, [1024, 1024]) if design == "virudra" else pedatar_step_flops(cfg, [1024, 1024])
            pf = prefill_run(model, cfg, rng, dkey, flops=fl)
            out["points"][f"{key}_prefill_2048"] = pf["value"]
            out["points_frac"][f"{key}_prefill_2048"] = pf["frac"]
            if args.profile_stages:
                print(f"==== {key}", file=sys.stderr)
                kernel_table(model, cfg, rng, args.batch, args.prompt_len)
            del model
    out["value"] = out["points"]["pedatar_124m_decode_b8"]
    out["config"] = {"model": "pedatar beside virudra at gpt2-124m and gpt2-355m layer sizes", "global_batch": 8,
                     "prompt_len": args.prompt_len,
                     "pedatar": "latent attention (48 + 16 query entries a head, values 64, query latent width / 2, latent width / 4 "
                                "+ key piece 16) and scans (2 x width channels, 16 state entries, 4 taps) in turn; 8 experts of the "
                                "width's size (2 a token) beside a shared one of twice the width", "parallelism": "single-gpu"}
    print(json.dumps(out))
    return 0


def virudra_compare(args):
    """Decode and prefill of Virudra beside GPT-2 at equal sizes; one JSON line."""
    import numpy as np
    el, dkey = 2, "bf16"
    out = {"metric": "decode tok/s at batch 8 of Virudra at GPT-2 124M layer sizes (beside GPT-2 itself: see points)",
           "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey, "steps": args.steps, "warmup": args.warmup,
           "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", "points": {}, "points_frac": {}}
    for size in ("124m", "355m"):
        for design in ("gpt2", "virudra"):
            rng = np.random.default_rng(0)
            cfg = model_config(size) if design == "gpt2" else virudra_config(size)
            model = engine_from_gpu_weights(cfg, "bfloat16", 64, kernels=args.kernels)
            key = f"{design}_{size}"
            for b in (1, 8, 64):
                steps = min(args.steps, 128)
                d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
                out["points"][f"{key}_decode_b{b}"] = round(b * steps / d, 1)
                wb = weight_bytes(cfg, el) if design == "gpt2" else virudra_weight_bytes(cfg, el, b)
                kv = 2 * cfg["n_embd"] * el * cfg["n_layer"]
                out["points_frac"][f"{key}_decode_b{b}"] = round((wb + b * cm * kv) / (d / steps) / 1e9 / HBM_GBS, 4)
            pf = prefill_run(model, cfg, rng, dkey, flops=None if design == "gpt2" else virudra_step_flops(cfg, [1024, 1024]))
            out["points"][f"{key}_prefill_2048"] = pf["value"]
            out["points_frac"][f"{key}_prefill_2048"] = pf["frac"]
            if args.profile_stages:
                print(f"==== {key}", file=sys.stderr)
                kernel_table(model, cfg, rng, args.batch, args.prompt_len)
            del model
    out["value"] = out["points"]["virudra_124m_decode_b8"]
    out["config"] = {"model": "virudra at gpt2-124m and gpt2-355m layer sizes", "global_batch": 8, "prompt_len": args.prompt_len,
                     "virudra": "heads = key heads, head size 64, gated feed-forward of 8/3 width and 8 experts (2 a token) of "
                                "half that in turn, bias rows 32 up to distance 512, temperature every 256", "parallelism": "single-gpu"}
    print(json.dumps(out))
    return 0


def decode_run(model, cfg, rng, batch, prompt_len, steps, warmup):
    """Prefill ``batch`` prompts and settle (untimed), ``warmup`` decode steps, then time ``steps`` decode
    steps.  The requests outlive the timed steps, so that none of them ends (and no smaller batch has its
    graph recorded) inside the timed region.  Returns (seconds, mean context length in the timed steps)."""
    import torch
    from deliverance_amd import GeneratorParameters
    # (requests admitted first decode while the others' prompts are still processed: one token a prefill step)
    stagger = -(-batch * prompt_len // model.engine_config.max_batch_tokens)
    total = stagger + SETTLE_STEPS + warmup + steps + 8
    assert prompt_len + total + 1 <= cfg["n_positions"], "prompt and decoded tokens exceed n_positions"
    params = GeneratorParameters(max_tokens=total, ignore_eos=True)
    rids = [model.add_request([int(t) for t in rng.integers(0, cfg["vocab_size"], size=prompt_len)], params)
            for _ in range(batch)]
    while any(r.n_computed < len(r.prompt) for r in model.scheduler.running) or model.scheduler.waiting:
        model.step()
    for _ in range(SETTLE_STEPS + warmup):
        model.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        model.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(model.scheduler.running) == batch, "a request ended inside the timed steps"
    ctx_mean = prompt_len + 1 + stagger / 2.0 + SETTLE_STEPS + warmup + steps / 2.0
    for rid in rids:
        model.cancel(rid)
    while model.has_work():
        model.step()
    model.drain()
    model.scheduler.finished.clear()
    return dt, ctx_mean


def prefill_run(model, cfg, rng, dkey, n_prompts=2, length=1024, flops=None):
    """``n_prompts`` x ``length``-token prompts (2 x 1,024 unless asked otherwise) in ONE step of the engine's step
    function, logits at the last row of each."""
    import torch
    from deliverance_amd.engine.step import StepEntry
    times = []
    for it in range(5):                       # the first rounds warm up; the best of the rest counts
        entries = [StepEntry(f"prefill{i}", [int(t) for t in rng.integers(0, cfg["vocab_size"], size=length)], [length - 1])
                   for i in range(n_prompts)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.runner.run(entries)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        for e in entries:
            model.cache.manager.close(e.rid)
    t = min(times[2:])
    fl = flops if flops is not None else step_flops(cfg, [length] * n_prompts)
    n = n_prompts * length
    return {"value": round(n / t, 1), "tokens": n, "ms": round(t * 1e3, 3), "frac": round(fl / t / PEAK_FLOPS[dkey], 4)}


def mixed_run(model, cfg, rng, n_req=64, new=128):
    """Continuous batching under load: every request arrives at once; the scheduler admits them as
    seats and pages allow, cuts prompts into portions of at most 512 tokens and runs them in the
    same steps as the other requests' decoding.  Run twice (the first run records the decode
    graphs): the two runs must generate the same tokens.  Returns a dict of what was measured."""
    import torch
    from deliverance_amd import GeneratorParameters
    longest = cfg["n_positions"] - new - 1
    lengths = [int(x) for x in rng.integers(16, longest + 1, size=n_req)]
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]
    params = GeneratorParameters(max_tokens=new, ignore_eos=True)
    best, tokens = None, []
    for _ in range(2):
        before = model.stats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = model.generate(prompts, params)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens.append([o.generated_tokens for o in outs])
        if best is None or dt < best:
            best = dt
            after = model.stats()
            steps = after["steps"] - before["steps"]
            batch_tokens = after["batch_tokens"] - before["batch_tokens"]
    assert all(len(t) == new for t in tokens[0])
    same = sum(a == b for a, b in zip(*tokens))
    return dict(value=round(n_req * new / best, 1), seconds=round(best, 4), prompt_tokens=sum(lengths),
                generated_tokens=n_req * new, all_tokens_per_second=round((sum(lengths) + n_req * new) / best, 1),
                steps=steps, mean_batch_tokens=round(batch_tokens / max(steps, 1), 1), longest_prompt=longest,
                requests_equal_in_both_runs=same, requests=n_req, preemptions=model.stats().get("preemptions", 0))


def kernel_table(model, cfg, rng, batch, prompt_len, n_prompts=2, length=1024):
    """--profile-stages: every kernel of a prefill step and of a few decode steps timed on the device,
    against the bytes it must move and the flops it must do (stderr)."""
    from deliverance_amd.profiler import KernelProfiler
    KernelProfiler.enable()
    prefill_run(model, cfg, rng, "bf16", n_prompts, length)
    print(KernelProfiler.summary(f"prefill, {n_prompts} x {length:,} tokens, 5 steps (% of 8 TB/s or of the matrix peak, whichever binds)"),
          file=sys.stderr)
    KernelProfiler.reset()
    decode_run(model, cfg, rng, batch, prompt_len, 16, 0)
    print(KernelProfiler.summary(f"prefill of {batch} x {prompt_len} tokens, then {SETTLE_STEPS + 16} decode steps at batch {batch}"),
          file=sys.stderr)
    KernelProfiler.disable()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="124m", choices=sorted(MODELS))
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--n-positions", type=int, default=1024, help="context length of the random model (GPT-2: 1,024)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--kernels", default="tuned", choices=["tuned", "reference"])
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the GPT-2 1.5B points and the 355M mixed workload")
    ap.add_argument("--profile-stages", action="store_true", help="also print a per-kernel table with roofline fractions (stderr)")
    ap.add_argument("--page-size", type=int, default=16, choices=[16, 32, 64], help="tokens a cache page")
    ap.add_argument("--prefill-shape", default="2x1024", help="prompts x tokens of the prefill step (the contract's: 2x1024)")
    ap.add_argument("--step-tokens", type=int, default=512 + 64,
                    help="mixed workload: the most tokens a step holds, decoded tokens and a prompt portion together (default: a portion of 512 beside 64 decoded tokens)")
    ap.add_argument("--pool-tokens", type=int, default=None,
                    help="mixed workload: tokens of cache the pool holds (default: every request at full length; fewer force "
                         "requests out of the cache and back, which the line reports as preemptions)")
    ap.add_argument("--design", default="gpt2", choices=["gpt2", "virudra", "pedatar", "pafolorn", "salivik"],
                    help="virudra: that design beside GPT-2 at equal sizes (decode at batch 1, 8, 64 and the prefill of 2,048 "
                         "tokens, at 124M and 355M layer sizes) instead of the default workload; pedatar: that design beside "
                         "Virudra, likewise; pafolorn: that design beside Pedatar, likewise; "
                         "salivik: that design beside Pedatar, likewise")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="mixed: only the mixed workload, on --model (64 requests with prompts of 16 to 895 tokens arrive at "
                         "once, prompt portions of 512 tokens run beside the decoding of the others, 128 new tokens each)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import numpy as np
    from deliverance_amd.random_model import random_model

    if args.design in ("virudra", "pedatar", "pafolorn", "salivik"):
        return design_compare(args)
    cfg = model_config(args.model, args.layers, args.n_positions)
    full_layers = MODELS[args.model]["n_layer"]
    el = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = np.random.default_rng(0)
    pf_n, pf_len = (int(x) for x in args.prefill_shape.lower().split("x"))
    if not args.no_prefill and args.workload == "decode" and pf_len > cfg["n_positions"]:
        print(f"a prompt of {pf_len} tokens exceeds n_positions {cfg['n_positions']}")
        return 2
    if args.prompt_len + SETTLE_STEPS + args.warmup + args.steps + 9 > cfg["n_positions"]:
        print(f"prompt {args.prompt_len} + {SETTLE_STEPS + args.warmup + args.steps + 9} decoded tokens exceed n_positions {cfg['n_positions']}")
        return 2

    if args.workload == "mixed":
        model = engine_from_gpu_weights(cfg, args.dtype, 64, kernels=args.kernels, max_batch_tokens=args.step_tokens, max_chunk=512, page_size=args.page_size,
                                        **({"max_cached_tokens": args.pool_tokens} if args.pool_tokens else {}))
        m = mixed_run(model, cfg, rng)
        print(json.dumps({
            "metric": "generated tok/s, %d requests at once (GPT-2 %s layer sizes, prompts 16..%d, 128 new tokens each, "
                      "prompt portions of 512 beside decoding)" % (m["requests"], args.model, m["longest_prompt"]),
            "value": m["value"], "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey,
            "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", **{k: m[k] for k in (
                "seconds", "prompt_tokens", "generated_tokens", "all_tokens_per_second", "requests_equal_in_both_runs")},
            "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_embd": cfg["n_embd"],
                       "n_head": cfg["n_head"], "requests": m["requests"], "max_chunk": 512, "step_tokens": args.step_tokens, "page_size": args.page_size,
                       "steps": m["steps"], "mean_batch_tokens": m["mean_batch_tokens"], "preemptions": m["preemptions"],
                       "pool_tokens": model.engine_config.max_cached_tokens}}))
        return 0

    with tempfile.TemporaryDirectory() as folder:
        random_model(folder, cfg, seed=0)
        model = engine_from_folder(folder, args.dtype, max(args.batch, 64 if not args.no_points else args.batch), cfg,
                                   kernels=args.kernels, max_batch_tokens=max(2048, args.batch, pf_n * pf_len), page_size=args.page_size)
    dt, ctx_mean = decode_run(model, cfg, rng, args.batch, args.prompt_len, args.steps, args.warmup)
    achieved = decode_roofline(cfg, el, args.batch, ctx_mean, dt / args.steps)
    out = {
        "metric": "decode tok/s (GPT-2 %s layer sizes, batch %d, %d-token prompts)" % (args.model, args.batch, args.prompt_len),
        "value": round(args.batch * args.steps / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic (random weights, uniform-random token ids)",
        "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_layer_full": full_layers,
                   "n_embd": cfg["n_embd"], "n_head": cfg["n_head"], "n_inner": 4 * cfg["n_embd"],
                   "vocab_size": cfg["vocab_size"], "n_positions": cfg["n_positions"],
                   "global_batch": args.batch, "seq_len": int(round(ctx_mean)),
                   "prompt_len": args.prompt_len, "page_size": args.page_size, "kernels": args.kernels, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
    }
    points, fracs = {}, {}
    if not args.no_points:
        for b in (1, 64):
            steps = min(args.steps, 128)
            d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            fracs[f"decode_b{b}"] = round(decode_roofline(cfg, el, b, cm, d / steps) / HBM_GBS, 4)
    if not args.no_prefill:
        out["prefill"] = prefill_run(model, cfg, rng, dkey, pf_n, pf_len)
    if args.profile_stages:
        kernel_table(model, cfg, rng, args.batch, args.prompt_len, pf_n, pf_len)
    del model

    if not args.no_extra and args.dtype == "bfloat16":
        # GPT-2 1.5B layer sizes, all 48 layers: decode at batch 1, 8 and 64 and the prefill of 2,048 tokens
        big = model_config("1.5b")
        model = engine_from_gpu_weights(big, args.dtype, 64, kernels=args.kernels)
        for b in (1, 8, 64):
            steps = min(args.steps, 64)
            d, cm = decode_run(model, big, rng, b, args.prompt_len, steps, 4)
            points[f"gpt2_1p5b_decode_b{b}"] = round(b * steps / d, 1)
            fracs[f"gpt2_1p5b_decode_b{b}"] = round(decode_roofline(big, el, b, cm, d / steps) / HBM_GBS, 4)
        pf = prefill_run(model, big, rng, dkey)
        points["gpt2_1p5b_prefill_2048"] = pf["value"]
        fracs["gpt2_1p5b_prefill_2048"] = pf["frac"]
        del model
        # GPT-2 355M layer sizes: the mixed workload
        mid = model_config("355m")
        model = engine_from_gpu_weights(mid, args.dtype, 64, kernels=args.kernels, max_batch_tokens=512 + 64, max_chunk=512)
        m = mixed_run(model, mid, rng)
        points["gpt2_355m_mixed_generated"] = m["value"]
        points["gpt2_355m_mixed_all_tokens"] = m["all_tokens_per_second"]
        points["gpt2_355m_mixed_requests_equal_in_both_runs"] = m["requests_equal_in_both_runs"]
        fracs["gpt2_355m_mixed_flops"] = round(
            (2 * (m["prompt_tokens"] + m["generated_tokens"]) * (weight_bytes(mid, 1) - mid["vocab_size"] * mid["n_embd"])
             + 2 * m["generated_tokens"] * mid["vocab_size"] * mid["n_embd"]) / m["seconds"] / PEAK_FLOPS[dkey], 4)
        out["config"]["points_gpt2_1p5b"] = "n_layer 48 of 48, n_embd 1600, n_head 25, n_inner 6400, decode after 512-token prompts"
        out["config"]["points_gpt2_355m_mixed"] = ("n_layer 24 of 24, n_embd 1024, n_head 16: %d requests at once, prompts 16..%d, "
                                                   "128 new tokens each, portions of 512 beside decoding, %d steps"
                                                   % (m["requests"], m["longest_prompt"], m["steps"]))
        del model
    if points:
        out["points"] = points
        out["points_frac"] = fracs          # decode: of 8 TB/s; prefill and mixed: of the matrix peak
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
