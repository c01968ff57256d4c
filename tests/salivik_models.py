"""Small Salivik configurations for the tests, each different in every size and option, and a model folder with
random weights beside its plain implementation."""
from __future__ import annotations

import functools

import numpy as np

import plain_salivik as P


def rot(base, dims, scaling=None):
    d = {"base": base, "dims": dims}
    if scaling is not None:
        d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return d


def att(heads, kv_heads, dim, scale, window, base, dims):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                                           "mask": {"size": window}, "rot": rot(base, dims)}}


def ret(heads, dim, vdim, decay, base, dims):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": rot(base, dims)}}


def lat(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window, base, scaling=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale, "mask": {"size": window}, "rot": rot(base, rot_dim, scaling)}}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def config(vocab, width, eps, layers, loop=None):
    d = {"architecture": "Salivik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


# S: sizes that the matrix-core kernels take; every mixer once; the middle two layers run three times; windows of 24
# and 40 keys, shorter than the prompts
CONFIG_S = config(300, 64, 1e-5,
                  [layer(ret(2, 16, 24, (0.9, 1.0), 10000.0, 16), dense(96, 2.0)),
                   layer(lat(2, 16, 8, 24, 24, 40, 0.2, 24, 10000.0, (4.0, 64, 8.0, 1.0)), moe(4, 2, 32, 1.25, (48, 2.0))),
                   layer(att(4, 2, 16, 0.25, 40, 10000.0, 8), moe(4, 2, 32, 1.25, (48, 2.0))),
                   layer(ret(1, 32, 16, (0.75,), 500.0, 8), None)],
                  loop=(1, 3, 3))

# T: no loop at all; sizes that are no multiple of 8 (plain products and plain attention kernels); one key head for
# all query heads; every expert used by every token; no shared expert; windows longer than any prompt; values larger
# than keys in the latent layer; a fast decay beside slow ones
CONFIG_T = config(130, 72, 1e-6,
                  [layer(att(3, 1, 12, 0.3, 500, 500.0, 6), moe(3, 3, 20, 0.7)),
                   layer(ret(3, 20, 12, (0.5, 0.9, 0.999), 100.0, 20), dense(40, 0.5)),
                   layer(lat(3, 8, 12, 20, 18, 27, 0.3, 300, 500.0), None)])

# U: the ones: one head, one expert, a loop of one layer that runs once and one that starts at the first layer; as
# many key heads as query heads; nothing turns in the attention layer; a scaling factor of 1 (nothing changes); a
# window of one key (a token sees itself only) and of two
CONFIG_U = config(64, 48, 1e-5,
                  [layer(lat(1, 16, 16, 16, 16, 16, 0.25, 2, 100.0, (1.0, 32, 4.0, 2.0)), moe(1, 1, 40, 3.0)),
                   layer(att(2, 2, 24, 0.2, 1, 10000.0, 0), moe(6, 2, 16, 1.0, (64, 0.4))),
                   layer(ret(4, 8, 8, (1.0, 0.5, 0.25, 0.9375), 10000.0, 4), dense(24, 1.0))],
                  loop=(0, 1, 1))


class TinySalivik:
    def __init__(self, folder, cfg, seed):
        self.folder, self.cfg, self.seed = str(folder), cfg, seed
        self.plain_cfg, self.W = P.read_model_folder(self.folder)

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids):
        return P.forward_logits(self.plain_cfg, self.W, list(ids))

    def plain_logits(self, ids, routes=None, slack=0.0):
        """The plain model's logits [T, V]; with ``routes`` (run -> position -> experts chosen by the engine) it makes
        the engine's choices where they are as good as its own within ``slack`` (plain_salivik.routed_ff)."""
        if routes is None:
            return self._logits(tuple(int(i) for i in ids))
        return P.forward(self.plain_cfg, self.W, list(ids), routes=routes, slack=slack)

    def prompt(self, length, salt=0):
        rng = np.random.default_rng(1000 * self.seed + 7 * length + salt)
        return [int(t) for t in rng.integers(0, self.cfg["vocab"], size=length)]


def make_model(folder, cfg, seed):
    from deliverance_amd.random_model import random_model
    random_model(str(folder), cfg, seed)
    return TinySalivik(folder, cfg, seed)


def moe_runs(cfg):
    """The runs (indices into the run order) that have a routed feed-forward, in order."""
    return [run for run, (i, _) in enumerate(P.run_order(cfg))
            if (cfg["layers"][i].get("mlp") or {}).get("kind") == "moe"]


def replay_routed(session, steps, cfg):
    """helpers.replay, and beside the logits the experts that the engine chose: {rid: {run: {position: [experts]}}}.
    The engine hands them to its layer debug hook once per run of a layer with a routed feed-forward, rows in the
    step's order (one-token entries first, then the portions, each group in the order of the entries)."""
    got, routes, at = {}, {}, {}
    seen = []
    session.runner.debug_hook = lambda layer, stage, tensor: seen.append(tensor.cpu().numpy()) if stage == "expert_choice" else None
    runs = moe_runs(cfg)
    try:
        for s in steps:
            seen.clear()
            out = session.run_step(s)
            r = 0
            for e in s["entries"]:
                for _ in e.get("want", []):
                    got.setdefault(e["id"], []).append(out[r])
                    r += 1
            order = sorted(range(len(s["entries"])), key=lambda i: (len(s["entries"][i]["tokens"]) != 1, i))
            assert len(seen) == len(runs), f"{len(seen)} routed feed-forwards reported, the model runs {len(runs)}"
            row = 0
            for i in order:
                e = s["entries"][i]
                start = at.get(e["id"], 0)
                for k, ids in enumerate(seen):
                    for j in range(len(e["tokens"])):
                        routes.setdefault(e["id"], {}).setdefault(runs[k], {})[start + j] = [int(x) for x in ids[row + j]]
                row += len(e["tokens"])
                at[e["id"]] = start + len(e["tokens"])
            for rid in s["end"]:
                at.pop(rid, None)
    finally:
        session.runner.debug_hook = None
    return {rid: np.stack(rows) for rid, rows in got.items()}, routes
