"""Small Pafolorn configurations for the tests, each different in every size and option, and a model folder with
random weights beside its plain implementation."""
from __future__ import annotations

import functools

import numpy as np

import plain_pafolorn as P


def delta(heads, kv_heads, dim, vdim, conv, a_rank=None, g_rank=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    if a_rank is not None:
        d["a_rank"], d["g_rank"] = a_rank, g_rank
    return d


def attention(heads, kv_heads, dim, vdim, scale, window, keep_first, base, dims, softcap=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "mask": {"size": window, "keep_first": keep_first}, "rot": {"base": base, "dims": dims}}
    if softcap is not None:
        d["softcap"] = softcap
    return d


def channel_layer(mixer, ff=None):
    return {"type": "channel_delta", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def parallel_layer(left, right, left_scale, right_scale, ff=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# F: a parallel layer first; head sizes that the matrix cores take; grouped key heads in both mixers; a window of 24
# that keeps 5 first tokens; half of every head turned; a cap on the scores
CONFIG_F = {"architecture": "Pafolorn", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 0.7,
            "layers": [parallel_layer(attention(4, 2, 32, 16, 0.18, 24, 5, 10000.0, 16, softcap=30.0),
                                      delta(4, 2, 16, 32, 4), 1.3, 0.8, ff=96),
                       channel_layer(delta(2, 2, 32, 16, 3, a_rank=8, g_rank=12)),
                       parallel_layer(attention(4, 2, 32, 16, 0.18, 24, 5, 10000.0, 16, softcap=30.0),
                                      delta(4, 2, 16, 32, 4), 1.3, 0.8, ff=96)]}

# G: sizes that are no multiple of 8 or 16 (plain products, partly filled lanes); a window that keeps nothing; every
# entry turned; no cap; two taps; one key head for three value heads; a feed-forward behind the channel-wise layer
CONFIG_G = {"architecture": "Pafolorn", "vocab": 130, "width": 72, "norm": {"eps": 1e-6}, "logit_scale": 1.0,
            "layers": [channel_layer(delta(3, 1, 20, 12, 2, a_rank=5, g_rank=3), ff=50),
                       parallel_layer(attention(3, 1, 12, 20, 0.3, 17, 0, 500.0, 12),
                                      delta(3, 3, 24, 40, 2), 0.5, 2.0),
                       parallel_layer(attention(2, 2, 24, 8, 0.2, 33, 40, 250000.0, 6, softcap=5.0),
                                      delta(1, 1, 72, 24, 5), 1.0, 1.0, ff=30)]}

# H: the ones: one head, one tap (no filter state), ranks of one, a window of one token beside three kept first tokens,
# nothing turned, kept first tokens beyond the window's reach, scales of one
CONFIG_H = {"architecture": "Pafolorn", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 2.5,
            "layers": [parallel_layer(attention(1, 1, 16, 16, 0.25, 1, 3, 100.0, 0), delta(1, 1, 16, 16, 1), 1.0, 1.0, ff=40),
                       channel_layer(delta(1, 1, 8, 48, 1, a_rank=1, g_rank=1)),
                       parallel_layer(attention(6, 3, 8, 8, 0.4, 9, 2, 10000.0, 8, softcap=50.0),
                                      delta(6, 2, 8, 8, 4), 0.9, 1.2)]}


class TinyPafolorn:
    def __init__(self, folder, cfg, seed):
        self.folder, self.cfg, self.seed = str(folder), cfg, seed
        self.plain_cfg, self.W = P.read_model_folder(self.folder)

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids):
        return P.forward_logits(self.plain_cfg, self.W, list(ids))

    def plain_logits(self, ids):
        return self._logits(tuple(int(i) for i in ids))

    def prompt(self, length, salt=0):
        rng = np.random.default_rng(1000 * self.seed + 7 * length + salt)
        return [int(t) for t in rng.integers(0, self.cfg["vocab"], size=length)]


def make_model(folder, cfg, seed):
    from deliverance_amd.random_model import random_model
    random_model(str(folder), cfg, seed)
    return TinyPafolorn(folder, cfg, seed)
