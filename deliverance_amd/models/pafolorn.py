"""Pafolorn: which checkpoint tensors feed which part.

Names: ``embed``, ``embed.norm``, ``final.norm``; per layer ``l<i>.norm1``, ``l<i>.ls1`` and, with a feed-forward,
``l<i>.norm2``, ``l<i>.ls2``, ``l<i>.mlp.{up, down}``.  A delta-rule mixer under ``<m>`` = ``l<i>.mix`` (alone) or
``l<i>.mix.right`` (beside attention): ``<m>.{q, k, v, b, o}``, the filters ``<m>.{q, k, v}.conv`` [channels, taps],
``<m>.A_log``, ``<m>.dt_bias``, ``<m>.norm``, and either ``<m>.a`` and ``<m>.g`` (decay a head) or the low-rank pairs
``<m>.{a1, a2}`` and ``<m>.{g1, g2}`` (decay a channel).  Attention under ``l<i>.mix.left``: ``{q, k, v, o}`` and the
gains ``{q, k}.norm``.  Linear weights are stored [out, in].  The head is the embedding table.
"""
from __future__ import annotations

from typing import List

from ..config.pafolorn import ARCHITECTURE, PafolornConfig
from ..config.specs import AttentionSpec, DeltaRuleSpec, ModelConfig, ParallelMixerSpec
from ..registry import Architecture, ModelSupport
from ..weights.loader import TensorDecl

# Random-weights distributions: matrices N(0, 0.05) (low-rank second factors N(0, 0.2)), gains 1 + N(0, 0.1), layer
# scales N(0.5, 0.1), filter taps N(0, 0.4), A_log N(0, 0.5), step biases N(0, 0.5).
W_STD, GAIN_STD = 0.05, 0.1


def read_config(d: dict) -> ModelConfig:
    return PafolornConfig.from_dict(d).to_model_config()


def _delta_decls(p: str, m: DeltaRuleSpec, E: int) -> List[TensorDecl]:
    H, G, D, Dv, K = m.n_heads, m.n_kv_heads, m.head_dim, m.v_head_dim, m.conv_taps
    decay_cols = H * D if m.decay == "channel" else H
    out = [TensorDecl(p + "q", (G * D, E), "normal", W_STD), TensorDecl(p + "q.conv", (G * D, K), "normal", 0.4),
           TensorDecl(p + "k", (G * D, E), "normal", W_STD), TensorDecl(p + "k.conv", (G * D, K), "normal", 0.4),
           TensorDecl(p + "v", (H * Dv, E), "normal", W_STD), TensorDecl(p + "v.conv", (H * Dv, K), "normal", 0.4),
           TensorDecl(p + "b", (H, E), "normal", W_STD), TensorDecl(p + "A_log", (H,), "normal", 0.5),
           TensorDecl(p + "norm", (Dv,), "ones_plus_normal", GAIN_STD),
           TensorDecl(p + "dt_bias", (decay_cols,), "normal", 0.5)]
    if m.decay_rank:
        out += [TensorDecl(p + "a1", (m.decay_rank, E), "normal", W_STD),
                TensorDecl(p + "a2", (decay_cols, m.decay_rank), "normal", 4 * W_STD)]
    else:
        out.append(TensorDecl(p + "a", (decay_cols, E), "normal", W_STD))
    if m.gate_rank:
        out += [TensorDecl(p + "g1", (m.gate_rank, E), "normal", W_STD),
                TensorDecl(p + "g2", (H * Dv, m.gate_rank), "normal", 4 * W_STD)]
    else:
        out.append(TensorDecl(p + "g", (H * Dv, E), "normal", W_STD))
    out.append(TensorDecl(p + "o", (E, H * Dv), "normal", W_STD))
    return out


def _attention_decls(p: str, m: AttentionSpec, E: int) -> List[TensorDecl]:
    H, G, D, Dv = m.n_heads, m.n_kv_heads, m.head_dim, m.value_dim
    return [TensorDecl(p + "q", (H * D, E), "normal", W_STD), TensorDecl(p + "k", (G * D, E), "normal", W_STD),
            TensorDecl(p + "v", (G * Dv, E), "normal", W_STD),
            TensorDecl(p + "q.norm", (H * D,), "ones_plus_normal", GAIN_STD),
            TensorDecl(p + "k.norm", (G * D,), "ones_plus_normal", GAIN_STD),
            TensorDecl(p + "o", (E, H * Dv), "normal", W_STD)]


def declare_tensors(mc: ModelConfig) -> List[TensorDecl]:
    E, V = mc.width, mc.vocab_size
    out = [TensorDecl("embed", (V, E), "normal", 0.3), TensorDecl("embed.norm", (E,), "ones_plus_normal", GAIN_STD)]
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        out.append(TensorDecl(p + "norm1", (E,), "ones_plus_normal", GAIN_STD))
        if isinstance(m, DeltaRuleSpec):
            out += _delta_decls(p + "mix.", m, E)
        elif isinstance(m, ParallelMixerSpec):
            out += _attention_decls(p + "mix.left.", m.branches[0], E) + _delta_decls(p + "mix.right.", m.branches[1], E)
        else:
            raise TypeError(f"no tensors are known for a mixer of kind {getattr(m, 'kind', m)!r}")
        out.append(TensorDecl(p + "ls1", (E,), "ones_plus_normal", GAIN_STD))
        if f is not None:
            out += [TensorDecl(p + "norm2", (E,), "ones_plus_normal", GAIN_STD),
                    TensorDecl(p + "mlp.up", (f.inner, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mlp.down", (E, f.inner), "normal", 2 * W_STD),
                    TensorDecl(p + "ls2", (E,), "ones_plus_normal", GAIN_STD)]
    out.append(TensorDecl("final.norm", (E,), "ones_plus_normal", GAIN_STD))
    return out


def _bind_delta(t: dict, p: str, m: DeltaRuleSpec) -> dict:
    d = {"q_weight": t[p + "q"], "k_weight": t[p + "k"], "v_weight": t[p + "v"], "q_conv": t[p + "q.conv"],
         "k_conv": t[p + "k.conv"], "v_conv": t[p + "v.conv"], "beta_weight": t[p + "b"], "a_log": t[p + "A_log"],
         "out_norm": t[p + "norm"], "dt_bias": t[p + "dt_bias"], "out_weight": t[p + "o"]}
    if m.decay_rank:
        d["decay_down"], d["decay_up"] = t[p + "a1"], t[p + "a2"]
    else:
        d["decay_weight"] = t[p + "a"]
    if m.gate_rank:
        d["gate_down"], d["gate_up"] = t[p + "g1"], t[p + "g2"]
    else:
        d["gate_weight"] = t[p + "g"]
    return d


def _bind_attention(t: dict, p: str) -> dict:
    import torch
    return {"qkv_weight": torch.cat([t[p + "q"], t[p + "k"], t[p + "v"]], 0), "out_weight": t[p + "o"],
            "q_norm": t[p + "q.norm"], "k_norm": t[p + "k.norm"]}


def bind_tensors(mc: ModelConfig, t: dict) -> dict:
    layers = []
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        d = {"post_mixer_norm": {"weight": t[p + "norm1"]}, "mixer_scale": t[p + "ls1"]}
        if isinstance(m, DeltaRuleSpec):
            d["mixer"] = _bind_delta(t, p + "mix.", m)
        else:
            d["mixer"] = {"branches": [_bind_attention(t, p + "mix.left."), _bind_delta(t, p + "mix.right.", m.branches[1])]}
        if f is not None:
            d["post_ff_norm"] = {"weight": t[p + "norm2"]}
            d["ff_scale"] = t[p + "ls2"]
            d["feed_forward"] = {"fc_weight": t[p + "mlp.up"], "proj_weight": t[p + "mlp.down"]}
        layers.append(d)
    return {"embed": {"tokens": t["embed"]}, "embed_norm": {"weight": t["embed.norm"]}, "layers": layers,
            "final_norm": {"weight": t["final.norm"]}, "head": {"weight": t["embed"]}}


PAFOLORN = Architecture(name=ARCHITECTURE, read_config=read_config, declare_tensors=declare_tensors,
                        bind_tensors=bind_tensors, aliases=("pafolorn",))
ModelSupport.add_model(PAFOLORN)
