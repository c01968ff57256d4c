"""Salivik: which checkpoint tensors feed which part.

Names: ``embed``, ``embed.norm``, ``loop.in`` (with a loop), ``head``, ``final.norm``; per layer ``l<i>.norm1``,
``l<i>.norm2``; an attention mixer ``l<i>.mix.{q, k, g, o}``; a retention mixer ``l<i>.mix.{q, k, v, g, o}``; a
latent-attention mixer ``l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, sink, o}``; a dense feed-forward
``l<i>.mlp.{gate, up, down}``; a routed one ``l<i>.mlp.router``, ``l<i>.mlp.router.b``, ``l<i>.mlp.e<j>.{gate, up,
down}`` and ``l<i>.mlp.shared.{gate, up, down}``.  Linear weights are stored [out, in].  Gate and up of a
feed-forward become one matrix and the experts of a layer one stack at load time; an attention mixer's one
product gives q | k | gate (the values are the keys before their turn).
"""
from __future__ import annotations

from typing import List

import torch

from ..config.salivik import ARCHITECTURE, SalivikConfig
from ..config.specs import (AttentionSpec, ExpertsFeedForwardSpec, GatedFeedForwardSpec, LatentAttentionSpec, ModelConfig,
                            RetentionSpec)
from ..registry import Architecture, ModelSupport
from ..weights.loader import TensorDecl

# Random-weights distributions: matrices N(0, 0.05) (the second factors of low ranks and the experts twice, routers
# four times that), norm gains 1 + N(0, 0.1), sinks and router biases N(0, 0.5).
W_STD, GAIN_STD = 0.05, 0.1


def read_config(d: dict) -> ModelConfig:
    return SalivikConfig.from_dict(d).to_model_config()


def _gated(p: str, inner: int, E: int, std: float) -> List[TensorDecl]:
    return [TensorDecl(p + "gate", (inner, E), "normal", std), TensorDecl(p + "up", (inner, E), "normal", std),
            TensorDecl(p + "down", (E, inner), "normal", std)]


def declare_tensors(mc: ModelConfig) -> List[TensorDecl]:
    E, V = mc.width, mc.vocab_size
    out = [TensorDecl("embed", (V, E), "normal", 0.3), TensorDecl("embed.norm", (E,), "ones_plus_normal", GAIN_STD)]
    if mc.input_mix:
        out.append(TensorDecl("loop.in", (E, 2 * E), "normal", 1.5 * W_STD))
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        out.append(TensorDecl(p + "norm1", (E,), "ones_plus_normal", GAIN_STD))
        if isinstance(m, AttentionSpec):
            out += [TensorDecl(p + "mix.q", (m.n_heads * m.head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.k", (m.n_kv_heads * m.head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.g", (m.n_heads * m.head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.o", (E, m.n_heads * m.head_dim), "normal", W_STD)]
        elif isinstance(m, RetentionSpec):
            out += [TensorDecl(p + "mix.q", (m.n_heads * m.head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.k", (m.n_heads * m.head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.v", (m.n_heads * m.v_head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.g", (m.n_heads * m.v_head_dim, E), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.o", (E, m.n_heads * m.v_head_dim), "normal", W_STD)]
        elif isinstance(m, LatentAttentionSpec):
            H = m.n_heads
            out += [TensorDecl(p + "mix.dq", (m.q_rank, E), "normal", W_STD),
                    TensorDecl(p + "mix.dq.norm", (m.q_rank,), "ones_plus_normal", GAIN_STD),
                    TensorDecl(p + "mix.uq", (H * (m.head_dim + m.rot_dim), m.q_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.dkv", (m.kv_rank + m.rot_dim, E), "normal", W_STD),
                    TensorDecl(p + "mix.dkv.norm", (m.kv_rank,), "ones_plus_normal", GAIN_STD),
                    TensorDecl(p + "mix.uk", (H * m.head_dim, m.kv_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.uv", (H * m.v_head_dim, m.kv_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.sink", (H,), "normal", 0.5),
                    TensorDecl(p + "mix.o", (E, H * m.v_head_dim), "normal", W_STD)]
        else:
            raise TypeError(f"no tensors are known for a mixer of kind {getattr(m, 'kind', m)!r}")
        if f is None:
            continue
        out.append(TensorDecl(p + "norm2", (E,), "ones_plus_normal", GAIN_STD))
        if isinstance(f, GatedFeedForwardSpec):
            out += _gated(p + "mlp.", f.inner, E, W_STD)
        elif isinstance(f, ExpertsFeedForwardSpec):
            for j in range(f.n_experts):
                out += _gated(f"{p}mlp.e{j}.", f.inner, E, 2 * W_STD)
            out += [TensorDecl(p + "mlp.router", (f.n_experts, E), "normal", 4 * W_STD),
                    TensorDecl(p + "mlp.router.b", (f.n_experts,), "normal", 0.5)]
            if f.shared_inner:
                out += _gated(p + "mlp.shared.", f.shared_inner, E, W_STD)
        else:
            raise TypeError(f"no tensors are known for a feed-forward of kind {getattr(f, 'kind', f)!r}")
    out += [TensorDecl("final.norm", (E,), "ones_plus_normal", GAIN_STD), TensorDecl("head", (V, E), "normal", W_STD)]
    return out


def bind_tensors(mc: ModelConfig, t: dict) -> dict:
    layers = []
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        d = {"pre_mixer_norm": {"weight": t[p + "norm1"]}}
        if isinstance(m, AttentionSpec):
            # q | k | gate in one product
            d["mixer"] = {"qkv_weight": torch.cat([t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.g"]], dim=0),
                          "out_weight": t[p + "mix.o"]}
        elif isinstance(m, RetentionSpec):
            d["mixer"] = {"q_weight": t[p + "mix.q"], "k_weight": t[p + "mix.k"], "v_weight": t[p + "mix.v"],
                          "gate_weight": t[p + "mix.g"], "out_weight": t[p + "mix.o"]}
        else:
            d["mixer"] = {"q_down_weight": t[p + "mix.dq"], "q_norm_weight": t[p + "mix.dq.norm"],
                          "q_up_weight": t[p + "mix.uq"], "kv_down_weight": t[p + "mix.dkv"],
                          "kv_norm_weight": t[p + "mix.dkv.norm"], "k_up_weight": t[p + "mix.uk"],
                          "v_up_weight": t[p + "mix.uv"], "sink": t[p + "mix.sink"], "out_weight": t[p + "mix.o"]}
        if f is not None:
            d["pre_ff_norm"] = {"weight": t[p + "norm2"]}
            if isinstance(f, GatedFeedForwardSpec):
                d["feed_forward"] = {"gate_up_weight": torch.cat([t[p + "mlp.gate"], t[p + "mlp.up"]], dim=0),
                                     "down_weight": t[p + "mlp.down"]}
            else:
                ff = {"gate_up_weight": torch.stack([torch.cat([t[f"{p}mlp.e{j}.gate"], t[f"{p}mlp.e{j}.up"]], dim=0)
                                                     for j in range(f.n_experts)]),
                      "down_weight": torch.stack([t[f"{p}mlp.e{j}.down"] for j in range(f.n_experts)]),
                      "router_weight": t[p + "mlp.router"], "router_bias": t[p + "mlp.router.b"]}
                if f.shared_inner:
                    ff["shared_gate_up_weight"] = torch.cat([t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"]], dim=0)
                    ff["shared_down_weight"] = t[p + "mlp.shared.down"]
                d["feed_forward"] = ff
        layers.append(d)
    out = {"embed": {"tokens": t["embed"]}, "embed_norm": {"weight": t["embed.norm"]}, "layers": layers,
           "final_norm": {"weight": t["final.norm"]}, "head": {"weight": t["head"]}}
    if mc.input_mix:
        out["input_mix"] = {"weight": t["loop.in"]}
    return out


SALIVIK = Architecture(name=ARCHITECTURE, read_config=read_config, declare_tensors=declare_tensors,
                       bind_tensors=bind_tensors, aliases=("salivik",))
ModelSupport.add_model(SALIVIK)
