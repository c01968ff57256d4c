"""Pafolorn without a GPU: its configuration, run order and cache slots, tensor declarations, the random-weights mode,
and the plain implementation against values worked out by hand."""
import json
import math

import numpy as np
import pytest
import torch

import plain_pafolorn as P
from pafolorn_models import CONFIG_F, CONFIG_G, CONFIG_H


def test_config_reads_every_size_and_constant():
    from deliverance_amd.config import ConfigError
    from deliverance_amd.config.pafolorn import PafolornConfig
    from deliverance_amd.config.specs import AttentionSpec, DeltaRuleSpec, DenseFeedForwardSpec, ParallelMixerSpec
    for raw_cfg in (CONFIG_F, CONFIG_G, CONFIG_H):
        mc = PafolornConfig.from_dict(raw_cfg).to_model_config()
        assert (mc.vocab_size, mc.width) == (raw_cfg["vocab"], raw_cfg["width"])
        assert math.isclose(mc.logit_multiplier, 1.0 / raw_cfg["logit_scale"])
        for norm in (mc.final_norm, mc.embed_norm):
            assert norm.kind == "rmsnorm" and norm.gain_offset == 0.0 and norm.eps == raw_cfg["norm"]["eps"]
        assert len(mc.layers) == len(raw_cfg["layers"])
        for spec, raw in zip(mc.layers, raw_cfg["layers"]):
            assert spec.pre_mixer_norm is None and spec.post_mixer_norm is not None and spec.mixer_scale
            if raw["type"] == "channel_delta":
                d, rd, att = spec.mixer, raw["mixer"], None
                assert isinstance(d, DeltaRuleSpec) and d.decay == "channel" and d.gate == "sigmoid"
                assert d.decay_rank == rd.get("a_rank", -1) and d.gate_rank == rd.get("g_rank", -1)
            else:
                assert isinstance(spec.mixer, ParallelMixerSpec)
                att, d = spec.mixer.branches
                rd, ra = raw["mixer"]["right"], raw["mixer"]["left"]
                assert spec.mixer.scales == (raw["mixer"]["left_scale"], raw["mixer"]["right_scale"])
                assert isinstance(att, AttentionSpec) and isinstance(d, DeltaRuleSpec)
                assert d.decay == "head" and d.gate == "silu" and d.decay_rank == 0 and d.gate_rank == 0
                assert (att.n_heads, att.n_kv_heads, att.head_dim, att.value_dim, att.scale) == \
                    (ra["heads"], ra["kv_heads"], ra["dim"], ra["vdim"], ra["scale"])
                assert (att.window, att.keep_first, att.score_softcap) == (ra["mask"]["size"], ra["mask"]["keep_first"], ra.get("softcap", 0.0))
                assert (att.position.dims, att.position.base, att.position.interleaved) == (ra["rot"]["dims"], ra["rot"]["base"], False)
                assert att.qk_norm.whole and att.qk_norm.eps == raw_cfg["norm"]["eps"] and not att.qkv_bias and not att.out_bias
            assert (d.n_heads, d.n_kv_heads, d.head_dim, d.v_head_dim, d.conv_taps) == \
                (rd["heads"], rd["kv_heads"], rd["dim"], rd["vdim"], rd["conv"])
            assert d.norm_eps == raw_cfg["norm"]["eps"] and d.unit_eps == 1e-6
            if raw["mlp"] is None:
                assert spec.feed_forward is None and spec.post_ff_norm is None and not spec.ff_scale
            else:
                f = spec.feed_forward
                assert isinstance(f, DenseFeedForwardSpec) and f.inner == raw["mlp"]["ff"] and f.activation == "relu2" and not f.bias
                assert spec.pre_ff_norm is None and spec.post_ff_norm is not None and spec.ff_scale
    # what is missing is named, all of it at once
    broken = json.loads(json.dumps(CONFIG_F))
    del broken["logit_scale"], broken["layers"][0]["mixer"]["left"]["mask"]["keep_first"], broken["layers"][1]["mixer"]["conv"]
    del broken["layers"][2]["mixer"]["right_scale"]
    with pytest.raises(ConfigError) as e:
        PafolornConfig.from_dict(broken)
    for key in ("logit_scale", "layers[0].mixer.left.mask.keep_first", "layers[1].mixer.conv", "layers[2].mixer.right_scale"):
        assert key in str(e.value)
    other = json.loads(json.dumps(CONFIG_F))
    other["layers"][1]["type"] = "recurrence"
    with pytest.raises(ConfigError, match="recurrence"):
        PafolornConfig.from_dict(other)
    other = json.loads(json.dumps(CONFIG_F))
    other["layers"][0]["mixer"]["left"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="multiple"):
        PafolornConfig.from_dict(other)
    other = json.loads(json.dumps(CONFIG_F))
    other["layers"][0]["mixer"]["left"]["rot"]["dims"] = 34
    with pytest.raises(ConfigError, match="rot.dims"):
        PafolornConfig.from_dict(other)
    other = json.loads(json.dumps(CONFIG_F))
    other["layers"][0]["mlp"]["kind"] = "moe"
    with pytest.raises(ConfigError, match="moe"):
        PafolornConfig.from_dict(other)


@pytest.mark.parametrize("cfg", [CONFIG_F, CONFIG_G, CONFIG_H])
def test_every_branch_has_a_cache_slot_of_its_own(cfg):
    from deliverance_amd.config.pafolorn import PafolornConfig
    mc = PafolornConfig.from_dict(cfg).to_model_config()
    assert [c.layer for c in mc.schedule] == list(range(len(cfg["layers"]))) and all(c.write for c in mc.schedule)
    slot = 0
    for call, raw in zip(mc.schedule, cfg["layers"]):
        assert call.cache == slot
        slot += 2 if raw["type"] == "parallel" else 1
    assert mc.n_cache_slots == slot


def test_registry_finds_the_design_by_its_name():
    from deliverance_amd import models  # noqa: F401
    from deliverance_amd.registry import ModelSupport
    assert ModelSupport.detect(CONFIG_F).name == "Pafolorn"
    assert ModelSupport.detect({"architecture": "pafolorn"}).name == "Pafolorn"
    assert {"Pafolorn", "Virudra", "GPT2LMHeadModel"} <= set(ModelSupport.names())


def test_random_model_round_trip(tmp_path):
    """The random-weights mode writes what the loader reads back; low ranks that config.json leaves out are the
    tensors' to say; a tensor of another shape is an error that names it."""
    from deliverance_amd import models  # noqa: F401
    from deliverance_amd.random_model import random_model
    from deliverance_amd.registry import ModelSupport
    from deliverance_amd.weights.loader import WeightError, load_declared
    folder = random_model(str(tmp_path / "m"), CONFIG_G, seed=5)
    cfg = json.load(open(f"{folder}/config.json"))
    arch = ModelSupport.detect(cfg)
    mc = arch.read_config(cfg)
    t = load_declared(folder, arch.declare_tensors(mc))
    m0, m1 = CONFIG_G["layers"][0]["mixer"], CONFIG_G["layers"][1]["mixer"]
    assert tuple(t["l0.mix.a1"].shape) == (m0["a_rank"], CONFIG_G["width"])
    assert tuple(t["l0.mix.a2"].shape) == (m0["heads"] * m0["dim"], m0["a_rank"])
    assert tuple(t["l0.mix.g2"].shape) == (m0["heads"] * m0["vdim"], m0["g_rank"])
    assert tuple(t["l0.mix.dt_bias"].shape) == (m0["heads"] * m0["dim"],)
    assert tuple(t["l1.mix.right.dt_bias"].shape) == (m1["right"]["heads"],)
    assert tuple(t["l1.mix.right.q.conv"].shape) == (m1["right"]["kv_heads"] * m1["right"]["dim"], m1["right"]["conv"])
    assert tuple(t["l1.mix.left.q.norm"].shape) == (m1["left"]["heads"] * m1["left"]["dim"],)
    assert "l1.norm2" not in t and "l1.mlp.up" not in t and "l0.norm2" in t and "l0.ls2" in t
    bound = arch.bind_tensors(mc, t)
    left = bound["layers"][1]["mixer"]["branches"][0]
    a = m1["left"]
    assert tuple(left["qkv_weight"].shape) == (a["heads"] * a["dim"] + a["kv_heads"] * (a["dim"] + a["vdim"]), CONFIG_G["width"])
    assert bound["head"]["weight"] is bound["embed"]["tokens"]
    for L in cfg["layers"]:
        L["mixer"].pop("a_rank", None); L["mixer"].pop("g_rank", None)
    t2 = load_declared(folder, arch.declare_tensors(arch.read_config(cfg)))
    assert t2["l0.mix.a1"].shape == t["l0.mix.a1"].shape and t2["l0.mix.g1"].shape == t["l0.mix.g1"].shape
    cfg["layers"][1]["mixer"]["right"]["heads"] = 9
    with pytest.raises(WeightError, match="l1.mix.right"):
        load_declared(folder, arch.declare_tensors(arch.read_config(cfg)))


def test_plain_mechanisms_in_closed_form():
    """The plain implementation against values worked out by hand."""
    assert np.allclose(P.unit_rms(np.array([[3.0, -4.0]]), 0.0), [[3 / math.sqrt(12.5), -4 / math.sqrt(12.5)]])
    assert np.allclose(P.unit_length(np.array([[3.0, -4.0]]), 0.0), [[0.6, -0.8]])
    assert math.isclose(float(P.soft_plus(np.array(0.0))), math.log(2)) and float(P.squared_ramp(np.array(-2.0))) == 0.0
    # the filter's last column is the current token's
    x = np.array([[1.0], [10.0], [100.0]])
    assert P.short_filter(x, np.array([[3.0, 2.0]])).ravel().tolist() == [2.0, 23.0, 230.0]
    # the window and its kept first tokens
    seen = P.visible(6, 2, 1)
    assert seen[5].tolist() == [True, False, False, False, True, True] and seen[1].tolist() == [True, True, False, False, False, False]
    assert P.visible(4, 1, 0)[3].tolist() == [False, False, False, True]
    # a quarter turn of the pair (entry 0, entry 1) of two turned entries; the third passes
    v = np.array([[[1.0, 0.0, 7.0]]])
    out = P.turn_halves(np.repeat(v, 2, axis=0), [0, 1], 2, 100.0)
    assert np.allclose(out[0], v[0]) and np.allclose(out[1, 0], [math.cos(1.0), math.sin(1.0), 7.0])
    # two tokens of the delta rule with keys at a right angle: the second reads what the first wrote, decayed
    q = np.array([[1.0, 0.0], [1.0, 0.0]]); k = np.array([[1.0, 0.0], [0.0, 1.0]]); v = np.array([[2.0], [5.0]])
    o, S = P.delta_recurrence(q, k, v, np.array([0.5, 1.0]), np.array([[1.0, 1.0], [0.25, 1.0]]))
    assert o.ravel().tolist() == [1.0, 0.25] and S.tolist() == [[0.25], [5.0]]
    # the same key twice with beta 1: the second write replaces the first
    o, S = P.delta_recurrence(q, q, v, np.array([1.0, 1.0]), np.ones((2, 2)))
    assert o.ravel().tolist() == [2.0, 5.0]
    # capped scores of one query over two keys
    m = {"scale": 2.0, "softcap": 3.0, "mask": {"size": 8, "keep_first": 0}}
    qq = np.array([[[1.0]], [[1.0]]]); kk = np.array([[[0.5]], [[-0.25]]]); vv = np.array([[[10.0]], [[20.0]]])
    s = 3.0 * np.tanh(np.array([1.0, -0.5]) / 3.0)
    w = np.exp(s) / np.exp(s).sum()
    out = P.attend(qq, kk, vv, m)
    assert math.isclose(out[0, 0, 0], 10.0) and math.isclose(out[1, 0, 0], w[0] * 10 + w[1] * 20)
