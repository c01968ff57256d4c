"""Typed Salivik configuration, read from the design's own config.json keys.

A Salivik model is a list of layers; each has one mixer behind a root-mean-square norm (softmax attention over a
window whose keys are also its values, retention with a fixed decay per head, or attention over a narrow latent
vector) and, behind a second norm, a capped gated feed-forward that is dense or a mixture of experts (or none).  A
range of layers may run several times with the same weights; every pass keeps a cache or state of its own and
starts by mixing the stream with the embedding output.  config.json::

    {"architecture": "Salivik", "vocab": V, "width": E, "norm": {"eps": e},
     "loop": null | {"start": a, "stop": b, "times": n},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}, "rot": {"base", "dims"}},
                 "mlp": null | {"kind": "dense", "ff": F, "limit": c}
                             | {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"},
                                "shared": null | {"ff", "limit"}}},
                {"type": "retention", "mixer": {"heads", "dim", "vdim", "decay": [..], "rot": {"base", "dims"}}, ...},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "mask": {"size"},
                           "rot": {"base", "dims", "scaling": null | {"factor", "original", "fast", "slow"}}}, ...}]}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

from .specs import (AttentionSpec, ConfigError, ExpertsFeedForwardSpec, GatedFeedForwardSpec, LatentAttentionSpec,
                    LayerCall, LayerSpec, ModelConfig, NormSpec, PositionSpec, RampedSpeedsSpec, RetentionSpec,
                    RotarySpec)

ARCHITECTURE = "Salivik"
# The design has no position limit of its own (positions enter through angles only): requests are bounded by
# the cache.  This is what the scheduler and the step function check against.
DEFAULT_MAX_POSITIONS = 1 << 20
FF_ACTIVATION = "glu_capped"        # the design fixes the feed-forwards' form; their limits come from config.json
MIXERS = ("attention", "retention", "latent_attention")


class _Reader:
    """Looks keys up in nested dicts and remembers every one that is missing, so that one error names them all."""

    def __init__(self):
        self.missing: List[str] = []

    def get(self, d, key: str, where: str):
        if not isinstance(d, dict) or d.get(key) is None:
            self.missing.append(f"{where}{key}")
            return None
        return d[key]


def _int(value, where: str, minimum: int = 1) -> int:
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config key {where!r} must be an integer, found {value!r}")
    if value < minimum:
        raise ConfigError(f"config key {where!r} must be at least {minimum}, found {value}")
    return value


def _float(value, where: str, positive: bool = False) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config key {where!r} must be a number, found {value!r}")
    if positive and not (float(value) > 0.0):
        raise ConfigError(f"config key {where!r} must be positive, found {value}")
    return float(value)


@dataclass(frozen=True)
class SalivikRotation:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]] = None      # factor, original, fast, slow

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            f, o, a, b = self.scaling
            d["scaling"] = {"factor": f, "original": o, "fast": a, "slow": b}
        return d

    def spec(self) -> RotarySpec:
        sc = None if self.scaling is None else RampedSpeedsSpec(*self.scaling)
        return RotarySpec("rotary", dims=self.dims, base=self.base, interleaved=False, scaling=sc)


@dataclass(frozen=True)
class SalivikFeedForward:
    kind: str                       # "dense" | "moe"
    ff: int
    limit: float
    experts: int = 0
    top: int = 0
    shared_ff: int = 0              # 0: no shared expert
    shared_limit: float = 0.0

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top},
                "shared": {"ff": self.shared_ff, "limit": self.shared_limit} if self.shared_ff else None}


@dataclass(frozen=True)
class SalivikLayer:
    kind: str
    sizes: Tuple[Tuple[str, int], ...]        # the mixer's integer sizes by their config names
    rot: SalivikRotation
    scale: float = 0.0                        # the score scale of the two attentions
    window: int = 0                           # mask.size of the two attentions
    decay: Tuple[float, ...] = ()             # retention: one a head
    mlp: Optional[SalivikFeedForward] = None

    def n(self, key: str) -> int:
        return dict(self.sizes)[key]


_INTS = {"attention": ("heads", "kv_heads", "dim", "vdim"),
         "retention": ("heads", "dim", "vdim"),
         "latent_attention": ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank")}


def _read_rotation(r: _Reader, m, w: str):
    rot = r.get(m, "rot", w)
    if rot is None:
        return None
    base, dims = r.get(rot, "base", w + "rot."), r.get(rot, "dims", w + "rot.")
    sc = rot.get("scaling") if isinstance(rot, dict) else None
    vals = None
    if sc is not None:
        vals = [r.get(sc, k, w + "rot.scaling.") for k in ("factor", "original", "fast", "slow")]
    if base is None or dims is None or (vals is not None and any(v is None for v in vals)):
        return None
    scaling = None
    if vals is not None:
        scaling = tuple(_float(v, w + "rot.scaling." + k, positive=True)
                        for v, k in zip(vals, ("factor", "original", "fast", "slow")))
    return SalivikRotation(_float(base, w + "rot.base", positive=True), _int(dims, w + "rot.dims", 0), scaling)


def _read_feed_forward(r: _Reader, mlp, w: str) -> Optional[SalivikFeedForward]:
    n0 = len(r.missing)
    kind = r.get(mlp, "kind", w)
    if kind is None:
        return None
    if kind == "dense":
        ff, limit = r.get(mlp, "ff", w), r.get(mlp, "limit", w)
        if len(r.missing) > n0:
            return None
        return SalivikFeedForward("dense", _int(ff, w + "ff"), _float(limit, w + "limit", positive=True))
    if kind != "moe":
        raise ConfigError(f"{w}kind is {kind!r}; this design's feed-forwards: 'dense', 'moe'")
    ex, ro = r.get(mlp, "expert", w), r.get(mlp, "router", w)
    ff = r.get(ex, "ff", w + "expert.") if ex is not None else None
    limit = r.get(ex, "limit", w + "expert.") if ex is not None else None
    n = r.get(ro, "experts", w + "router.") if ro is not None else None
    top = r.get(ro, "top", w + "router.") if ro is not None else None
    sh = mlp.get("shared") if isinstance(mlp, dict) else None
    sf = r.get(sh, "ff", w + "shared.") if sh is not None else None
    sl = r.get(sh, "limit", w + "shared.") if sh is not None else None
    if len(r.missing) > n0:
        return None
    return SalivikFeedForward("moe", _int(ff, w + "expert.ff"), _float(limit, w + "expert.limit", positive=True),
                              experts=_int(n, w + "router.experts"), top=_int(top, w + "router.top"),
                              shared_ff=_int(sf, w + "shared.ff") if sh is not None else 0,
                              shared_limit=_float(sl, w + "shared.limit", positive=True) if sh is not None else 0.0)


@dataclass(frozen=True)
class SalivikConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[SalivikLayer, ...]
    loop: Optional[Tuple[int, int, int]] = None       # start, stop, times
    max_positions: int = DEFAULT_MAX_POSITIONS
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: dict) -> "SalivikConfig":
        r = _Reader()
        vocab, width = r.get(d, "vocab", ""), r.get(d, "width", "")
        norm = r.get(d, "norm", "")
        eps = r.get(norm, "eps", "norm.") if norm is not None else None
        raw_layers = r.get(d, "layers", "")
        layers: List[SalivikLayer] = []
        for i, L in enumerate(raw_layers or []):
            w = f"layers[{i}]."
            kind = r.get(L, "type", w)
            if kind is not None and kind not in MIXERS:
                raise ConfigError(f"{w}type is {kind!r}; this design's mixers: {', '.join(repr(k) for k in MIXERS)}")
            m = r.get(L, "mixer", w)
            if kind is None or m is None:
                continue
            n0 = len(r.missing)
            wm = w + "mixer."
            # (an attention mixer's values are its keys: a missing vdim is the keys' size)
            ints = {k: m.get("dim") if (kind == "attention" and k == "vdim" and isinstance(m, dict) and m.get("vdim") is None)
                    else r.get(m, k, wm) for k in _INTS[kind]}
            rot = _read_rotation(r, m, wm)
            scale = window = decay = None
            if kind == "retention":
                decay = r.get(m, "decay", wm)
            else:
                scale = r.get(m, "scale", wm)
                mask = r.get(m, "mask", wm)
                window = r.get(mask, "size", wm + "mask.") if mask is not None else None
            mlp = L.get("mlp") if isinstance(L, dict) else None
            ff = _read_feed_forward(r, mlp, w + "mlp.") if mlp is not None else None
            if len(r.missing) > n0:
                continue
            if decay is not None and (not isinstance(decay, (list, tuple)) or not decay):
                raise ConfigError(f"{wm}decay must be a list with one number a head, found {decay!r}")
            layers.append(SalivikLayer(
                kind=kind, sizes=tuple((k, _int(v, wm + k)) for k, v in ints.items()), rot=rot,
                scale=0.0 if scale is None else _float(scale, wm + "scale", positive=True),
                window=0 if window is None else _int(window, wm + "mask.size"),
                decay=() if decay is None else tuple(_float(g, wm + "decay") for g in decay), mlp=ff))
        loop = None
        lp = d.get("loop") if isinstance(d, dict) else None
        if lp is not None:
            vals = [r.get(lp, k, "loop.") for k in ("start", "stop", "times")]
            if all(v is not None for v in vals):
                loop = (_int(vals[0], "loop.start", 0), _int(vals[1], "loop.stop", 0), _int(vals[2], "loop.times"))
        if r.missing:
            raise ConfigError("Salivik config.json lacks required keys: " + ", ".join(r.missing))
        cfg = cls(vocab=_int(vocab, "vocab"), width=_int(width, "width"), eps=_float(eps, "norm.eps", positive=True),
                  layers=tuple(layers), loop=loop,
                  max_positions=_int(d.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions"),
                  bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.layers:
            raise ConfigError("a Salivik model needs at least one layer")
        if self.loop is not None:
            a, b, _ = self.loop
            if not (0 <= a < b <= len(self.layers)):
                raise ConfigError(f"loop.start {a} and loop.stop {b} must name a range of the {len(self.layers)} layers")
        for i, L in enumerate(self.layers):
            w = f"layers[{i}]"
            turned = L.n("rot_dim") if L.kind == "latent_attention" else L.n("dim")
            if L.rot.dims % 2 != 0 or L.rot.dims > turned:
                raise ConfigError(f"{w}: rot.dims {L.rot.dims} must be even and at most {turned}")
            if L.kind == "attention":
                if L.n("heads") % L.n("kv_heads") != 0:
                    raise ConfigError(f"{w}: {L.n('heads')} heads are not a multiple of {L.n('kv_heads')} key heads")
                if L.n("vdim") != L.n("dim"):
                    raise ConfigError(f"{w}: the values are the keys, so vdim {L.n('vdim')} must equal dim {L.n('dim')}")
            if L.kind == "retention":
                if len(L.decay) != L.n("heads"):
                    raise ConfigError(f"{w}: {len(L.decay)} decays for {L.n('heads')} heads")
                if any(not (0.0 <= g <= 1.0) for g in L.decay):
                    raise ConfigError(f"{w}: decays must lie in [0, 1], found {list(L.decay)}")
            if L.mlp is not None and L.mlp.kind == "moe" and L.mlp.top > L.mlp.experts:
                raise ConfigError(f"{w}: top {L.mlp.top} of {L.mlp.experts} experts")

    def to_dict(self) -> dict:
        layers = []
        for L in self.layers:
            mixer = dict(L.sizes)
            mixer["rot"] = L.rot.to_dict()
            if L.kind == "retention":
                mixer["decay"] = list(L.decay)
            else:
                mixer["scale"] = L.scale
                mixer["mask"] = {"size": L.window}
            layers.append({"type": L.kind, "mixer": mixer, "mlp": None if L.mlp is None else L.mlp.to_dict()})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "layers": layers}
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    def run_order(self) -> List[Tuple[int, bool]]:
        """(layer, whether a pass of the loop starts here), in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop
        order = [(i, False) for i in range(a)]
        for _ in range(times):
            order += [(i, i == a) for i in range(a, b)]
        return order + [(i, False) for i in range(b, n)]

    # ---- the model as parts ------------------------------------------------------------------
    def to_model_config(self) -> ModelConfig:
        E = self.width
        norm = NormSpec("rmsnorm", E, self.eps, bias=False, gain_offset=0.0)
        specs = []
        for i, L in enumerate(self.layers):
            if L.kind == "attention":
                mixer = AttentionSpec(
                    kind="attention", width=E, n_heads=L.n("heads"), n_kv_heads=L.n("kv_heads"), head_dim=L.n("dim"),
                    scale=L.scale, qkv_bias=False, out_bias=False, window=L.window, position=L.rot.spec(),
                    values_are_keys=True, sink="zero", out_gate="sigmoid")
            elif L.kind == "retention":
                mixer = RetentionSpec(kind="retention", width=E, n_heads=L.n("heads"), head_dim=L.n("dim"),
                                      v_head_dim=L.n("vdim"), decay=L.decay, norm_eps=self.eps, rotary=L.rot.spec(),
                                      gate="silu")
            else:
                mixer = LatentAttentionSpec(
                    kind="latent_attention", width=E, n_heads=L.n("heads"), head_dim=L.n("dim"), rot_dim=L.n("rot_dim"),
                    v_head_dim=L.n("vdim"), q_rank=L.n("q_rank"), kv_rank=L.n("kv_rank"), scale=L.scale,
                    norm_eps=self.eps, rotary=L.rot.spec(), window=L.window, sink=True)
            ff = None
            if L.mlp is not None and L.mlp.kind == "dense":
                ff = GatedFeedForwardSpec("gated", E, L.mlp.ff, FF_ACTIVATION, limit=L.mlp.limit)
            elif L.mlp is not None:
                ff = ExpertsFeedForwardSpec("experts", E, L.mlp.ff, L.mlp.experts, L.mlp.top, FF_ACTIVATION,
                                            router="softmax_top", gated=True, weight_on="output", limit=L.mlp.limit,
                                            shared_inner=L.mlp.shared_ff, shared_activation=FF_ACTIVATION,
                                            shared_gated=True, shared_limit=L.mlp.shared_limit, router_bias=True)
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, pre_mixer_norm=norm,
                                   pre_ff_norm=None if ff is None else norm, weight_prefix=f"l{i}."))
        # every run of a layer has a cache slot or state of its own
        schedule = tuple(LayerCall(layer, run, True, mix_input=starts) for run, (layer, starts) in enumerate(self.run_order()))
        eos = () if self.eos_token_id is None else (int(self.eos_token_id),)
        return ModelConfig(
            architecture=ARCHITECTURE, vocab_size=self.vocab, width=E, max_positions=self.max_positions,
            layers=tuple(specs), schedule=schedule, embed_position=PositionSpec("none"), final_norm=norm,
            tie_word_embeddings=False, bos_token_id=self.bos_token_id, eos_token_ids=eos, raw=self.to_dict(),
            embed_norm=norm, input_mix=self.loop is not None)
