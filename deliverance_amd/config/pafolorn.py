"""Typed Pafolorn configuration, read from the design's own config.json keys.

A Pafolorn model is a list of layers.  Every layer has a mixer that reads the residual stream itself (no norm in
front), a root-mean-square norm behind it, and a learned scale per channel; then, unless its ``mlp`` is null, a dense
feed-forward (the square of relu) wired the same way.  The mixer is a gated delta rule with a decay per key channel
(``channel_delta``), or two mixers side by side whose results are added with two constants (``parallel``): softmax
attention over a sliding window that also keeps a sequence's first tokens, beside a gated delta rule with a decay per
head.  The embedded tokens pass a norm before the first layer; the head is the embedding table times a constant.
config.json::

    {"architecture": "Pafolorn", "vocab": V, "width": E, "norm": {"eps": e}, "logit_scale": s,
     "layers": [{"type": "channel_delta",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"},
                 "mlp": null | {"kind": "dense", "ff": F}},
                {"type": "parallel",
                 "mixer": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap",
                                    "mask": {"size", "keep_first"}, "rot": {"base", "dims"}},
                           "right": {"heads", "kv_heads", "dim", "vdim", "conv"},
                           "left_scale": a, "right_scale": b},
                 "mlp": ...}, ...]}

The low ranks of a ``channel_delta`` mixer's decay and gate projections are the checkpoint's to say (its tensors'
shapes); a config.json may name them as ``mixer.a_rank`` and ``mixer.g_rank``, which the random-weights mode needs.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

from .pedatar import _float, _get, _int
from .specs import (AttentionSpec, ConfigError, DeltaRuleSpec, DenseFeedForwardSpec, LayerCall, LayerSpec, ModelConfig,
                    NormSpec, ParallelMixerSpec, PositionSpec, QKNormSpec, RotarySpec)

ARCHITECTURE = "Pafolorn"
DEFAULT_MAX_POSITIONS = 1 << 20     # positions enter through angles only: requests are bounded by the cache
FF_ACTIVATION = "relu2"             # fixed by the design
UNIT_EPS = 1e-6                     # under the root when q and k are scaled to unit length; fixed by the design
MIXERS = ("channel_delta", "parallel")

_DELTA_INTS = ("heads", "kv_heads", "dim", "vdim", "conv")
_ATT_INTS = ("heads", "kv_heads", "dim", "vdim")


@dataclass(frozen=True)
class PafolornDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # the low ranks of a channel-wise decay and its gate; -1: as the checkpoint's tensors say
    a_rank: int = -1
    g_rank: int = -1

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        if self.a_rank > 0:
            d["a_rank"] = self.a_rank
        if self.g_rank > 0:
            d["g_rank"] = self.g_rank
        return d


@dataclass(frozen=True)
class PafolornAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float          # 0: none
    window: int
    keep_first: int
    rot_base: float
    rot_dims: int

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "softcap": self.softcap, "mask": {"size": self.window, "keep_first": self.keep_first},
                "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class PafolornLayer:
    kind: str                                   # "channel_delta" | "parallel"
    delta: PafolornDelta                        # the layer's delta rule (the right one of a parallel layer)
    attention: Optional[PafolornAttention]      # the left one of a parallel layer
    left_scale: float = 1.0
    right_scale: float = 1.0
    ff: int = 0                                 # 0: no feed-forward


def _read_delta(m, where: str, missing: List[str]) -> Optional[PafolornDelta]:
    n0 = len(missing)
    v = {k: _get(m, k, where, missing) for k in _DELTA_INTS}
    if len(missing) > n0:
        return None
    ranks = {k: _int(m[k], where + k) for k in ("a_rank", "g_rank") if m.get(k) is not None}
    return PafolornDelta(**{k: _int(v[k], where + k) for k in _DELTA_INTS}, **ranks)


def _read_attention(m, where: str, missing: List[str]) -> Optional[PafolornAttention]:
    n0 = len(missing)
    v = {k: _get(m, k, where, missing) for k in _ATT_INTS}
    scale = _get(m, "scale", where, missing)
    mask, rot = _get(m, "mask", where, missing), _get(m, "rot", where, missing)
    size = _get(mask, "size", where + "mask.", missing) if mask is not None else None
    keep = _get(mask, "keep_first", where + "mask.", missing) if mask is not None else None
    base = _get(rot, "base", where + "rot.", missing) if rot is not None else None
    dims = _get(rot, "dims", where + "rot.", missing) if rot is not None else None
    if len(missing) > n0:
        return None
    cap = m.get("softcap")
    return PafolornAttention(**{k: _int(v[k], where + k) for k in _ATT_INTS}, scale=_float(scale, where + "scale"),
                             softcap=0.0 if cap is None else _float(cap, where + "softcap"),
                             window=_int(size, where + "mask.size"), keep_first=_int(keep, where + "mask.keep_first", 0),
                             rot_base=_float(base, where + "rot.base"), rot_dims=_int(dims, where + "rot.dims", 0))


@dataclass(frozen=True)
class PafolornConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: Tuple[PafolornLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: dict) -> "PafolornConfig":
        missing: List[str] = []
        vocab, width = _get(d, "vocab", "", missing), _get(d, "width", "", missing)
        norm = _get(d, "norm", "", missing)
        eps = _get(norm, "eps", "norm.", missing) if norm is not None else None
        logit_scale = _get(d, "logit_scale", "", missing)
        raw_layers = _get(d, "layers", "", missing)
        layers: List[PafolornLayer] = []
        for i, L in enumerate(raw_layers or []):
            w = f"layers[{i}]."
            kind = _get(L, "type", w, missing)
            if kind is not None and kind not in MIXERS:
                raise ConfigError(f"{w}type is {kind!r}; this design's mixers: {', '.join(repr(k) for k in MIXERS)}")
            m = _get(L, "mixer", w, missing)
            if kind is None or m is None:
                continue
            n0 = len(missing)
            attention, ls, rs = None, 1.0, 1.0
            if kind == "channel_delta":
                delta = _read_delta(m, w + "mixer.", missing)
            else:
                left, right = _get(m, "left", w + "mixer.", missing), _get(m, "right", w + "mixer.", missing)
                attention = _read_attention(left, w + "mixer.left.", missing) if left is not None else None
                delta = _read_delta(right, w + "mixer.right.", missing) if right is not None else None
                ls, rs = _get(m, "left_scale", w + "mixer.", missing), _get(m, "right_scale", w + "mixer.", missing)
            mlp = L.get("mlp") if isinstance(L, dict) else None
            ff = 0
            if mlp is not None:
                mk = _get(mlp, "kind", w + "mlp.", missing)
                if mk is not None and mk != "dense":
                    raise ConfigError(f"{w}mlp.kind is {mk!r}; this design's feed-forward: 'dense'")
                f = _get(mlp, "ff", w + "mlp.", missing)
                ff = _int(f, w + "mlp.ff") if f is not None else 0
            if len(missing) > n0:
                continue
            layers.append(PafolornLayer(kind=kind, delta=delta, attention=attention,
                                        left_scale=_float(ls, w + "mixer.left_scale"),
                                        right_scale=_float(rs, w + "mixer.right_scale"), ff=ff))
        if missing:
            raise ConfigError("Pafolorn config.json lacks required keys: " + ", ".join(missing))
        cfg = cls(vocab=_int(vocab, "vocab"), width=_int(width, "width"), eps=_float(eps, "norm.eps"),
                  logit_scale=_float(logit_scale, "logit_scale"), layers=tuple(layers),
                  max_positions=_int(d.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions"),
                  bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.layers:
            raise ConfigError("a Pafolorn model needs at least one layer")
        if not (self.eps > 0.0):
            raise ConfigError(f"norm.eps must be > 0, found {self.eps}")
        if self.logit_scale == 0.0:
            raise ConfigError("logit_scale must not be 0")
        for i, L in enumerate(self.layers):
            for name, m in (("delta rule", L.delta), ("attention", L.attention)):
                if m is not None and m.heads % m.kv_heads != 0:
                    raise ConfigError(f"layers[{i}]: the {name}'s {m.heads} heads are not a multiple of its "
                                      f"{m.kv_heads} key heads")
            a = L.attention
            if a is not None:
                if not (a.scale > 0.0):
                    raise ConfigError(f"layers[{i}]: the score scale must be positive, found {a.scale}")
                if a.softcap < 0.0:
                    raise ConfigError(f"layers[{i}]: softcap must not be negative, found {a.softcap}")
                if a.rot_dims % 2 != 0 or a.rot_dims > a.dim:
                    raise ConfigError(f"layers[{i}]: rot.dims {a.rot_dims} must be even and at most dim {a.dim}")
                if not (a.rot_base > 0.0):
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")

    def to_dict(self) -> dict:
        layers = []
        for L in self.layers:
            if L.kind == "channel_delta":
                mixer = L.delta.to_dict()
            else:
                mixer = {"left": L.attention.to_dict(), "right": L.delta.to_dict(), "left_scale": L.left_scale,
                         "right_scale": L.right_scale}
            layers.append({"type": L.kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "logit_scale": self.logit_scale, "layers": layers}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    # ---- the model as parts ------------------------------------------------------------------
    def _delta_spec(self, m: PafolornDelta, channel: bool) -> DeltaRuleSpec:
        # a channel-wise decay and its gate go through low ranks (-1: the tensors' shapes name them)
        return DeltaRuleSpec(kind="delta_rule", width=self.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                             v_head_dim=m.vdim, conv_taps=m.conv, norm_eps=self.eps,
                             decay="channel" if channel else "head", decay_rank=m.a_rank if channel else 0,
                             gate="sigmoid" if channel else "silu", gate_rank=m.g_rank if channel else 0,
                             unit_eps=UNIT_EPS)

    def _attention_spec(self, a: PafolornAttention) -> AttentionSpec:
        return AttentionSpec(kind="attention", width=self.width, n_heads=a.heads, n_kv_heads=a.kv_heads, head_dim=a.dim,
                             scale=a.scale, qkv_bias=False, out_bias=False, window=a.window,
                             position=RotarySpec("rotary", dims=a.rot_dims, base=a.rot_base, interleaved=False),
                             v_head_dim=a.vdim, qk_norm=QKNormSpec(eps=self.eps, whole=True), score_softcap=a.softcap,
                             keep_first=a.keep_first)

    def to_model_config(self) -> ModelConfig:
        norm = NormSpec("rmsnorm", self.width, self.eps, bias=False, gain_offset=0.0)
        specs, schedule, slot = [], [], 0
        for i, L in enumerate(self.layers):
            if L.kind == "channel_delta":
                mixer, n_slots = self._delta_spec(L.delta, True), 1
            else:
                mixer = ParallelMixerSpec("parallel", branches=(self._attention_spec(L.attention),
                                                                self._delta_spec(L.delta, False)),
                                          scales=(L.left_scale, L.right_scale))
                n_slots = 2
            ff = DenseFeedForwardSpec("dense", self.width, L.ff, FF_ACTIVATION, bias=False) if L.ff else None
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, post_mixer_norm=norm,
                                   post_ff_norm=None if ff is None else norm, weight_prefix=f"l{i}.",
                                   mixer_scale=True, ff_scale=ff is not None))
            schedule.append(LayerCall(i, slot, True))
            slot += n_slots
        eos = () if self.eos_token_id is None else (int(self.eos_token_id),)
        return ModelConfig(
            architecture=ARCHITECTURE, vocab_size=self.vocab, width=self.width, max_positions=self.max_positions,
            layers=tuple(specs), schedule=tuple(schedule), embed_position=PositionSpec("none"), final_norm=norm,
            tie_word_embeddings=True, bos_token_id=self.bos_token_id, eos_token_ids=eos, raw=self.to_dict(),
            logit_multiplier=1.0 / self.logit_scale, embed_norm=norm)
