"""Typed Virudra configuration, read from the design's own config.json keys.

A Virudra model is a list of layers, each with an attention mixer and a feed-forward (dense and gated,
a mixture of experts chosen by a table, or none), a range of layers that runs several times in a row with
the same weights (every pass with a cache of its own), root-mean-square norms in front of and behind every
part, and a soft cap on the logits.  config.json::

    {"architecture": "Virudra", "vocab": V, "width": E, "norm": {"eps": e}, "logit_softcap": c,
     "loop": {"start": a, "stop": b, "times": t},
     "layers": [{"type": "attention",
                 "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "bias_max",
                           "q_temp": {"coef", "every"}},
                 "mlp": null | {"kind": "dense", "ff": F}
                             | {"kind": "moe", "expert": {"ff": F}, "router": {"experts": n, "top": k}}}, ...]}

The number of rows of a layer's distance-bias table is not in config.json: it is the table's first
dimension in the checkpoint (``bias_buckets`` may name it, and must when a random model is written).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

from .specs import (AttentionSpec, ConfigError, DistanceBiasSpec, ExpertsFeedForwardSpec, GatedFeedForwardSpec,
                    LayerCall, LayerSpec, ModelConfig, NormSpec, PositionSpec, QueryTemperatureSpec)

ARCHITECTURE = "Virudra"
# The design has no position limit of its own (positions enter through distances and a logarithm only):
# requests are bounded by the cache.  This is what the scheduler and the step function check against.
DEFAULT_MAX_POSITIONS = 1 << 20
DENSE_ACTIVATION = "gelu_pytorch_tanh"      # the design fixes both
EXPERT_ACTIVATION = "silu"


def _get(d: dict, key: str, where: str, missing: List[str]):
    if not isinstance(d, dict) or d.get(key) is None:
        missing.append(f"{where}{key}")
        return None
    return d[key]


def _int(value, where: str, minimum: int = 1) -> int:
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config key {where!r} must be an integer, found {value!r}")
    if value < minimum:
        raise ConfigError(f"config key {where!r} must be at least {minimum}, found {value}")
    return value


def _float(value, where: str) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config key {where!r} must be a number, found {value!r}")
    return float(value)


@dataclass(frozen=True)
class VirudraLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    bias_buckets: Optional[int]     # rows of the distance-bias table; None: the checkpoint's shape says
    temp_coef: float
    temp_every: int
    mlp_kind: Optional[str]         # None | "dense" | "moe"
    ff: int = 0
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class VirudraConfig:
    vocab: int
    width: int
    eps: float
    logit_softcap: float
    layers: Tuple[VirudraLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_positions: int = DEFAULT_MAX_POSITIONS
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: dict) -> "VirudraConfig":
        missing: List[str] = []
        vocab, width = _get(d, "vocab", "", missing), _get(d, "width", "", missing)
        norm = _get(d, "norm", "", missing)
        eps = _get(norm, "eps", "norm.", missing) if norm is not None else None
        raw_layers = _get(d, "layers", "", missing)
        layers: List[VirudraLayer] = []
        for i, L in enumerate(raw_layers or []):
            w = f"layers[{i}]."
            kind = _get(L, "type", w, missing)
            if kind is not None and kind != "attention":
                raise ConfigError(f"{w}type is {kind!r}; this design's mixers: 'attention'")
            m = _get(L, "mixer", w, missing)
            if m is None:
                continue
            vals = {k: _get(m, k, w + "mixer.", missing) for k in ("heads", "kv_heads", "dim", "vdim", "scale", "bias_max")}
            qt = _get(m, "q_temp", w + "mixer.", missing)
            coef = _get(qt, "coef", w + "mixer.q_temp.", missing) if qt is not None else None
            every = _get(qt, "every", w + "mixer.q_temp.", missing) if qt is not None else None
            mlp = L.get("mlp") if isinstance(L, dict) else None
            mlp_kind, ff, experts, top = None, 0, 0, 0
            if mlp is not None:
                mlp_kind = _get(mlp, "kind", w + "mlp.", missing)
                if mlp_kind == "dense":
                    ff = _get(mlp, "ff", w + "mlp.", missing)
                elif mlp_kind == "moe":
                    ex, ro = _get(mlp, "expert", w + "mlp.", missing), _get(mlp, "router", w + "mlp.", missing)
                    ff = _get(ex, "ff", w + "mlp.expert.", missing) if ex is not None else None
                    experts = _get(ro, "experts", w + "mlp.router.", missing) if ro is not None else None
                    top = _get(ro, "top", w + "mlp.router.", missing) if ro is not None else None
                elif mlp_kind is not None:
                    raise ConfigError(f"{w}mlp.kind is {mlp_kind!r}; this design's feed-forwards: 'dense', 'moe'")
            if missing:
                continue
            buckets = m.get("bias_buckets")
            layers.append(VirudraLayer(
                heads=_int(vals["heads"], w + "mixer.heads"), kv_heads=_int(vals["kv_heads"], w + "mixer.kv_heads"),
                dim=_int(vals["dim"], w + "mixer.dim"), vdim=_int(vals["vdim"], w + "mixer.vdim"),
                scale=_float(vals["scale"], w + "mixer.scale"), bias_max=_int(vals["bias_max"], w + "mixer.bias_max"),
                bias_buckets=None if buckets is None else _int(buckets, w + "mixer.bias_buckets", 2),
                temp_coef=_float(coef, w + "mixer.q_temp.coef"), temp_every=_int(every, w + "mixer.q_temp.every"),
                mlp_kind=mlp_kind, ff=0 if mlp_kind is None else _int(ff, w + "mlp ff"),
                experts=_int(experts, w + "mlp.router.experts") if mlp_kind == "moe" else 0,
                top=_int(top, w + "mlp.router.top") if mlp_kind == "moe" else 0))
        if missing:
            raise ConfigError("Virudra config.json lacks required keys: " + ", ".join(missing))
        loop = d.get("loop") or {}
        cfg = cls(vocab=_int(vocab, "vocab"), width=_int(width, "width"), eps=_float(eps, "norm.eps"),
                  logit_softcap=_float(d.get("logit_softcap", 0.0), "logit_softcap"), layers=tuple(layers),
                  loop_start=_int(loop.get("start", 0), "loop.start", 0), loop_stop=_int(loop.get("stop", 0), "loop.stop", 0),
                  loop_times=_int(loop.get("times", 1), "loop.times", 1),
                  max_positions=_int(d.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions"),
                  bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.layers:
            raise ConfigError("a Virudra model needs at least one layer")
        if not (self.eps > 0.0):
            raise ConfigError(f"norm.eps must be > 0, found {self.eps}")
        if self.logit_softcap < 0.0:
            raise ConfigError(f"logit_softcap must not be negative, found {self.logit_softcap}")
        if not (0 <= self.loop_start <= self.loop_stop <= len(self.layers)):
            raise ConfigError(f"loop {self.loop_start}..{self.loop_stop} does not lie within {len(self.layers)} layers")
        for i, L in enumerate(self.layers):
            if L.heads % L.kv_heads != 0:
                raise ConfigError(f"layers[{i}]: {L.heads} query heads are not a multiple of {L.kv_heads} key heads")
            if not (L.scale > 0.0):
                raise ConfigError(f"layers[{i}]: the score scale must be positive, found {L.scale}")
            if L.mlp_kind == "moe" and not (L.top <= L.experts):
                raise ConfigError(f"layers[{i}]: top {L.top} of {L.experts} experts")
            if L.bias_buckets is not None and L.bias_max <= L.bias_buckets // 2:
                raise ConfigError(f"layers[{i}]: bias_max {L.bias_max} must exceed half of the {L.bias_buckets} buckets")

    def run_order(self) -> List[int]:
        """Layers before the loop, the looped range ``times`` times in a row, the layers behind it."""
        n = len(self.layers)
        if self.loop_stop <= self.loop_start:
            return list(range(n))
        return (list(range(self.loop_start)) + list(range(self.loop_start, self.loop_stop)) * self.loop_times
                + list(range(self.loop_stop, n)))

    def with_bias_buckets(self, buckets: List[int]) -> "VirudraConfig":
        """The same configuration with every layer's number of bias rows filled in (from the checkpoint)."""
        layers = tuple(VirudraLayer(**{**L.__dict__, "bias_buckets": int(b)}) for L, b in zip(self.layers, buckets))
        out = VirudraConfig(**{**self.__dict__, "layers": layers})
        out.validate()
        return out

    def to_dict(self) -> dict:
        layers = []
        for L in self.layers:
            mixer = {"heads": L.heads, "kv_heads": L.kv_heads, "dim": L.dim, "vdim": L.vdim, "scale": L.scale,
                     "bias_max": L.bias_max, "q_temp": {"coef": L.temp_coef, "every": L.temp_every}}
            if L.bias_buckets is not None:
                mixer["bias_buckets"] = L.bias_buckets
            mlp = None
            if L.mlp_kind == "dense":
                mlp = {"kind": "dense", "ff": L.ff}
            elif L.mlp_kind == "moe":
                mlp = {"kind": "moe", "expert": {"ff": L.ff}, "router": {"experts": L.experts, "top": L.top}}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "logit_softcap": self.logit_softcap, "layers": layers,
             "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    # ---- the model as parts ------------------------------------------------------------------
    def to_model_config(self) -> ModelConfig:
        norm = NormSpec("rmsnorm", self.width, self.eps, bias=False, gain_offset=1.0)
        layers = []
        for i, L in enumerate(self.layers):
            mixer = AttentionSpec(
                kind="attention", width=self.width, n_heads=L.heads, n_kv_heads=L.kv_heads, head_dim=L.dim,
                scale=L.scale, qkv_bias=False, out_bias=False, window=None, position=None, v_head_dim=L.vdim,
                distance_bias=DistanceBiasSpec(n_buckets=L.bias_buckets or 0, max_distance=L.bias_max),
                query_temperature=QueryTemperatureSpec(coef=L.temp_coef, every=L.temp_every))
            if L.mlp_kind == "dense":
                ff = GatedFeedForwardSpec("gated", self.width, L.ff, DENSE_ACTIVATION)
            elif L.mlp_kind == "moe":
                ff = ExpertsFeedForwardSpec("experts", self.width, L.ff, L.experts, L.top, EXPERT_ACTIVATION,
                                            router="token_table", vocab_size=self.vocab)
            else:
                ff = None
            layers.append(LayerSpec(mixer=mixer, feed_forward=ff, pre_mixer_norm=norm, post_mixer_norm=norm,
                                    pre_ff_norm=None if ff is None else norm,
                                    post_ff_norm=None if ff is None else norm, weight_prefix=f"l{i}."))
        # every run of a layer (a looped layer runs several times) keeps a cache of its own
        schedule = tuple(LayerCall(layer, run, True) for run, layer in enumerate(self.run_order()))
        eos = () if self.eos_token_id is None else (int(self.eos_token_id),)
        return ModelConfig(
            architecture=ARCHITECTURE, vocab_size=self.vocab, width=self.width, max_positions=self.max_positions,
            layers=tuple(layers), schedule=schedule, embed_position=PositionSpec("none"), final_norm=norm,
            tie_word_embeddings=False, bos_token_id=self.bos_token_id, eos_token_ids=eos, raw=self.to_dict(),
            logit_softcap=self.logit_softcap)
