"""Typed Pedatar configuration, read from the design's own config.json keys.

A Pedatar model is a list of layers; each has one mixer (attention over a narrow latent vector, or a selective
state-space scan) behind a root-mean-square norm, and a mixture-of-experts feed-forward (or none) behind another.
A layer may use another layer's weights (norms, mixer, feed-forward) while keeping a cache or state of its own.
config.json::

    {"architecture": "Pedatar", "vocab": V, "width": E, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "latent_attention",
                 "mixer": {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale",
                           "rot": {"base", "dims"}},
                 "mlp": null | {"kind": "moe", "expert": {"ff": F}, "router": {"experts": n, "top": k},
                                "shared": null | {"ff": Fs}},
                 "weights_of": j (optional)},
                {"type": "mamba1", "mixer": {"inner", "state", "dt_rank", "conv"}, "mlp": ...}, ...]}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

from .specs import (ConfigError, ExpertsFeedForwardSpec, LatentAttentionSpec, LayerCall, LayerSpec, ModelConfig,
                    NormSpec, PositionSpec, RotarySpec, SelectiveScanSpec)

ARCHITECTURE = "Pedatar"
# The design has no position limit of its own (positions enter through angles only): requests are bounded by
# the cache.  This is what the scheduler and the step function check against.
DEFAULT_MAX_POSITIONS = 1 << 20
EXPERT_ACTIVATION = "relu2"         # the design fixes it: the square of max(x, 0), for experts and the shared one
MIXERS = ("latent_attention", "mamba1")


def _get(d, key: str, where: str, missing: List[str]):
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
class PedatarFeedForward:
    ff: int
    experts: int
    top: int
    shared_ff: int = 0              # 0: no shared expert


@dataclass(frozen=True)
class PedatarLayer:
    kind: str                       # "latent_attention" | "mamba1"
    mixer: Tuple[Tuple[str, float], ...]      # the mixer's sizes and constants by their config names
    mlp: Optional[PedatarFeedForward]
    weights_of: Optional[int] = None          # the layer whose tensors this one uses (None: its own)

    def m(self, key: str):
        return dict(self.mixer)[key]


_ATT_INTS = ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank")
_SCAN_INTS = ("inner", "state", "dt_rank", "conv")


@dataclass(frozen=True)
class PedatarConfig:
    vocab: int
    width: int
    eps: float
    embed_scale: float
    layers: Tuple[PedatarLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: dict) -> "PedatarConfig":
        missing: List[str] = []
        vocab, width = _get(d, "vocab", "", missing), _get(d, "width", "", missing)
        norm = _get(d, "norm", "", missing)
        eps = _get(norm, "eps", "norm.", missing) if norm is not None else None
        emb = _get(d, "embedding", "", missing)
        scale = _get(emb, "scale", "embedding.", missing) if emb is not None else None
        raw_layers = _get(d, "layers", "", missing)
        layers: List[PedatarLayer] = []
        for i, L in enumerate(raw_layers or []):
            w = f"layers[{i}]."
            kind = _get(L, "type", w, missing)
            if kind is not None and kind not in MIXERS:
                raise ConfigError(f"{w}type is {kind!r}; this design's mixers: {', '.join(repr(k) for k in MIXERS)}")
            m = _get(L, "mixer", w, missing)
            if kind is None or m is None:
                continue
            n0 = len(missing)
            vals = {}
            if kind == "latent_attention":
                for k in _ATT_INTS:
                    vals[k] = _get(m, k, w + "mixer.", missing)
                vals["scale"] = _get(m, "scale", w + "mixer.", missing)
                rot = _get(m, "rot", w + "mixer.", missing)
                vals["rot.base"] = _get(rot, "base", w + "mixer.rot.", missing) if rot is not None else None
                vals["rot.dims"] = _get(rot, "dims", w + "mixer.rot.", missing) if rot is not None else None
            else:
                for k in _SCAN_INTS:
                    vals[k] = _get(m, k, w + "mixer.", missing)
            mlp = L.get("mlp") if isinstance(L, dict) else None
            ff = None
            if mlp is not None:
                mk = _get(mlp, "kind", w + "mlp.", missing)
                if mk is not None and mk != "moe":
                    raise ConfigError(f"{w}mlp.kind is {mk!r}; this design's feed-forward: 'moe'")
                ex, ro = _get(mlp, "expert", w + "mlp.", missing), _get(mlp, "router", w + "mlp.", missing)
                f = _get(ex, "ff", w + "mlp.expert.", missing) if ex is not None else None
                n = _get(ro, "experts", w + "mlp.router.", missing) if ro is not None else None
                top = _get(ro, "top", w + "mlp.router.", missing) if ro is not None else None
                sh = mlp.get("shared") if isinstance(mlp, dict) else None
                sf = _get(sh, "ff", w + "mlp.shared.", missing) if sh is not None else 0
                if len(missing) == n0:
                    ff = PedatarFeedForward(ff=_int(f, w + "mlp.expert.ff"), experts=_int(n, w + "mlp.router.experts"),
                                            top=_int(top, w + "mlp.router.top"),
                                            shared_ff=_int(sf, w + "mlp.shared.ff") if sh is not None else 0)
            if len(missing) > n0:
                continue
            mixer = []
            for k, v in vals.items():
                if k in ("scale", "rot.base"):
                    mixer.append((k, _float(v, w + "mixer." + k)))
                else:
                    mixer.append((k, _int(v, w + "mixer." + k, 0 if k == "rot.dims" else 1)))
            wo = L.get("weights_of")
            layers.append(PedatarLayer(kind=kind, mixer=tuple(mixer), mlp=ff,
                                       weights_of=None if wo is None else _int(wo, w + "weights_of", 0)))
        if missing:
            raise ConfigError("Pedatar config.json lacks required keys: " + ", ".join(missing))
        cfg = cls(vocab=_int(vocab, "vocab"), width=_int(width, "width"), eps=_float(eps, "norm.eps"),
                  embed_scale=_float(scale, "embedding.scale"), layers=tuple(layers),
                  max_positions=_int(d.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions"),
                  bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"))
        cfg.validate()
        return cfg

    def owner(self, i: int) -> int:
        """The layer whose tensors layer ``i`` uses (itself, or the end of its ``weights_of`` chain)."""
        seen = set()
        while self.layers[i].weights_of is not None:
            if i in seen:
                raise ConfigError(f"layers[{i}].weights_of runs in a circle")
            seen.add(i)
            i = self.layers[i].weights_of
        return i

    def validate(self) -> None:
        if not self.layers:
            raise ConfigError("a Pedatar model needs at least one layer")
        if not (self.eps > 0.0):
            raise ConfigError(f"norm.eps must be > 0, found {self.eps}")
        for i, L in enumerate(self.layers):
            if L.weights_of is not None:
                if not (0 <= L.weights_of < len(self.layers)) or L.weights_of == i:
                    raise ConfigError(f"layers[{i}].weights_of names layer {L.weights_of}")
                o = self.layers[self.owner(i)]
                if (o.kind, o.mixer, o.mlp) != (L.kind, L.mixer, L.mlp):
                    raise ConfigError(f"layers[{i}] uses the weights of layer {self.owner(i)} but differs from it")
            if L.kind == "latent_attention":
                if not (L.m("scale") > 0.0):
                    raise ConfigError(f"layers[{i}]: the score scale must be positive, found {L.m('scale')}")
                if L.m("rot.dims") % 2 != 0 or L.m("rot.dims") > L.m("rot_dim"):
                    raise ConfigError(f"layers[{i}]: rot.dims {L.m('rot.dims')} must be even and at most rot_dim {L.m('rot_dim')}")
                if not (L.m("rot.base") > 0.0):
                    raise ConfigError(f"layers[{i}]: rot.base must be positive")
            if L.mlp is not None and L.mlp.top > L.mlp.experts:
                raise ConfigError(f"layers[{i}]: top {L.mlp.top} of {L.mlp.experts} experts")

    def to_dict(self) -> dict:
        layers = []
        for L in self.layers:
            if L.kind == "latent_attention":
                mixer = {k: L.m(k) for k in _ATT_INTS}
                mixer["scale"] = L.m("scale")
                mixer["rot"] = {"base": L.m("rot.base"), "dims": L.m("rot.dims")}
            else:
                mixer = {k: L.m(k) for k in _SCAN_INTS}
            mlp = None
            if L.mlp is not None:
                mlp = {"kind": "moe", "expert": {"ff": L.mlp.ff}, "router": {"experts": L.mlp.experts, "top": L.mlp.top},
                       "shared": {"ff": L.mlp.shared_ff} if L.mlp.shared_ff else None}
            entry = {"type": L.kind, "mixer": mixer, "mlp": mlp}
            if L.weights_of is not None:
                entry["weights_of"] = L.weights_of
            layers.append(entry)
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "embedding": {"scale": self.embed_scale}, "layers": layers}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    # ---- the model as parts ------------------------------------------------------------------
    def to_model_config(self) -> ModelConfig:
        norm = NormSpec("rmsnorm", self.width, self.eps, bias=False, gain_offset=0.0)
        specs, index_of = [], {}
        for i, L in enumerate(self.layers):
            if L.weights_of is not None:
                continue
            if L.kind == "latent_attention":
                mixer = LatentAttentionSpec(
                    kind="latent_attention", width=self.width, n_heads=L.m("heads"), head_dim=L.m("dim"),
                    rot_dim=L.m("rot_dim"), v_head_dim=L.m("vdim"), q_rank=L.m("q_rank"), kv_rank=L.m("kv_rank"),
                    scale=L.m("scale"), norm_eps=self.eps,
                    rotary=RotarySpec("rotary", dims=L.m("rot.dims"), base=L.m("rot.base"), interleaved=True))
            else:
                mixer = SelectiveScanSpec(kind="selective_scan", width=self.width, inner=L.m("inner"), state=L.m("state"),
                                          dt_rank=L.m("dt_rank"), conv_taps=L.m("conv"))
            ff = None
            if L.mlp is not None:
                ff = ExpertsFeedForwardSpec("experts", self.width, L.mlp.ff, L.mlp.experts, L.mlp.top, EXPERT_ACTIVATION,
                                            router="logistic_top", gated=False, weight_on="input", renormalize=False,
                                            shared_inner=L.mlp.shared_ff, shared_activation=EXPERT_ACTIVATION)
            index_of[i] = len(specs)
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, pre_mixer_norm=norm,
                                   pre_ff_norm=None if ff is None else norm, weight_prefix=f"l{i}."))
        # every layer of the list runs once, with a cache slot or state of its own, on its owner's weights
        schedule = tuple(LayerCall(index_of[self.owner(i)], i, True) for i in range(len(self.layers)))
        eos = () if self.eos_token_id is None else (int(self.eos_token_id),)
        return ModelConfig(
            architecture=ARCHITECTURE, vocab_size=self.vocab, width=self.width, max_positions=self.max_positions,
            layers=tuple(specs), schedule=schedule, embed_position=PositionSpec("none"), final_norm=norm,
            tie_word_embeddings=False, bos_token_id=self.bos_token_id, eos_token_ids=eos, raw=self.to_dict(),
            embed_scale=self.embed_scale)
