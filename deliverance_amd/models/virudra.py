"""Virudra: which checkpoint tensors feed which part.

Names: ``embed``, ``head``, ``final.norm``; per layer ``l<i>.norm1``, ``norm1b`` (in front of and behind the
mixer), ``norm2``, ``norm2b`` (the feed-forward), ``l<i>.mix.{q,k,v,o,rel}``, and ``l<i>.mlp.{gate,up,down}``
or ``l<i>.mlp.e<j>.{gate,up,down}`` with ``l<i>.mlp.table``.  Linear weights are stored [out, in].  The
three projections of a mixer become one q | k | v matrix, gate and up one matrix, and the experts of a layer
one stack, at load time.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.specs import ConfigError, ExpertsFeedForwardSpec, GatedFeedForwardSpec, ModelConfig
from ..config.virudra import ARCHITECTURE, VirudraConfig
from ..registry import Architecture, ModelSupport
from ..weights.loader import TensorDecl

# Random-weights distributions: matrices N(0, 0.05), norm gains (stored around zero) N(0, 0.1), the
# distance-bias table N(0, 0.5), expert tables rows of distinct integers.
W_STD, GAIN_STD, BIAS_STD = 0.05, 0.1, 0.5


def read_config(d: dict) -> ModelConfig:
    return VirudraConfig.from_dict(d).to_model_config()


def declare_tensors(mc: ModelConfig) -> List[TensorDecl]:
    E, V = mc.width, mc.vocab_size
    out = [TensorDecl("embed", (V, E), "normal", 1.0)]
    for spec in mc.layers:
        p, a, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        # the rows of the bias table are the checkpoint's to say (-1) unless the configuration names them
        buckets = a.distance_bias.n_buckets or -1
        out += [TensorDecl(p + "norm1", (E,), "normal", GAIN_STD), TensorDecl(p + "norm1b", (E,), "normal", GAIN_STD),
                TensorDecl(p + "mix.q", (a.n_heads * a.head_dim, E), "normal", W_STD),
                TensorDecl(p + "mix.k", (a.n_kv_heads * a.head_dim, E), "normal", W_STD),
                TensorDecl(p + "mix.v", (a.n_kv_heads * a.value_dim, E), "normal", W_STD),
                TensorDecl(p + "mix.rel", (buckets, a.n_heads), "normal", BIAS_STD),
                TensorDecl(p + "mix.o", (E, a.n_heads * a.value_dim), "normal", W_STD)]
        if f is None:
            continue
        out += [TensorDecl(p + "norm2", (E,), "normal", GAIN_STD), TensorDecl(p + "norm2b", (E,), "normal", GAIN_STD)]
        if isinstance(f, GatedFeedForwardSpec):
            out += [TensorDecl(p + "mlp.gate", (f.inner, E), "normal", W_STD),
                    TensorDecl(p + "mlp.up", (f.inner, E), "normal", W_STD),
                    TensorDecl(p + "mlp.down", (E, f.inner), "normal", W_STD)]
        elif isinstance(f, ExpertsFeedForwardSpec):
            for j in range(f.n_experts):
                out += [TensorDecl(f"{p}mlp.e{j}.gate", (f.inner, E), "normal", W_STD),
                        TensorDecl(f"{p}mlp.e{j}.up", (f.inner, E), "normal", W_STD),
                        TensorDecl(f"{p}mlp.e{j}.down", (E, f.inner), "normal", W_STD)]
            out.append(TensorDecl(p + "mlp.table", (V, f.top), "distinct_ints", float(f.n_experts)))
    out += [TensorDecl("final.norm", (E,), "normal", GAIN_STD), TensorDecl("head", (V, E), "normal", W_STD)]
    return out


def bind_tensors(mc: ModelConfig, t: dict) -> dict:
    layers = []
    for spec in mc.layers:
        p, f = spec.weight_prefix, spec.feed_forward
        d = {"pre_mixer_norm": {"weight": t[p + "norm1"]}, "post_mixer_norm": {"weight": t[p + "norm1b"]},
             "mixer": {"qkv_weight": torch.cat([t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"]], dim=0),
                       "out_weight": t[p + "mix.o"], "distance_bias": t[p + "mix.rel"]}}
        if f is not None:
            d["pre_ff_norm"] = {"weight": t[p + "norm2"]}
            d["post_ff_norm"] = {"weight": t[p + "norm2b"]}
            if isinstance(f, GatedFeedForwardSpec):
                d["feed_forward"] = {"gate_up_weight": torch.cat([t[p + "mlp.gate"], t[p + "mlp.up"]], dim=0),
                                     "down_weight": t[p + "mlp.down"]}
            else:
                table = t[p + "mlp.table"]
                if table.dtype != torch.int32:
                    raise ConfigError(f"{p}mlp.table must hold integers, found {table.dtype}")
                d["feed_forward"] = {
                    "gate_up_weight": torch.stack([torch.cat([t[f"{p}mlp.e{j}.gate"], t[f"{p}mlp.e{j}.up"]], dim=0)
                                                   for j in range(f.n_experts)]),
                    "down_weight": torch.stack([t[f"{p}mlp.e{j}.down"] for j in range(f.n_experts)]),
                    "table": table}
        layers.append(d)
    return {"embed": {"tokens": t["embed"]}, "layers": layers, "final_norm": {"weight": t["final.norm"]},
            "head": {"weight": t["head"]}}


VIRUDRA = Architecture(name=ARCHITECTURE, read_config=read_config, declare_tensors=declare_tensors,
                       bind_tensors=bind_tensors, aliases=("virudra",))
ModelSupport.add_model(VIRUDRA)
