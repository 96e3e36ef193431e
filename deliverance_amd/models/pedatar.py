"""Pedatar: which checkpoint tensors feed which part.

Names: ``embed``, ``head``, ``final.norm``; per layer with tensors of its own ``l<i>.norm1``, ``l<i>.norm2``;
a latent-attention mixer ``l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, o}``; a scan mixer
``l<i>.mix.{in, conv, conv.b, x, dt, dt.b, A_log, D, o}``; a feed-forward ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.{up, down}`` and ``l<i>.mlp.shared.{up, down}``.  Linear weights are stored [out, in].  The
experts of a layer become one stack at load time.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.pedatar import ARCHITECTURE, PedatarConfig
from ..config.specs import LatentAttentionSpec, ModelConfig, SelectiveScanSpec
from ..registry import Architecture, ModelSupport
from ..weights.loader import TensorDecl

# Random-weights distributions: matrices N(0, 0.05), norm gains 1 + N(0, 0.1), the scan's step bias N(0, 0.5),
# its A_log N(0, 0.5), D and the filter's bias N(0, 0.3), the filter's taps N(0, 0.4).
W_STD, GAIN_STD = 0.05, 0.1


def read_config(d: dict) -> ModelConfig:
    return PedatarConfig.from_dict(d).to_model_config()


def declare_tensors(mc: ModelConfig) -> List[TensorDecl]:
    E, V = mc.width, mc.vocab_size
    out = [TensorDecl("embed", (V, E), "normal", 0.3)]
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        out.append(TensorDecl(p + "norm1", (E,), "ones_plus_normal", GAIN_STD))
        if isinstance(m, LatentAttentionSpec):
            H = m.n_heads
            out += [TensorDecl(p + "mix.dq", (m.q_rank, E), "normal", W_STD),
                    TensorDecl(p + "mix.dq.norm", (m.q_rank,), "ones_plus_normal", GAIN_STD),
                    TensorDecl(p + "mix.uq", (H * (m.head_dim + m.rot_dim), m.q_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.dkv", (m.kv_rank + m.rot_dim, E), "normal", W_STD),
                    TensorDecl(p + "mix.dkv.norm", (m.kv_rank,), "ones_plus_normal", GAIN_STD),
                    TensorDecl(p + "mix.uk", (H * m.head_dim, m.kv_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.uv", (H * m.v_head_dim, m.kv_rank), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.o", (E, H * m.v_head_dim), "normal", W_STD)]
        elif isinstance(m, SelectiveScanSpec):
            out += [TensorDecl(p + "mix.in", (2 * m.inner, E), "normal", W_STD),
                    TensorDecl(p + "mix.conv", (m.inner, m.conv_taps), "normal", 0.4),
                    TensorDecl(p + "mix.conv.b", (m.inner,), "normal", 0.3),
                    TensorDecl(p + "mix.x", (m.dt_rank + 2 * m.state, m.inner), "normal", 2 * W_STD),
                    TensorDecl(p + "mix.dt", (m.inner, m.dt_rank), "normal", 4 * W_STD),
                    TensorDecl(p + "mix.dt.b", (m.inner,), "normal", 0.5),
                    TensorDecl(p + "mix.A_log", (m.inner, m.state), "normal", 0.5),
                    TensorDecl(p + "mix.D", (m.inner,), "normal", 0.3),
                    TensorDecl(p + "mix.o", (E, m.inner), "normal", W_STD)]
        else:
            raise TypeError(f"no tensors are known for a mixer of kind {getattr(m, 'kind', m)!r}")
        if f is None:
            continue
        out.append(TensorDecl(p + "norm2", (E,), "ones_plus_normal", GAIN_STD))
        for j in range(f.n_experts):
            out += [TensorDecl(f"{p}mlp.e{j}.up", (f.inner, E), "normal", 2 * W_STD),
                    TensorDecl(f"{p}mlp.e{j}.down", (E, f.inner), "normal", 2 * W_STD)]
        out.append(TensorDecl(p + "mlp.router", (f.n_experts, E), "normal", 4 * W_STD))
        if f.shared_inner:
            out += [TensorDecl(p + "mlp.shared.up", (f.shared_inner, E), "normal", W_STD),
                    TensorDecl(p + "mlp.shared.down", (E, f.shared_inner), "normal", W_STD)]
    out += [TensorDecl("final.norm", (E,), "ones_plus_normal", GAIN_STD), TensorDecl("head", (V, E), "normal", W_STD)]
    return out


def bind_tensors(mc: ModelConfig, t: dict) -> dict:
    layers = []
    for spec in mc.layers:
        p, m, f = spec.weight_prefix, spec.mixer, spec.feed_forward
        d = {"pre_mixer_norm": {"weight": t[p + "norm1"]}}
        if isinstance(m, LatentAttentionSpec):
            d["mixer"] = {"q_down_weight": t[p + "mix.dq"], "q_norm_weight": t[p + "mix.dq.norm"],
                          "q_up_weight": t[p + "mix.uq"], "kv_down_weight": t[p + "mix.dkv"],
                          "kv_norm_weight": t[p + "mix.dkv.norm"], "k_up_weight": t[p + "mix.uk"],
                          "v_up_weight": t[p + "mix.uv"], "out_weight": t[p + "mix.o"]}
        else:
            d["mixer"] = {"in_weight": t[p + "mix.in"], "conv_weight": t[p + "mix.conv"], "conv_bias": t[p + "mix.conv.b"],
                          "x_weight": t[p + "mix.x"], "dt_weight": t[p + "mix.dt"], "dt_bias": t[p + "mix.dt.b"],
                          "a_log": t[p + "mix.A_log"], "d": t[p + "mix.D"], "out_weight": t[p + "mix.o"]}
        if f is not None:
            d["pre_ff_norm"] = {"weight": t[p + "norm2"]}
            ff = {"up_weight": torch.stack([t[f"{p}mlp.e{j}.up"] for j in range(f.n_experts)]),
                  "down_weight": torch.stack([t[f"{p}mlp.e{j}.down"] for j in range(f.n_experts)]),
                  "router_weight": t[p + "mlp.router"]}
            if f.shared_inner:
                ff["shared_up_weight"], ff["shared_down_weight"] = t[p + "mlp.shared.up"], t[p + "mlp.shared.down"]
            d["feed_forward"] = ff
        layers.append(d)
    return {"embed": {"tokens": t["embed"]}, "layers": layers, "final_norm": {"weight": t["final.norm"]},
            "head": {"weight": t["head"]}}


PEDATAR = Architecture(name=ARCHITECTURE, read_config=read_config, declare_tensors=declare_tensors,
                       bind_tensors=bind_tensors, aliases=("pedatar",))
ModelSupport.add_model(PEDATAR)
