"""A plain, slow Virudra in NumPy float64: one function per mechanism, whole sequences only, no cache.
It is what the engine is compared with; it shares no code with it (the model folder is read with the
safetensors package, the formulas are written out here)."""
from __future__ import annotations

import json
import math
import os

import numpy as np


def read_model_folder(folder):
    """config.json as a dict, tensors as float64 (integer tables as int64) NumPy arrays by name."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(torch.float64).numpy() if t.dtype.is_floating_point else t.to(torch.int64).numpy()
    return cfg, tensors


# --------------------------------------------------------------------------- mechanisms
def unit_rms_norm(x, stored_gain, eps):
    """Rows scaled to a root mean square of one (eps under the root), times 1 + the stored gain."""
    ms = np.mean(np.square(x), axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * (1.0 + stored_gain)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def bias_row(distance, n_rows, far):
    """Which row of a layer's bias table a key `distance` >= 0 behind the query reads: the first half of
    the rows are exact distances, the second half is spread over ln(distance) up to `far`."""
    exact = n_rows // 2
    if distance < exact:
        return distance
    stretched = math.log(distance / exact) / math.log(far / exact) * (n_rows - exact)
    return min(n_rows - 1, exact + int(math.floor(stretched)))


def query_gain(position, coef, every):
    """What a query at `position` is multiplied by."""
    return 1.0 + coef * math.log((position + 1) // every + 1)


def attend(q, k, v, table, m):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] of one whole sequence -> [T, H, dv]: causal softmax attention
    with grouped key heads, the query gain and the bias by distance (`table` [rows, H], or None)."""
    T, H, _ = q.shape
    G, dv = k.shape[1], v.shape[2]
    gain = np.array([query_gain(p, m["q_temp"]["coef"], m["q_temp"]["every"]) for p in range(T)])
    q = q * gain[:, None, None]
    if table is not None:
        n_rows = table.shape[0]
        by_distance = np.array([bias_row(n, n_rows, m["bias_max"]) for n in range(T)])
        rows = by_distance[np.maximum(np.arange(T)[:, None] - np.arange(T)[None, :], 0)]
    hidden = np.triu(np.ones((T, T), dtype=bool), 1)
    out = np.zeros((T, H, dv))
    for head in range(H):
        g = head // (H // G)
        s = q[:, head] @ k[:, g].T * m["scale"]
        if table is not None:
            s = s + table[rows, head]
        s = np.where(hidden, -np.inf, s)
        s = s - s.max(axis=-1, keepdims=True)
        wgt = np.exp(s)
        wgt /= wgt.sum(axis=-1, keepdims=True)
        out[:, head] = wgt @ v[:, g]
    return out


def attention(h, Wq, Wk, Wv, Wo, table, m):
    """The mixer over a whole sequence h [T, E]; `m` is the layer's "mixer" record of config.json."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    out = attend((h @ Wq.T).reshape(T, H, dk), (h @ Wk.T).reshape(T, G, dk), (h @ Wv.T).reshape(T, G, dv), table, m)
    return out.reshape(T, H * dv) @ Wo.T


def gated_ff(h, Wg, Wu, Wd, act):
    return (act(h @ Wg.T) * (h @ Wu.T)) @ Wd.T


def experts_ff(h, ids, table, W, prefix):
    """Every token's experts are the entries of row `token id` of `table`; equal weights."""
    top = table.shape[1]
    y = np.zeros_like(h)
    for t, tok in enumerate(ids):
        for e in table[tok]:
            p = f"{prefix}e{int(e)}."
            y[t] += gated_ff(h[t:t + 1], W[p + "gate"], W[p + "up"], W[p + "down"], silu)[0] / top
    return y


def layer_runs(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return list(range(n))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, n))


def softcap(z, cap):
    return cap * np.tanh(z / cap) if cap else z


# --------------------------------------------------------------------------- the model
def forward_logits(cfg, W, ids, streams=None):
    """[T, vocab] logits of a whole sequence; `streams` (a list) receives the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(ids)]
    for li in layer_runs(cfg):
        L, p = cfg["layers"][li], f"l{li}."
        y = attention(unit_rms_norm(x, W[p + "norm1"], eps), W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"], W[p + "mix.o"],
                      W[p + "mix.rel"], L["mixer"])
        x = x + unit_rms_norm(y, W[p + "norm1b"], eps)
        if L.get("mlp") is not None:
            h = unit_rms_norm(x, W[p + "norm2"], eps)
            if L["mlp"]["kind"] == "dense":
                y = gated_ff(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"], gelu_tanh)
            else:
                y = experts_ff(h, ids, W[p + "mlp.table"], W, p + "mlp.")
            x = x + unit_rms_norm(y, W[p + "norm2b"], eps)
        if streams is not None:
            streams.append(x.copy())
    return softcap(unit_rms_norm(x, W["final.norm"], eps) @ W["head"].T, cfg.get("logit_softcap", 0.0))


def greedy_generate(cfg, W, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(np.argmax(forward_logits(cfg, W, ids)[-1])))
    return ids[len(prompt):]
