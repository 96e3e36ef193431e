"""A plain, slow Pedatar in NumPy float64: one function per mechanism, whole sequences only, no cache and no
state kept between calls.  It is what the engine is compared with; it shares no code with it (the model folder
is read with the safetensors package, the formulas are written out here)."""
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


# --------------------------------------------------------------------------- small functions
def unit_rms(x, gain, eps):
    """Rows scaled to a root mean square of one (eps under the root), times the gain."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps) * gain


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def swish(z):
    return z * logistic(z)


def soft_plus(z):
    return np.logaddexp(0.0, z)


def squared_ramp(z):
    return np.square(np.maximum(z, 0.0))


# --------------------------------------------------------------------------- rotation
def turn_pairs(v, places, n_turned, base):
    """v [T, ..., d]: neighbours (2i, 2i + 1) of the first ``n_turned`` entries are turned by the angle
    place * base^(-2i / n_turned); what lies behind them passes."""
    out = v.copy()
    half = n_turned // 2
    speed = base ** (-2.0 * np.arange(half) / n_turned)
    ang = np.asarray(places, dtype=np.float64)[:, None] * speed[None, :]          # [T, half]
    shape = (len(places),) + (1,) * (v.ndim - 2) + (half,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    a, b = v[..., 0:n_turned:2], v[..., 1:n_turned:2]
    out[..., 0:n_turned:2] = a * c - b * s
    out[..., 1:n_turned:2] = b * c + a * s
    return out


# --------------------------------------------------------------------------- mixers
def latent_attention(W, p, m, h, eps):
    """h [T, E] of one whole sequence -> [T, E].  Queries pass a narrow normalised vector; keys and values are
    unfolded per head from one narrow normalised vector a token, beside which one turned key piece is shared
    by all heads."""
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    places = np.arange(T)
    cq = unit_rms(h @ W[p + "mix.dq"].T, W[p + "mix.dq.norm"], eps)
    q = (cq @ W[p + "mix.uq"].T).reshape(T, H, dn + dr)
    q_flat, q_turn = q[..., :dn], turn_pairs(q[..., dn:], places, rot["dims"], rot["base"])
    down = h @ W[p + "mix.dkv"].T
    c = unit_rms(down[:, :r], W[p + "mix.dkv.norm"], eps)
    k_turn = turn_pairs(down[:, r:], places, rot["dims"], rot["base"])           # [T, dr], one for all heads
    k_flat = (c @ W[p + "mix.uk"].T).reshape(T, H, dn)
    val = (c @ W[p + "mix.uv"].T).reshape(T, H, dv)
    hidden = np.triu(np.ones((T, T), dtype=bool), 1)
    out = np.zeros((T, H, dv))
    for head in range(H):
        s = (q_flat[:, head] @ k_flat[:, head].T + q_turn[:, head] @ k_turn.T) * m["scale"]
        s = np.where(hidden, -np.inf, s)
        s = s - s.max(axis=-1, keepdims=True)
        wgt = np.exp(s)
        wgt /= wgt.sum(axis=-1, keepdims=True)
        out[:, head] = wgt @ val[:, head]
    return out.reshape(T, H * dv) @ W[p + "mix.o"].T


def short_filter(x, taps, bias):
    """x [T, C], taps [C, K]: y[t, c] = bias[c] + sum_k taps[c, k] * x[t - (K - 1 - k), c], zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), x], axis=0)
    y = np.tile(bias[None, :], (T, 1))
    for k in range(K):
        y += padded[k:k + T] * taps[:, k][None, :]
    return y


def selective_scan(x, step, A, B, C, D):
    """x, step [T, I]; A [I, N]; B, C [T, N]; D [I].  S_t = exp(step_t A) * S_{t-1} + step_t x_t B_t (outer
    product over channel and state index), y_t = S_t C_t + D x_t.  The state starts at zero."""
    T, I = x.shape
    S = np.zeros_like(A)
    y = np.zeros((T, I))
    for t in range(T):
        S = np.exp(step[t][:, None] * A) * S + (step[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y


def mamba1(W, p, m, h):
    inner, n, rk = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[p + "mix.in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = swish(short_filter(x, W[p + "mix.conv"], W[p + "mix.conv.b"]))
    proj = x @ W[p + "mix.x"].T
    low, B, C = proj[:, :rk], proj[:, rk:rk + n], proj[:, rk + n:rk + 2 * n]
    step = soft_plus(low @ W[p + "mix.dt"].T + W[p + "mix.dt.b"])
    y = selective_scan(x, step, -np.exp(W[p + "mix.A_log"]), B, C, W[p + "mix.D"])
    return (y * swish(z)) @ W[p + "mix.o"].T


# --------------------------------------------------------------------------- feed-forward
def small_ff(W, p, h):
    return squared_ramp(h @ W[p + "up"].T) @ W[p + "down"].T


class FarChoice(AssertionError):
    """A choice of experts that was handed in ranks far below the ones this implementation makes."""


def routed_ff(W, p, mlp, h, given=None, slack=0.0):
    """Every token's ``top`` best experts by logistic(router h); an expert sees the token times its score; a
    shared expert sees every token as it is.  ``given[t]`` (optional) are experts that someone else chose for
    token t: they are used instead of the best ones, provided that each of them lies within ``slack`` (a fraction
    of the largest router logit's size) of the last place among the best; else FarChoice is raised.  A reduced
    number format may rank two experts of nearly equal score the other way round, and everything behind such a
    choice can only be compared when both sides make the same one."""
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[p + "mlp.router"].T
    score = logistic(z)                                                  # [T, n]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        best = np.argsort(-score[t], kind="stable")[:top]
        if given is not None and set(int(e) for e in given[t]) != set(int(e) for e in best):
            theirs = [int(e) for e in given[t]]
            edge = z[t, best[-1]]
            if len(set(theirs)) != top or any(z[t, e] < edge - slack * np.abs(z[t]).max() for e in theirs):
                raise FarChoice(f"{p} token {t}: experts {sorted(theirs)} were chosen, the best are {sorted(int(e) for e in best)} "
                                f"(router logits {np.round(z[t], 4).tolist()})")
            best = theirs
        for e in best:
            out[t] += small_ff(W, f"{p}mlp.e{int(e)}.", score[t, e] * h[t][None, :])[0]
    if mlp.get("shared") is not None:
        out += small_ff(W, p + "mlp.shared.", h)
    return out


def router_margin(W, p, mlp, h):
    """How far the last chosen expert's score lies above the best one that was left out, per token."""
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    if top >= n:
        return np.full(h.shape[0], np.inf)
    score = np.sort(logistic(h @ W[p + "mlp.router"].T), axis=-1)[:, ::-1]
    return score[:, top - 1] - score[:, top]


# --------------------------------------------------------------------------- the model
def layer_runs(cfg):
    """(entry of config 'layers', prefix of the tensors it uses) in the order the layers run."""
    for i, L in enumerate(cfg["layers"]):
        yield L, f"l{L.get('weights_of', i)}."


def forward(cfg, W, ids, with_layers=False, with_margins=False, routes=None, slack=0.0):
    """Logits [T, V] of one whole sequence; with_layers: also the stream after every layer [runs, T, E];
    with_margins: also the smallest router margin met.  ``routes[run][t]``: experts chosen elsewhere for token t in
    the run-th layer (see routed_ff)."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(ids, dtype=np.int64)] * cfg["embedding"]["scale"]
    after, margin = [], np.inf
    for run, (L, p) in enumerate(layer_runs(cfg)):
        h = unit_rms(x, W[p + "norm1"], eps)
        if L["type"] == "latent_attention":
            x = x + latent_attention(W, p, L["mixer"], h, eps)
        elif L["type"] == "mamba1":
            x = x + mamba1(W, p, L["mixer"], h)
        else:
            raise ValueError(f"unknown mixer {L['type']!r}")
        if L.get("mlp") is not None:
            h = unit_rms(x, W[p + "norm2"], eps)
            if with_margins:
                margin = min(margin, float(router_margin(W, p, L["mlp"], h).min()))
            x = x + routed_ff(W, p, L["mlp"], h, None if routes is None else routes.get(run), slack)
        after.append(x.copy())
    logits = unit_rms(x, W["final.norm"], eps) @ W["head"].T
    out = (logits,)
    if with_layers:
        out += (np.stack(after),)
    if with_margins:
        out += (margin,)
    return out[0] if len(out) == 1 else out


def forward_logits(cfg, W, ids):
    return forward(cfg, W, ids)
