"""Small Pedatar configurations for the tests, each different in every size and option, and a model folder with
random weights beside its plain implementation."""
from __future__ import annotations

import functools

import numpy as np

import plain_pedatar as P


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
            "scale": scale, "rot": {"base": base, "dims": rot_dim if dims is None else dims}}


def scan(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def moe(experts, top, ff, shared=None):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": None if shared is None else {"ff": shared}}


def att_layer(mixer, mlp, weights_of=None):
    d = {"type": "latent_attention", "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def scan_layer(mixer, mlp, weights_of=None):
    d = {"type": "mamba1", "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


# P: sizes that the matrix-core kernels take; two experts a token; layers 2 and 3 run on the weights of 0 and 1
_PA, _PS, _PM = latent(2, 16, 8, 24, 24, 40, 0.2, 10000.0), scan(96, 16, 8, 4), moe(4, 2, 32, shared=48)
CONFIG_P = {"architecture": "Pedatar", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
            "layers": [att_layer(_PA, _PM), scan_layer(_PS, _PM), att_layer(_PA, _PM, 0), scan_layer(_PS, _PM, 1)]}

# Q: a scan first; only some of the rotated entries turn; values larger than keys; ranks and widths that are no
# multiple of 8 (plain products); a state of 24 entries (two lanes a channel, one half full); two taps; every
# expert used by every token; no shared expert; a layer without a feed-forward
CONFIG_Q = {"architecture": "Pedatar", "vocab": 130, "width": 72, "norm": {"eps": 1e-6}, "embedding": {"scale": 0.5},
            "layers": [scan_layer(scan(100, 24, 3, 2), moe(3, 3, 20)),
                       att_layer(latent(3, 8, 12, 20, 18, 27, 0.3, 500.0, dims=6), None),
                       att_layer(latent(1, 32, 4, 16, 40, 16, 0.15, 10000.0, dims=4), moe(5, 1, 24, shared=16))]}

# R: the ones: one head, one expert, one tap (no filter state), one step-size number, one state entry; nothing turns
# in the second attention layer; an embedding scale of 1
CONFIG_R = {"architecture": "Pedatar", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "layers": [att_layer(latent(1, 16, 16, 16, 16, 16, 0.25, 100.0), moe(1, 1, 40)),
                       scan_layer(scan(48, 1, 1, 1), moe(6, 2, 16, shared=64)),
                       scan_layer(scan(64, 40, 2, 3), None),
                       att_layer(latent(4, 8, 8, 8, 8, 8, 0.4, 10000.0, dims=0), moe(2, 2, 8))]}


class TinyPedatar:
    def __init__(self, folder, cfg, seed):
        self.folder, self.cfg, self.seed = str(folder), cfg, seed
        self.plain_cfg, self.W = P.read_model_folder(self.folder)

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids):
        return P.forward_logits(self.plain_cfg, self.W, list(ids))

    def plain_logits(self, ids, routes=None, slack=0.0):
        """The plain model's logits [T, V]; with ``routes`` (run -> position -> experts chosen by the engine) it makes
        the engine's choices where they are as good as its own within ``slack`` (plain_pedatar.routed_ff)."""
        if routes is None:
            return self._logits(tuple(int(i) for i in ids))
        return P.forward(self.plain_cfg, self.W, list(ids), routes=routes, slack=slack)

    def prompt(self, length, salt=0):
        rng = np.random.default_rng(1000 * self.seed + 7 * length + salt)
        return [int(t) for t in rng.integers(0, self.cfg["vocab"], size=length)]


def make_model(folder, cfg, seed):
    from deliverance_amd.random_model import random_model
    random_model(str(folder), cfg, seed)
    return TinyPedatar(folder, cfg, seed)


def replay_routed(session, steps, cfg):
    """helpers.replay, and beside the logits the experts that the engine chose: {rid: {run: {position: [experts]}}}.
    The engine hands them to its layer debug hook once per run of a layer with a routed feed-forward, rows in the
    step's order (one-token entries first, then the portions, each group in the order of the entries)."""
    got, routes, at = {}, {}, {}
    seen = []
    session.runner.debug_hook = lambda layer, stage, tensor: seen.append(tensor.cpu().numpy()) if stage == "expert_choice" else None
    try:
        for s in steps:
            seen.clear()
            out = session.run_step(s)
            r = 0
            for e in s["entries"]:
                for _ in e.get("want", []):
                    got.setdefault(e["id"], []).append(out[r])
                    r += 1
            order = sorted(range(len(s["entries"])), key=lambda i: (len(s["entries"][i]["tokens"]) != 1, i))
            runs = moe_runs(cfg)
            assert len(seen) == len(runs), f"{len(seen)} routed feed-forwards reported, the model runs {len(runs)}"
            row = 0
            for i in order:
                e = s["entries"][i]
                start = at.get(e["id"], 0)
                for k, ids in enumerate(seen):
                    for j in range(len(e["tokens"])):
                        routes.setdefault(e["id"], {}).setdefault(runs[k], {})[start + j] = [int(x) for x in ids[row + j]]
                row += len(e["tokens"])
                at[e["id"]] = start + len(e["tokens"])
            for rid in s["end"]:
                at.pop(rid, None)
    finally:
        session.runner.debug_hook = None
    return {rid: np.stack(rows) for rid, rows in got.items()}, routes


def moe_runs(cfg):
    """The runs (indices into the list of layers) that have a routed feed-forward, in order."""
    return [i for i, L in enumerate(cfg["layers"]) if L.get("mlp") is not None]
