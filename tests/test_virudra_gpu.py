"""Virudra on the engine against the plain implementation (tests/plain_virudra.py): each mechanism alone
through its kernels and parts, then whole models through the step function (whole prompts, decoding token by
token, portions down to two tokens, mixed batches over a small pool whose pages come back and go out again),
and greedy generation through the engine's entry point and scheduler.  Sizes differ from test to test; where
random numbers would hide a fault (one far key among hundreds, the edge of a bias row) the inputs are made so
that it shows."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_virudra as P
from helpers import quick
from virudra_models import CONFIG_X, CONFIG_Y, CONFIG_Z, make_model

pytestmark = pytest.mark.gpu
DEV = helpers.DEVICE
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def bf16(a):
    """What bfloat16 keeps of an array (as float64)."""
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def dev(a, dtype=torch.int32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


# ------------------------------------------------------------------------------------------ norms
@pytest.mark.parametrize("E", [quick(64), 203, quick(1536), 4100])
@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
def test_rms_norm_kernels(E, out_dtype):
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(E)
    R = 9
    x = rng.normal(size=(R, E)) * 3
    wa, wb = bf16(rng.normal(size=E) * 0.2), bf16(rng.normal(size=E) * 0.2)
    src = rng.normal(size=(R, E)) * 0.01          # small rows: eps matters
    eps, tol = 1e-5, (3e-6 if out_dtype == "float32" else 2.0 ** -7)
    xd, wad, wbd = dev(x, torch.float32), dev(wa, torch.bfloat16), dev(wb, torch.float32)
    out = torch.empty(R, E, dtype=DTYPES[out_dtype], device=DEV)
    ops.rmsnorm(xd, wad, 1.0, eps, out)
    want = P.unit_rms_norm(x.astype(np.float32).astype(np.float64), wa, eps)
    assert np.abs(out.double().cpu().numpy() - want).max() <= tol * np.abs(want).max()
    rows = [7, 0, 7, 3]
    got = ops.rmsnorm(xd, wad, 1.0, eps, torch.empty(4, E, dtype=DTYPES[out_dtype], device=DEV), dev(rows))
    assert np.abs(got.double().cpu().numpy() - want[rows]).max() <= tol * np.abs(want).max()
    # a gain that is stored as it is applied (offset 0)
    got = ops.rmsnorm(xd, wbd, 0.0, eps, torch.empty(R, E, dtype=torch.float32, device=DEV))
    want0 = P.unit_rms_norm(x.astype(np.float32).astype(np.float64), wb.astype(np.float32) - 1.0, eps)
    assert np.abs(got.double().cpu().numpy() - want0).max() <= 3e-6 * np.abs(want0).max()
    # the norm behind a part, the addition and the next norm in one pass
    stream = dev(x, torch.float32)
    h = torch.empty(R, E, dtype=DTYPES[out_dtype], device=DEV)
    ops.rmsnorm_add(dev(src, torch.float32), wad, stream, 1.0, eps, wbd, h)
    x32, s32 = x.astype(np.float32).astype(np.float64), src.astype(np.float32).astype(np.float64)
    new = x32 + P.unit_rms_norm(s32, wa, eps)
    assert np.abs(stream.double().cpu().numpy() - new).max() <= 3e-6 * np.abs(new).max()
    want_h = P.unit_rms_norm(new, wb.astype(np.float32).astype(np.float64), eps)
    assert np.abs(h.double().cpu().numpy() - want_h).max() <= tol * np.abs(want_h).max()
    stream2 = dev(x, torch.float32)
    ops.rmsnorm_add(dev(src, torch.float32), wad, stream2, 1.0, eps)
    assert torch.equal(stream2, stream)


def test_softcap_and_gated_activation():
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(3)
    z = rng.normal(size=(5, 77)) * 40
    got = ops.softcap(dev(z, torch.float32), 12.5)
    assert np.abs(got.double().cpu().numpy() - P.softcap(z.astype(np.float32).astype(np.float64), 12.5)).max() < 1e-5
    gu = rng.normal(size=(6, 2 * 40)) * 2
    for name, act, f in (("float32", "gelu_pytorch_tanh", P.gelu_tanh), ("bfloat16", "silu", P.silu)):
        g = dev(gu, DTYPES[name])
        mid = ops.gated_act(g, torch.empty(6, 40, dtype=DTYPES[name], device=DEV), act)
        src = g.double().cpu().numpy()
        want = f(src[:, :40]) * src[:, 40:]
        assert np.abs(mid.double().cpu().numpy() - want).max() <= (2e-6 if name == "float32" else 2.0 ** -7) * np.abs(want).max()


# ------------------------------------------------------------------------------------------ attention
def make_ctx(dtype, lens_new, past, Hkv, D, Dv, page=16, shuffle_seed=1):
    """A step context by hand: sequences with `past` cached positions bring `lens_new` tokens each (one-token
    sequences first, as the step function orders them); pages are handed out in a shuffled order."""
    from deliverance_amd.parts import Arena, StepContext
    S = len(lens_new)
    assert all(a == 1 for a in lens_new[:sum(1 for a in lens_new if a == 1)])
    total = [p + n for p, n in zip(past, lens_new)]
    n_pages = sum(-(-t // page) for t in total) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(shuffle_seed)).tolist()
    max_blocks = max(-(-t // page) for t in total)
    bt = torch.full((S, max_blocks), -1, dtype=torch.int32)
    for s, t in enumerate(total):
        for j in range(-(-t // page)):
            bt[s, j] = perm.pop()
    ctx = StepContext()
    ctx.device, ctx.dtype = torch.device(DEV), dtype
    ctx.n_seqs, ctx.n_tokens = S, sum(lens_new)
    ctx.n_decode = sum(1 for n in lens_new if n == 1)
    return ctx, bt, total, n_pages, max_blocks


def fill_ctx(ctx, bt, lens_new, past, total, page):
    pos, seq_of, slots, q_start = [], [], [], [0]
    for s in range(len(lens_new)):
        for i in range(lens_new[s]):
            p_ = past[s] + i
            pos.append(p_); seq_of.append(s); slots.append(int(bt[s, p_ // page]) * page + p_ % page)
        q_start.append(len(pos))
    ctx.positions, ctx.seq_of_token, ctx.q_start, ctx.seq_lens = dev(pos), dev(seq_of), dev(q_start), dev(total)
    ctx.tokens = dev([0] * len(pos))
    ctx.q_start_host, ctx.seq_lens_host = q_start, total
    ctx.max_query_len, ctx.max_seq_len = max(lens_new), max(total)
    ctx.block_tables, ctx.slot_maps = [bt.to(DEV)], [dev(slots)]


class AttentionBench:
    """Sequences with given q, k, v; their keys and values go to a paged cache in steps of any cut, and the
    attention of a step's rows is compared with the plain attention over the whole sequences."""

    def __init__(self, dtype, H, G, D, Dv, seqs, page=16, m=None):
        from deliverance_amd.parts import Arena
        self.dtype, self.H, self.G, self.D, self.Dv, self.page = DTYPES[dtype], H, G, D, Dv, page
        self.name = dtype
        self.seqs = seqs                      # list of (q [T,H,D], k [T,G,D], v [T,G,Dv]) float64, already rounded
        self.m = m
        n_pages = sum(-(-len(s[0]) // page) for s in seqs) + 3
        perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(7)).tolist()
        self.tables = [[perm.pop() for _ in range(-(-len(s[0]) // page))] for s in seqs]
        shape = (n_pages, 2, G, page, D) if D == Dv else (n_pages, G * page * (D + Dv))
        self.cache = torch.full(shape, float("nan"), dtype=self.dtype, device=DEV)
        self.arena = Arena(DEV)
        self.done = [0] * len(seqs)
        self.plain = None

    def step(self, takes, table=None, bias_max=0, coef=0.0, every=0, scale=1.0):
        """takes[s] tokens of sequence s (0: left out); returns the largest error of the step's rows against
        the plain attention, relative to the largest plain value."""
        from deliverance_amd.kernels import ops
        from deliverance_amd.parts import StepContext
        from deliverance_amd.parts.attention import bias_by_distance
        order = sorted((s for s in range(len(self.seqs)) if takes[s]), key=lambda s: (takes[s] != 1, s))
        lens_new, past = [takes[s] for s in order], [self.done[s] for s in order]
        total = [a + b for a, b in zip(past, lens_new)]
        max_blocks = max(len(self.tables[s]) for s in order)
        bt = torch.full((len(order), max_blocks), -1, dtype=torch.int32)
        for i, s in enumerate(order):
            bt[i, :len(self.tables[s])] = torch.tensor(self.tables[s], dtype=torch.int32)
        ctx = StepContext()
        ctx.device, ctx.dtype = torch.device(DEV), self.dtype
        ctx.n_seqs, ctx.n_tokens, ctx.n_decode = len(order), sum(lens_new), sum(1 for n in lens_new if n == 1)
        fill_ctx(ctx, bt, lens_new, past, total, self.page)
        ctx.cache = SimpleNamespace(page_size=self.page)
        ctx._arena = self.arena
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        rows = []
        for s, n, p in zip(order, lens_new, past):
            q, k, v = self.seqs[s]
            rows.append(np.concatenate([q[p:p + n].reshape(n, H * D), k[p:p + n].reshape(n, G * D), v[p:p + n].reshape(n, G * Dv)], axis=1))
        qkv = dev(np.concatenate(rows), self.dtype)
        if D == Dv:
            ops.kv_write(qkv, H * D, H * D + G * D, self.cache, ctx.slot_maps[0], G, D)
        else:
            ops.kv_write_split(qkv, H * D, H * D + G * D, self.cache, ctx.slot_maps[0], G, D, Dv, self.page)
        flat = None if table is None else bias_by_distance(torch.tensor(table), bias_max).to(DEV)
        out = torch.empty(ctx.n_tokens, H * Dv, dtype=self.dtype, device=DEV)
        ops.paged_attention_rel(ctx, qkv[:, :H * D], self.cache, 0, H, G, D, Dv, scale, None, flat, coef, every, out)
        got = out.double().cpu().numpy()
        m = {"scale": scale, "bias_max": bias_max, "q_temp": {"coef": coef, "every": every or 1 << 30}}
        if self.plain is None:
            self.plain = [P.attend(q, k, v, None if table is None else np.asarray(table, dtype=np.float64), m).reshape(len(q), H * Dv)
                          for q, k, v in self.seqs]
        worst, r = 0.0, 0
        for s, n, p in zip(order, lens_new, past):
            want = self.plain[s][p:p + n]
            worst = max(worst, np.abs(got[r:r + n] - want).max() / max(np.abs(self.plain[s]).max(), 1e-30))
            r += n
            self.done[s] = p + n
        return worst


def random_seqs(rng, lens, H, G, D, Dv, dtype):
    rd = bf16 if dtype == "bfloat16" else (lambda a: np.asarray(a, dtype=np.float32).astype(np.float64))
    return [(rd(rng.normal(size=(T, H, D))), rd(rng.normal(size=(T, G, D))), rd(rng.normal(size=(T, G, Dv)))) for T in lens]


ATT_TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("H,G,D,Dv", [quick(4, 2, 16, 16), (3, 3, 32, 16), (2, 1, 64, 64), (2, 2, 48, 48), (5, 5, 24, 40), (1, 1, 128, 128)])
def test_attention_with_bias_and_temperature(dtype, H, G, D, Dv):
    """A whole prompt, then decode tokens beside portions that start mid-page; the bias table has rows of very
    different values, so that a row read for a neighbouring distance shows, and the temperature steps every 5
    positions with a large coefficient."""
    rng = np.random.default_rng(H * 100 + D)
    n_rows, far = 10, 37
    table = rng.normal(size=(n_rows, H)) * 3
    table = bf16(table)
    lens = [83, 50, 21]
    b = AttentionBench(dtype, H, G, D, Dv, random_seqs(rng, lens, H, G, D, Dv, dtype))
    kw = dict(table=table, bias_max=far, coef=0.8, every=5, scale=0.9 / math.sqrt(D))
    tol = ATT_TOL[dtype]
    assert b.step([70, 0, 0], **kw) <= tol                # a whole portion from position 0
    assert b.step([1, 33, 2], **kw) <= tol                # a decode row beside portions
    assert b.step([1, 1, 1], **kw) <= tol                 # decode rows only, past of 71, 33 and 2
    assert b.step([11, 16, 18], **kw) <= tol              # portions after a past that ends mid-page
    assert b.done == lens


@pytest.mark.parametrize("dtype", [quick("float32"), "bfloat16"])
@pytest.mark.parametrize("decode", [False, True])
def test_one_far_key_among_hundreds(dtype, decode):
    """The last query matches key 3 of 600 (and nothing else): its output is that key's value.  The same with the
    match just inside and just outside the distance from which the bias no longer changes."""
    H, G, D, Dv, T = 2, 1, 32, 32, 600
    rng = np.random.default_rng(11)
    far = 150
    table = np.zeros((8, H))
    table[7] = -6.0                                         # the last row pushes far keys down, but not out
    for target in (3, T - 1 - far, T - far, T - 2):
        q = rng.normal(size=(T, H, D)) * 0.05
        k = rng.normal(size=(T, G, D)) * 0.05
        v = rng.normal(size=(T, G, Dv))
        direction = np.zeros(D); direction[5] = 1.0
        k[target, 0] = 6.0 * direction
        q[T - 1, :] = 6.0 * direction
        seqs = [(bf16(q), bf16(k), bf16(v))]
        b = AttentionBench(dtype, H, G, D, Dv, seqs)
        kw = dict(table=table, bias_max=far, coef=0.0, every=0, scale=1.0)
        if decode:
            assert b.step([T - 1], **kw) <= ATT_TOL[dtype]
            err = b.step([1], **kw)
        else:
            assert b.step([T - 40], **kw) <= ATT_TOL[dtype]
            err = b.step([40], **kw)
        assert err <= ATT_TOL[dtype]
        last = b.plain[0][T - 1].reshape(H, Dv)
        assert np.abs(last - seqs[0][2][target, 0]).max() < 0.02 * np.abs(seqs[0][2]).max()   # the plain model itself finds it


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_every_edge_of_the_bias_rows(dtype):
    """Equal keys everywhere, so that the weights are the bias alone: a row's edge that is one distance off moves
    a whole key's weight.  Values are one-hot by position, so the output spells out the weights."""
    H, G, D, T = 1, 1, 16, 64
    n_rows, far = 12, 40
    table = (np.arange(n_rows)[:, None] % 2) * 4.0 - 2.0 + np.arange(n_rows)[:, None] * 0.25
    q = np.ones((T, H, D)) * 0.1
    k = np.ones((T, G, D)) * 0.1
    v = np.zeros((T, G, T)); v[np.arange(T), 0, np.arange(T)] = 1.0
    b = AttentionBench(dtype, H, G, D, T, [(q, k, v)])
    kw = dict(table=bf16(table), bias_max=far, coef=0.0, every=0, scale=1.0)
    tol = 1e-5 if dtype == "float32" else 6e-3
    assert b.step([50], **kw) <= tol
    for _ in range(T - 50):
        assert b.step([1], **kw) <= tol


# ------------------------------------------------------------------------------------------ feed-forwards
def ff_ctx(dtype, tokens):
    from deliverance_amd.parts import Arena, StepContext
    ctx = StepContext()
    ctx.device, ctx.dtype = torch.device(DEV), DTYPES[dtype]
    ctx.n_tokens = len(tokens)
    ctx.tokens = dev(tokens)
    ctx._arena = Arena(DEV)
    return ctx


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("E,F,N", [quick(64, 40, 5), (80, 104, 40), (96, 200, 70)])
def test_gated_feed_forward_part(dtype, E, F, N):
    from deliverance_amd.config.specs import GatedFeedForwardSpec
    from deliverance_amd.parts import build_feed_forward
    rng = np.random.default_rng(E + N)
    Wg, Wu, Wd = (bf16(rng.normal(size=s) * 0.2) for s in ((F, E), (F, E), (E, F)))
    p = {"gate_up_weight": torch.tensor(np.concatenate([Wg, Wu])).to(torch.bfloat16), "down_weight": torch.tensor(Wd).to(torch.bfloat16)}
    ff = build_feed_forward(GatedFeedForwardSpec("gated", E, F, "gelu_pytorch_tanh"), p, DTYPES[dtype], DEV)
    h = bf16(rng.normal(size=(N, E)))
    x0 = rng.normal(size=(N, E)).astype(np.float32)
    want = P.gated_ff(h, Wg, Wu, Wd, P.gelu_tanh)
    tol = (3e-6 if dtype == "float32" else 1.5e-2) * np.abs(want).max()
    ctx = ff_ctx(dtype, [0] * N)
    x = dev(x0, torch.float32)
    ff.forward(ctx, dev(h, DTYPES[dtype]), x)                       # adds into what it is given
    assert np.abs(x.double().cpu().numpy() - (x0 + want)).max() <= tol
    ctx.part_accumulate = False                                     # ... or stores, when told so
    x = dev(x0, torch.float32)
    ff.forward(ctx, dev(h, DTYPES[dtype]), x)
    assert np.abs(x.double().cpu().numpy() - want).max() <= tol
    with pytest.raises(ValueError, match="gate"):
        build_feed_forward(GatedFeedForwardSpec("gated", E, F + 8, "gelu_pytorch_tanh"), p, DTYPES[dtype], DEV)


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("E,F,n_experts,top,N", [quick(64, 24, 4, 2, 9), (96, 40, 3, 3, 5), (64, 72, 7, 1, 150), (128, 64, 5, 2, 300)])
def test_experts_feed_forward_part(dtype, E, F, n_experts, top, N):
    """Tokens pick their experts by a table; one expert is used by no token of the step, another by most."""
    from deliverance_amd.config.specs import ExpertsFeedForwardSpec
    from deliverance_amd.parts import build_feed_forward
    rng = np.random.default_rng(E + N + top)
    V = 50
    table = np.stack([rng.permutation(n_experts)[:top] for _ in range(V)])
    unused = n_experts - 1
    if top < n_experts:                         # rows that name the last expert name another one instead
        spare = [[e for e in range(n_experts - 1) if e not in row] for row in table]
        table = np.array([[spare[i][0] if e == unused else e for e in row] for i, row in enumerate(table)])
    W = {}
    for e in range(n_experts):
        W[f"m.e{e}.gate"], W[f"m.e{e}.up"], W[f"m.e{e}.down"] = (bf16(rng.normal(size=s) * 0.2) for s in ((F, E), (F, E), (E, F)))
    p = {"gate_up_weight": torch.tensor(np.stack([np.concatenate([W[f"m.e{e}.gate"], W[f"m.e{e}.up"]]) for e in range(n_experts)])).to(torch.bfloat16),
         "down_weight": torch.tensor(np.stack([W[f"m.e{e}.down"] for e in range(n_experts)])).to(torch.bfloat16),
         "table": torch.tensor(table, dtype=torch.int32)}
    spec = ExpertsFeedForwardSpec("experts", E, F, n_experts, top, "silu", vocab_size=V)
    ff = build_feed_forward(spec, p, DTYPES[dtype], DEV)
    tokens = [int(t) for t in rng.integers(0, V, size=N)]
    tokens[:max(1, N // 2)] = [tokens[0]] * max(1, N // 2)          # most rows go to the same experts
    h = bf16(rng.normal(size=(N, E)))
    x0 = rng.normal(size=(N, E)).astype(np.float32)
    want = P.experts_ff(h, tokens, table, W, "m.")
    tol = (3e-6 if dtype == "float32" else 1.5e-2) * np.abs(want).max()
    ctx = ff_ctx(dtype, tokens)
    x = dev(x0, torch.float32)
    ff.forward(ctx, dev(h, DTYPES[dtype]), x)
    assert np.abs(x.double().cpu().numpy() - (x0 + want)).max() <= tol
    ctx.part_accumulate = False
    ff.forward(ctx, dev(h, DTYPES[dtype]), x)
    assert np.abs(x.double().cpu().numpy() - want).max() <= tol
    bad = dict(p, table=torch.full((V, top), n_experts, dtype=torch.int32))
    with pytest.raises(ValueError, match="expert table"):
        build_feed_forward(spec, bad, DTYPES[dtype], DEV)


# ------------------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def vmodels(tmp_path_factory):
    return {"X": make_model(tmp_path_factory.mktemp("vx"), CONFIG_X, 11), "Y": make_model(tmp_path_factory.mktemp("vy"), CONFIG_Y, 12),
            "Z": make_model(tmp_path_factory.mktemp("vz"), CONFIG_Z, 13)}


def check(model, got, requests, dtype, what=""):
    """32-bit: every logit within 3e-5 of the largest plain logit.  bfloat16: the largest error within 6 % of the
    logits' root mean square and the rms error within 2^-6 of it (norms behind every part and looped layers: about
    twice the roundings of a plain pre-norm model of the same depth)."""
    for rid, ids in requests:
        ref = model.plain_logits(ids)
        out = got[rid].astype(np.float64)
        assert out.shape == ref.shape, f"{what} {rid}: shape {out.shape} vs {ref.shape}"
        err = np.abs(out - ref)
        rms = float(np.sqrt((ref ** 2).mean()))
        bound = 3e-5 * np.abs(ref).max() if dtype == "float32" else 6e-2 * rms
        first = int(np.argmax(err.max(axis=1) > bound))
        assert err.max() <= bound, f"{what} {rid} ({dtype}): max error {err.max():.3e} > {bound:.3e}, first at position {first}"
        if dtype == "bfloat16":
            assert float(np.sqrt((err ** 2).mean())) <= 2.0 ** -6 * rms, f"{what} {rid}: rms error"


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("X"), "Y", "Z"])
def test_whole_prompts_and_first_tokens(vmodels, name, dtype):
    m = vmodels[name]
    reqs = [("one", m.prompt(1)), ("two", m.prompt(2)), ("long", m.prompt(90 if name != "Z" else 140))]
    s = helpers.trace_session(m.folder, dtype, 256)
    for rid, ids in reqs:
        check(m, helpers.replay(s, helpers.trace_whole(rid, ids)), [(rid, ids)], dtype, "whole")
    s.cache.manager.check()


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["X", quick("Y"), "Z"])
def test_prefill_against_token_by_token_decoding(vmodels, name, dtype):
    """All but the last 45 tokens at once, the rest one by one: they cross page borders, steps of the
    temperature and (in Y) the distance from which the bias stays."""
    m = vmodels[name]
    ids = m.prompt(75, salt=1)
    s = helpers.trace_session(m.folder, dtype, 128)
    check(m, helpers.replay(s, helpers.trace_bulk_then_single("r", ids, tail=45)), [("r", ids)], dtype, "decode")
    # ... and from the very first token on
    ids2 = m.prompt(20, salt=2)
    check(m, helpers.replay(s, helpers.trace_bulk_then_single("q", ids2, tail=19)), [("q", ids2)], dtype, "decode from 1")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("X"), "Y", "Z"])
@pytest.mark.parametrize("sizes", [(7, 2, 13, 3, 5, 2), quick((2, 2, 31, 1, 16, 33, 2))])
def test_portions_of_any_size(vmodels, name, dtype, sizes):
    m = vmodels[name]
    ids = m.prompt(97, salt=3)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True)
    check(m, helpers.replay(s, helpers.trace_portions("r", ids, sizes)), [("r", ids)], dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["X", "Y", quick("Z")])
def test_mixed_batches_over_a_small_pool(vmodels, name, dtype):
    """Seven unequal requests, four live at a time, over a pool that holds just what is live: pages and the
    requests' places come back and go out again (freed pages are filled with NaN).  Then every request alone:
    what a request gets must not depend on its neighbours beyond rounding."""
    m = vmodels[name]
    reqs = [(f"r{i}", m.prompt(n, salt=10 + i)) for i, n in enumerate((40, 3, 71, 18, 64, 1, 33))]
    steps = helpers.trace_mixed(reqs, seed=5, max_live=4)
    s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True)
    got = helpers.replay(s, steps)
    check(m, got, reqs, dtype, "mixed")
    s.cache.manager.check()
    alone = helpers.trace_session(m.folder, dtype, 128)
    for rid, ids in reqs[:3]:
        one = helpers.replay(alone, helpers.trace_whole(rid, ids))[rid]
        scale = float(np.sqrt((one.astype(np.float64) ** 2).mean()))
        assert np.abs(one.astype(np.float64) - got[rid]).max() <= (2e-5 if dtype == "float32" else 4e-2) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(vmodels, dtype):
    """Two hundred tokens one by one beside a neighbour that comes and goes."""
    m = vmodels["X"]
    ids, other = m.prompt(210, salt=20), m.prompt(60, salt=21)
    helpers.skip_in_simulation_if(True)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:10], "want": list(range(10))}], "end": []}]
    for i in range(10, len(ids)):
        entries = [{"id": "a", "tokens": [ids[i]], "want": [0]}]
        j = i - 50
        if 0 <= j < len(other):
            entries.append({"id": "b", "tokens": [other[j]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["b"] if j == len(other) - 1 else []})
    steps[-1]["end"].append("a")
    s = helpers.trace_session(m.folder, dtype, 320, poison_freed=True)
    check(m, helpers.replay(s, steps), [("a", ids), ("b", other)], dtype, "long decode")


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["X", "Y"])
def test_greedy_generation_through_the_engine(vmodels, name, dtype):
    """The engine's own entry point and scheduler: several prompts at once over a pool that forces portions,
    with recorded decode steps and steps launched ahead, against the plain model's greedy choice."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = vmodels[name]
    prompts = [m.prompt(n, salt=30 + n) for n in (5, 33, 70, 2)]
    model = AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=512, max_num_seqs=3,
                                                 max_batch_tokens=48, max_chunk=32)
    outs = model.generate(prompts, GeneratorParameters(max_tokens=24, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.finish_reason == "length" and len(out.generated_tokens) == 24
        if dtype == "float32":
            assert out.generated_tokens == P.greedy_generate(m.plain_cfg, m.W, prompt, 24)
        else:
            ids = list(prompt)
            for t in out.generated_tokens:            # bfloat16 may flip a near-tie, nothing more
                row = m.plain_logits(ids)[-1]
                assert row[t] >= row.max() - 2 * 6e-2 * float(np.sqrt((row ** 2).mean()))
                ids.append(t)


# ------------------------------------------------------------------------------------------ random configurations
def random_config(seed):
    """Sizes drawn at random, among them what the kernels take only on their plain paths: widths that are no
    multiple of 8 or 4, head sizes that are no multiple of 16, values of another size, bias tables longer than the
    prefill kernel's copy, one expert, as many experts a token as there are, loops over any range."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = pick(40, 50, 64, 100, 72, 36)
    n_layers = int(rng.integers(1, 4))
    layers = []
    for _ in range(n_layers):
        G = pick(1, 2, 3)
        H = G * pick(1, 2, 3)
        D = pick(8, 16, 24, 32, 64)
        Dv = pick(D, D, 8, 40)
        buckets = pick(2, 4, 5, 9, 16, 30)
        far = buckets // 2 + pick(1, 3, 20, 200, 1500)
        mlp = pick(None, "dense", "moe", "moe")
        if mlp == "dense":
            mlp = _dense = {"kind": "dense", "ff": pick(24, 40, 100)}
        elif mlp == "moe":
            n = pick(1, 2, 5, 9)
            mlp = {"kind": "moe", "expert": {"ff": pick(8, 20, 32)}, "router": {"experts": n, "top": pick(1, n, max(1, n // 2))}}
        layers.append({"type": "attention", "mlp": mlp,
                       "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": float(pick(0.1, D ** -0.5, 0.3)),
                                 "bias_max": far, "bias_buckets": buckets,
                                 "q_temp": {"coef": float(pick(0.0, 0.25, 1.5)), "every": pick(1, 3, 16, 500)}}})
    a = int(rng.integers(0, n_layers + 1))
    b = int(rng.integers(a, n_layers + 1))
    cfg = {"architecture": "Virudra", "vocab": pick(50, 130, 257), "width": width, "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))},
           "logit_softcap": float(pick(5.0, 25.0, 100.0)), "layers": layers}
    if pick(True, True, False):
        cfg["loop"] = {"start": a, "stop": b, "times": pick(1, 2, 3)}
    return cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(tmp_path, seed, dtype):
    m = make_model(tmp_path / "m", random_config(seed), 100 + seed)
    ids = m.prompt(45, salt=seed)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True)
    check(m, helpers.replay(s, helpers.trace_whole("w", ids)), [("w", ids)], dtype, f"seed {seed} whole")
    check(m, helpers.replay(s, helpers.trace_portions("p", ids, (5, 2, 17, 1, 1, 9))), [("p", ids)], dtype, f"seed {seed} portions")
