"""Pedatar on the engine against the plain implementation (tests/plain_pedatar.py): each mechanism alone through
its kernels and parts, then whole models through the step function (whole prompts, decoding token by token,
portions down to two tokens, mixed batches over a small pool whose pages and state slots come back and go out
again), and greedy generation through the engine's entry point and scheduler.  Sizes differ from test to test;
where random numbers would hide a fault (one far key among hundreds, a page's edge) the inputs are made so that it
shows.  In bfloat16 two experts of nearly equal score may be ranked the other way round: the engine reports its
choices through the layer debug hook and the plain model follows them where they are as good as its own."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_pedatar as P
from helpers import quick
from pedatar_models import CONFIG_P, CONFIG_Q, CONFIG_R, att_layer, latent, make_model, moe, replay_routed, scan, scan_layer

pytestmark = pytest.mark.gpu
DEV = helpers.DEVICE
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
SLACK = {"float32": 1e-4, "bfloat16": 0.06}      # how far below the plain model's last choice an engine's choice may lie


def bf16(a):
    """What bfloat16 keeps of an array (as float64)."""
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def dev(a, dtype=torch.int32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def host(t):
    return t.double().cpu().numpy()


def step_ctx(dtype, lens_new, past, page=16, n_state_slots=0, slots=None, shuffle_seed=1):
    """A step context by hand: sequences with `past` cached positions bring `lens_new` tokens each (one-token
    sequences first, as the step function orders them); pages are handed out in a shuffled order."""
    from deliverance_amd.parts import Arena, StepContext
    S = len(lens_new)
    total = [p + n for p, n in zip(past, lens_new)]
    n_pages = sum(-(-t // page) for t in total) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(shuffle_seed)).tolist()
    max_blocks = max(-(-t // page) for t in total)
    bt = torch.full((S, max_blocks), -1, dtype=torch.int32)
    for s, t in enumerate(total):
        for j in range(-(-t // page)):
            bt[s, j] = perm.pop()
    ctx = StepContext()
    ctx.device, ctx.dtype = torch.device(DEV), DTYPES[dtype]
    ctx.n_seqs, ctx.n_tokens = S, sum(lens_new)
    ctx.n_decode = sum(1 for n in lens_new if n == 1)
    pos, seq_of, rows, q_start = [], [], [], [0]
    for s in range(S):
        for i in range(lens_new[s]):
            p_ = past[s] + i
            pos.append(p_); seq_of.append(s); rows.append(int(bt[s, p_ // page]) * page + p_ % page)
        q_start.append(len(pos))
    ctx.positions, ctx.seq_of_token, ctx.q_start, ctx.seq_lens = dev(pos), dev(seq_of), dev(q_start), dev(total)
    ctx.tokens = dev([0] * len(pos))
    ctx.q_start_host, ctx.seq_lens_host = q_start, total
    ctx.max_query_len, ctx.max_seq_len = max(lens_new), max(total)
    ctx.block_tables, ctx.slot_maps = [bt.to(DEV)], [dev(rows)]
    ctx.state_slots = dev(slots if slots is not None else list(range(S)))
    ctx.state_slots_host = list(slots) if slots is not None else list(range(S))
    ctx._arena = Arena(DEV)
    ctx.cache = SimpleNamespace(page_size=page, group_of_slot={0: 0}, kv={}, state={})
    return ctx, n_pages


# ------------------------------------------------------------------------------------------ rotation
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
def test_rotation_of_pairs(dtype, interleaved):
    """Heads at a stride inside wider rows, only the first entries turned, into another place and in place; positions
    in the thousands, where an angle in 32-bit would be off by more than the bound."""
    from deliverance_amd.config.specs import RotarySpec
    from deliverance_amd.parts import build_position
    rng = np.random.default_rng(4)
    N, H, width, dims, base = 7, 3, 12, 8, 300.0
    places = [0, 1, 2, 1000, 4097, 65000, 3]
    src = bf16(rng.normal(size=(N, 5 + H * 20)))
    rot = build_position(RotarySpec("rotary", dims, base, interleaved), {}, DTYPES[dtype], DEV)
    ctx = SimpleNamespace(positions=dev(places))
    s = dev(src, DTYPES[dtype])
    out = torch.zeros(N, H * width + 3, dtype=DTYPES[dtype], device=DEV)
    rot.apply(ctx, s[:, 5:], out[:, 3:], H, 20, width, width)
    v = src[:, 5:].reshape(N, H, 20)[:, :, :width]
    if interleaved:
        want = P.turn_pairs(v, places, dims, base)
    else:                      # the pair of entry i is entry i + dims / 2
        idx = np.arange(dims).reshape(2, dims // 2).T.reshape(-1)
        w2 = v.copy()
        w2[..., :dims] = v[..., idx]
        w2 = P.turn_pairs(w2, places, dims, base)
        want = w2.copy()
        want[..., idx] = w2[..., :dims]
    tol = 2e-6 if dtype == "float32" else 2.0 ** -7
    got = host(out[:, 3:]).reshape(N, H, width)
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    assert float(out[:, :3].abs().max()) == 0.0
    s2 = s.clone()
    rot.apply(ctx, s2[:, 5:], s2[:, 5:], H, 20, 20, width)          # in place
    assert np.abs(host(s2[:, 5:]).reshape(N, H, 20)[:, :, :width] - want).max() <= tol * np.abs(want).max()
    assert torch.equal(s2[:, :5], s[:, :5])


# ------------------------------------------------------------------------------------------ latent attention
class LatentBench:
    """One latent-attention part with weights of its own, fed with rows h of whole sequences in steps of any cut; its
    additions to the stream are compared with the plain mixer over the whole sequences."""

    def __init__(self, dtype, m, width, seqs, page=16, seed=0, make=None):
        from deliverance_amd.config.specs import LatentAttentionSpec, RotarySpec
        from deliverance_amd.parts import build_mixer
        rng = np.random.default_rng(seed)
        H, dn, dr, dv, rq, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
        W = {"mix.dq": rng.normal(size=(rq, width)) * 0.2, "mix.dq.norm": 1 + rng.normal(size=rq) * 0.1,
             "mix.uq": rng.normal(size=(H * (dn + dr), rq)) * 0.3, "mix.dkv": rng.normal(size=(r + dr, width)) * 0.2,
             "mix.dkv.norm": 1 + rng.normal(size=r) * 0.1, "mix.uk": rng.normal(size=(H * dn, r)) * 0.3,
             "mix.uv": rng.normal(size=(H * dv, r)) * 0.3, "mix.o": rng.normal(size=(width, H * dv)) * 0.2}
        if make is not None:
            make(W)
        self.W = {k: bf16(v) for k, v in W.items()}
        self.m, self.width, self.dtype, self.page, self.eps = m, width, dtype, page, 1e-5
        spec = LatentAttentionSpec("latent_attention", width, H, dn, dr, dv, rq, r, m["scale"], self.eps,
                                   RotarySpec("rotary", m["rot"]["dims"], m["rot"]["base"]))
        t = lambda k: torch.tensor(self.W[k], dtype=torch.float32).to(torch.bfloat16)
        self.part = build_mixer(spec, {"q_down_weight": t("mix.dq"), "q_norm_weight": t("mix.dq.norm"), "q_up_weight": t("mix.uq"),
                                       "kv_down_weight": t("mix.dkv"), "kv_norm_weight": t("mix.dkv.norm"),
                                       "k_up_weight": t("mix.uk"), "v_up_weight": t("mix.uv"), "out_weight": t("mix.o")},
                                DTYPES[dtype], DEV)
        self.seqs = [bf16(s) for s in seqs]                       # h of every sequence, [T, width]
        self.want = [P.latent_attention(self.W, "", m, s, self.eps) for s in self.seqs]
        n_pages = sum(-(-len(s) // page) for s in seqs) + 3
        perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(7)).tolist()
        self.tables = [[perm.pop() for _ in range(-(-len(s) // page))] for s in seqs]
        self.cache = torch.full((n_pages, page * (r + dr)), float("nan"), dtype=DTYPES[dtype], device=DEV)
        self.done = [0] * len(seqs)

    def step(self, takes):
        """takes: {sequence: number of next tokens}; returns the largest error of the step relative to the largest
        value of the plain result."""
        order = sorted(takes, key=lambda s: (takes[s] != 1, s))
        ctx, _ = step_ctx(self.dtype, [takes[s] for s in order], [self.done[s] for s in order], self.page)
        mb = max(len(self.tables[s]) for s in order)
        bt = torch.full((len(order), mb), -1, dtype=torch.int32)
        rows = []
        for i, s in enumerate(order):
            bt[i, :len(self.tables[s])] = torch.tensor(self.tables[s], dtype=torch.int32)
            rows += [self.tables[s][p // self.page] * self.page + p % self.page for p in range(self.done[s], self.done[s] + takes[s])]
        ctx.block_tables, ctx.slot_maps = [bt.to(DEV)], [dev(rows)]
        ctx.cache.kv = {0: self.cache}
        h = np.concatenate([self.seqs[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        x = torch.zeros(len(h), self.width, dtype=torch.float32, device=DEV)
        self.part.forward(ctx, dev(h, DTYPES[self.dtype]), x, SimpleNamespace(layer=0, cache=0, write=True))
        want = np.concatenate([self.want[s][self.done[s]:self.done[s] + takes[s]] for s in order])
        for s in order:
            self.done[s] += takes[s]
        scale = max(np.abs(w).max() for w in self.want)
        return np.abs(host(x) - want).max() / scale


LATENT_SIZES = [quick(latent(2, 16, 8, 24, 24, 40, 0.2, 10000.0)),          # matrix cores, values behind R in a partly filled block
                latent(3, 8, 12, 20, 18, 27, 0.3, 500.0, dims=6),             # rows of 39 entries: the plain kernel
                quick(latent(5, 32, 32, 16, 48, 160, 0.1, 10000.0)),          # rows of 192 entries: the middle form of the kernel
                latent(1, 64, 64, 64, 32, 320, 0.08, 1e6, dims=32),           # rows of 384 entries: the third form, one head
                latent(2, 16, 48, 32, 24, 400, 0.06, 10000.0)]                # rows of 448 entries: the largest form


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", LATENT_SIZES)
def test_latent_attention_part_prompt_portions_and_decoding(m, dtype):
    rng = np.random.default_rng(5)
    helpers.skip_in_simulation_if(m["kv_rank"] > 100 and (dtype == "float32" or m["kv_rank"] > 350))
    lens = (70, 33, 1)
    b = LatentBench(dtype, m, 64, [rng.normal(size=(n, 64)) for n in lens])
    tol = 2e-5 if dtype == "float32" else 3e-2
    assert b.step({0: 33, 1: 2}) <= tol                  # portions; the second ends inside a page
    assert b.step({0: 1, 1: 1, 2: 1}) <= tol             # decoding beside a first token
    assert b.step({0: 30, 1: 14}) <= tol                 # across a tile of 32 keys and page borders
    assert b.step({0: 1, 1: 1}) <= tol
    assert b.step({0: 5, 1: 15}) <= tol
    assert b.done == [70, 33, 1]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("where", [0, 15, 16, quick(31), 32, 47, 200, quick(319)])
def test_latent_attention_finds_one_far_key(dtype, where):
    """Among 320 tokens one has a key piece that the last query matches with a score far above all others, and a
    latent of its own: the output at the last position must be that token's value.  A key that is lost, shifted by
    one, or read from the wrong page shows as an error of the order of the output."""
    m = latent(2, 16, 16, 16, 16, 32, 1.0, 10000.0, dims=0)          # nothing turns: the key piece is matched as it is
    T, width = 320, 32
    rng = np.random.default_rng(where)
    h = rng.normal(size=(T, width)) * 0.1
    h[where, 0] = 6.0                                                # a marked token ...
    h[T - 1, 1] = 6.0                                                # ... and the one that asks for it

    def make(W):
        W["mix.dkv"][32:, 0] = 3.0          # the marked token's key piece is large in every entry
        W["mix.uq"][:, :] *= 0.05
        W["mix.dq"][0, 1] = 8.0             # the asking token's query latent is large in entry 0 ...
        for head in range(2):
            W["mix.uq"][head * 32 + 16:head * 32 + 32, 0] = 2.0       # ... which feeds every head's rotated query entries

    for decode in (False, True):
        b = LatentBench(dtype, m, width, [h], seed=1, make=make)
        if decode:
            assert b.step({0: T - 1}) < 1.0
            err = b.step({0: 1})
        else:
            err = b.step({0: T})
        # (a key that is missed costs an error of the order of the output itself; the bound leaves room for the
        # roundings of a bfloat16 row that is all one token's value)
        assert err <= (3e-5 if dtype == "float32" else 6e-2), f"key at {where}, decode={decode}"
    # the case is what it says: the plain weights of the last row put nearly everything on `where`
    W = b.W
    cq = P.unit_rms(b.seqs[0] @ W["mix.dq"].T, W["mix.dq.norm"], 1e-5)
    q = (cq @ W["mix.uq"].T).reshape(T, 2, 32)
    down = b.seqs[0] @ W["mix.dkv"].T
    c = P.unit_rms(down[:, :32], W["mix.dkv.norm"], 1e-5)
    s = (q[-1, 0, :16] @ (c @ W["mix.uk"].T).reshape(T, 2, 16)[:, 0].T + q[-1, 0, 16:] @ down[:, 32:].T)
    assert int(np.argmax(s)) == where and np.sort(s)[-1] - np.sort(s)[-2] > 8.0


# ------------------------------------------------------------------------------------------ short filter and scan
def scan_weights(rng, width, m):
    I, n, r, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
    W = {"mix.in": rng.normal(size=(2 * I, width)) * 0.3, "mix.conv": rng.normal(size=(I, K)) * 0.5,
         "mix.conv.b": rng.normal(size=I) * 0.3, "mix.x": rng.normal(size=(r + 2 * n, I)) * 0.2,
         "mix.dt": rng.normal(size=(I, r)) * 0.5, "mix.dt.b": rng.normal(size=I) * 0.5,
         "mix.A_log": rng.normal(size=(I, n)) * 0.7, "mix.D": rng.normal(size=I) * 0.3, "mix.o": rng.normal(size=(width, I)) * 0.2}
    return {k: bf16(v) for k, v in W.items()}


SCAN_SIZES = [quick(scan(96, 16, 8, 4)), scan(100, 24, 3, 2), quick(scan(48, 1, 1, 1)), scan(64, 40, 2, 3), scan(40, 70, 5, 7)]


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("m", SCAN_SIZES)
def test_selective_scan_part_any_cut_and_slots_used_again(m, dtype, monkeypatch):
    """Three sequences in portions of every size (shorter than the filter, one token, long ones cut into chunks that run
    side by side), their states in slots that are not in order; then a new sequence takes a slot that was used."""
    from deliverance_amd.config.specs import SelectiveScanSpec
    from deliverance_amd.kernels import ops
    from deliverance_amd.parts import build_mixer
    monkeypatch.setattr(ops, "SCAN_CHUNK", 8)
    monkeypatch.setattr(ops, "SCAN_CHUNK_FROM", 20)
    rng = np.random.default_rng(9)
    width = 32
    W = scan_weights(rng, width, m)
    t = lambda k: torch.tensor(W[k], dtype=torch.float32).to(torch.bfloat16)
    part = build_mixer(SelectiveScanSpec("selective_scan", width, m["inner"], m["state"], m["dt_rank"], m["conv"]),
                       {"in_weight": t("mix.in"), "conv_weight": t("mix.conv"), "conv_bias": t("mix.conv.b"), "x_weight": t("mix.x"),
                        "dt_weight": t("mix.dt"), "dt_bias": t("mix.dt.b"), "a_log": t("mix.A_log"), "d": t("mix.D"),
                        "out_weight": t("mix.o")}, DTYPES[dtype], DEV)
    need = part.cache_need()
    state = torch.full((5, need.elems), float("nan"), dtype=torch.float32, device=DEV)
    seqs = [bf16(rng.normal(size=(n, width))) for n in (61, 23, 9, 30)]
    want = [P.mamba1(W, "", m, s) for s in seqs]
    scale = max(np.abs(w).max() for w in want)
    slot_of = {0: 3, 1: 0, 2: 4, 3: 0}             # sequence 3 starts when sequence 1 has ended, in its slot
    done = [0] * 4
    tol = 3e-5 if dtype == "float32" else 3e-2

    def step(takes):
        order = sorted(takes, key=lambda s: (takes[s] != 1, s))
        for s in order:
            if done[s] == 0:
                state[slot_of[s]].zero_()          # what the engine does when a request is opened
        ctx, _ = step_ctx(dtype, [takes[s] for s in order], [done[s] for s in order], slots=[slot_of[s] for s in order])
        ctx.cache.state = {0: state}
        h = np.concatenate([seqs[s][done[s]:done[s] + takes[s]] for s in order])
        x = torch.zeros(len(h), width, dtype=torch.float32, device=DEV)
        part.forward(ctx, dev(h, DTYPES[dtype]), x, SimpleNamespace(layer=0, cache=0, write=True))
        ref = np.concatenate([want[s][done[s]:done[s] + takes[s]] for s in order])
        for s in order:
            done[s] += takes[s]
        assert np.abs(host(x) - ref).max() <= tol * scale, f"step {takes}"

    step({0: 2, 1: 1})              # shorter than the filter
    step({0: 1, 1: 2, 2: 9})
    step({0: 25, 1: 20})            # chunks of 8: three and a bit, two and a half
    step({0: 1, 3: 22})             # a decoded token beside a portion in chunks; slot 0 again, from zero
    step({0: 32, 3: 8})
    assert done == [61, 23, 9, 30]


def test_short_filter_and_state_kernels_alone():
    """The filter over rows that come from the state, and the state after portions shorter than it."""
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(2)
    C, K = 20, 5
    w, b = bf16(rng.normal(size=(C, K))), bf16(rng.normal(size=C))
    seq = bf16(rng.normal(size=(12, C)))
    want = P.short_filter(seq, w, b)
    state = torch.zeros(2, 7 + (K - 1) * C, dtype=torch.float32, device=DEV)     # the filter's part starts at entry 7
    done = 0
    for n in (1, 2, 1, 6, 2):
        ctx, _ = step_ctx("float32", [n], [done], slots=[1])
        x = dev(seq[done:done + n], torch.float32)
        y = torch.empty(n, C, dtype=torch.float32, device=DEV)
        ops.conv_causal(ctx, x, state, 7, dev(w, torch.float32), dev(b, torch.float32), None, y)
        ops.conv_state_update(ctx, x, state, 7, C, K)
        assert np.abs(host(y) - want[done:done + n]).max() <= 1e-5
        done += n
        kept = host(state[1, 7:]).reshape(K - 1, C)
        last = np.concatenate([np.zeros((K - 1, C)), seq[:done]])[-(K - 1):]
        assert np.abs(kept - last).max() == 0.0
    assert float(state[0].abs().max()) == 0.0 and float(state[1, :7].abs().max()) == 0.0


# ------------------------------------------------------------------------------------------ routed feed-forward
@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("n_experts,top,ff,shared,N", [quick(4, 2, 32, 48, 9), (1, 1, 40, 0, 5), (3, 3, 20, 0, 70),
                                                        (12, 3, 24, 16, 300), quick(6, 1, 16, 64, 130)])
def test_routed_feed_forward_part(n_experts, top, ff, shared, N, dtype):
    """Scores from a logistic router, the best experts, each fed with the row times its score; a shared expert beside
    them.  Few rows (decoding's grouped products) and many (the block tiles with gathered rows)."""
    from deliverance_amd.config.specs import ExpertsFeedForwardSpec
    from deliverance_amd.parts import build_feed_forward
    rng = np.random.default_rng(n_experts * 10 + top)
    width = 64
    W = {"mlp.router": bf16(rng.normal(size=(n_experts, width)) * 0.3)}
    for e in range(n_experts):
        W[f"mlp.e{e}.up"], W[f"mlp.e{e}.down"] = bf16(rng.normal(size=(ff, width)) * 0.2), bf16(rng.normal(size=(width, ff)) * 0.2)
    if shared:
        W["mlp.shared.up"], W["mlp.shared.down"] = bf16(rng.normal(size=(shared, width)) * 0.2), bf16(rng.normal(size=(width, shared)) * 0.2)
    mlp = moe(n_experts, top, ff, shared or None)
    h = bf16(rng.normal(size=(N, width)))
    if top < n_experts:                          # keep the rows whose choice does not hang on a hair
        keep = P.router_margin(W, "", mlp, h) > 0.02
        h = h[keep]
        N = len(h)
    t = lambda a: torch.tensor(a, dtype=torch.float32).to(torch.bfloat16)
    params = {"up_weight": torch.stack([t(W[f"mlp.e{e}.up"]) for e in range(n_experts)]),
              "down_weight": torch.stack([t(W[f"mlp.e{e}.down"]) for e in range(n_experts)]), "router_weight": t(W["mlp.router"])}
    if shared:
        params["shared_up_weight"], params["shared_down_weight"] = t(W["mlp.shared.up"]), t(W["mlp.shared.down"])
    spec = ExpertsFeedForwardSpec("experts", width, ff, n_experts, top, "relu2", router="logistic_top", gated=False,
                                  weight_on="input", shared_inner=shared, shared_activation="relu2")
    part = build_feed_forward(spec, params, DTYPES[dtype], DEV)
    ctx, _ = step_ctx(dtype, [N], [0])
    want = P.routed_ff(W, "", mlp, h)
    x0 = rng.normal(size=(N, width))
    x = dev(x0, torch.float32)
    part.forward(ctx, dev(h, DTYPES[dtype]), x)
    tol = (2e-5 if dtype == "float32" else 2e-2) * np.abs(want).max()
    assert np.abs(host(x) - (x0.astype(np.float32) + want)).max() <= tol
    ctx.part_accumulate = False
    part.forward(ctx, dev(h, DTYPES[dtype]), x)                 # stores the experts' sum, then adds the shared expert
    assert np.abs(host(x) - want).max() <= tol


def test_router_takes_the_largest_scores_and_the_lower_index_on_a_tie():
    from deliverance_amd.kernels import ops
    z = np.array([[0.5, 2.0, 2.0, -1.0, 1.5], [-3.0, -3.0, -3.0, -3.0, -3.0], [9.0, -9.0, 0.0, 8.0, 8.5]], dtype=np.float32)
    ids = torch.zeros(3, 3, dtype=torch.int32, device=DEV)
    w = torch.zeros(3, 3, dtype=torch.float32, device=DEV)
    ops.moe_top_logistic(dev(z, torch.float32), 3, False, ids, w)
    assert ids.cpu().tolist() == [[1, 2, 4], [0, 1, 2], [0, 4, 3]]
    want = P.logistic(np.take_along_axis(z.astype(np.float64), ids.cpu().numpy().astype(np.int64), 1))
    assert np.abs(host(w) - want).max() <= 1e-6
    ops.moe_top_logistic(dev(z, torch.float32), 3, True, ids, w)
    assert np.abs(host(w) - want / want.sum(1, keepdims=True)).max() <= 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_squared_ramp_in_the_products(dtype):
    from deliverance_amd.kernels import ops
    rng = np.random.default_rng(1)
    for M, N, K in ((3, 40, 64), (70, 136, 64), (300, 256, 128)):
        a, w = bf16(rng.normal(size=(M, K))), bf16(rng.normal(size=(N, K)) * 0.2)
        out = torch.empty(M, N, dtype=DTYPES[dtype], device=DEV)
        ops.linear(dev(a, DTYPES[dtype]), dev(w, DTYPES[dtype]), None, out, act="relu2")
        want = P.squared_ramp(a @ w.T)
        assert np.abs(host(out) - want).max() <= (1e-5 if dtype == "float32" else 2.0 ** -7) * np.abs(want).max()


# ------------------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def pmodels(tmp_path_factory):
    return {"P": make_model(tmp_path_factory.mktemp("pp"), CONFIG_P, 21), "Q": make_model(tmp_path_factory.mktemp("pq"), CONFIG_Q, 22),
            "R": make_model(tmp_path_factory.mktemp("pr"), CONFIG_R, 23)}


def check(model, got, routes, requests, dtype, what=""):
    """32-bit: every logit within 3e-5 of the largest plain logit.  bfloat16: the largest error within 5 % of the
    logits' root mean square and the rms error within 2^-6 of it.  The plain model follows the engine's choice of
    experts where two scores are nearly equal, and fails where the engine's choice is not nearly as good as its own."""
    for rid, ids in requests:
        ref = model.plain_logits(ids, routes.get(rid, {}), SLACK[dtype])
        out = got[rid].astype(np.float64)
        assert out.shape == ref.shape, f"{what} {rid}: shape {out.shape} vs {ref.shape}"
        err = np.abs(out - ref)
        rms = float(np.sqrt((ref ** 2).mean()))
        bound = 3e-5 * np.abs(ref).max() if dtype == "float32" else 5e-2 * rms
        first = int(np.argmax(err.max(axis=1) > bound))
        assert err.max() <= bound, f"{what} {rid} ({dtype}): max error {err.max():.3e} > {bound:.3e}, first at position {first}"
        if dtype == "bfloat16":
            assert float(np.sqrt((err ** 2).mean())) <= 2.0 ** -6 * rms, f"{what} {rid}: rms error"


def run(model, session, steps, requests, dtype, what):
    got, routes = replay_routed(session, steps, model.cfg)
    check(model, got, routes, requests, dtype, what)
    return got


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("P"), "Q", "R"])
def test_whole_prompts_and_first_tokens(pmodels, name, dtype):
    m = pmodels[name]
    reqs = [("one", m.prompt(1)), ("two", m.prompt(2)), ("three", m.prompt(3)), ("long", m.prompt(90))]
    s = helpers.trace_session(m.folder, dtype, 256)
    for rid, ids in reqs:
        run(m, s, helpers.trace_whole(rid, ids), [(rid, ids)], dtype, "whole")
    s.cache.manager.check()


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["P", quick("Q"), "R"])
def test_prefill_against_token_by_token_decoding(pmodels, name, dtype):
    """All but the last 45 tokens at once, the rest one by one, across page borders and tiles of keys; then a
    request that is decoded from its very first token on."""
    m = pmodels[name]
    ids = m.prompt(75, salt=1)
    s = helpers.trace_session(m.folder, dtype, 128)
    run(m, s, helpers.trace_bulk_then_single("r", ids, tail=45), [("r", ids)], dtype, "decode")
    ids2 = m.prompt(20, salt=2)
    run(m, s, helpers.trace_bulk_then_single("q", ids2, tail=19), [("q", ids2)], dtype, "decode from 1")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", [quick("P"), "Q", "R"])
@pytest.mark.parametrize("sizes", [(7, 2, 13, 3, 5, 2), quick((2, 2, 31, 1, 16, 33, 2))])
def test_portions_of_any_size(pmodels, name, dtype, sizes):
    m = pmodels[name]
    ids = m.prompt(97, salt=3)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True)
    run(m, s, helpers.trace_portions("r", ids, sizes), [("r", ids)], dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", ["float32", quick("bfloat16")])
@pytest.mark.parametrize("name", ["P", "Q", quick("R")])
def test_mixed_batches_over_a_small_pool(pmodels, name, dtype):
    """Seven unequal requests, four live at a time, over a pool that holds just what is live and four state slots:
    pages and slots come back and go out again (freed pages are filled with NaN).  Then some of them alone: what
    a request gets must not depend on its neighbours beyond rounding."""
    m = pmodels[name]
    reqs = [(f"r{i}", m.prompt(n, salt=10 + i)) for i, n in enumerate((40, 3, 71, 18, 64, 1, 33))]
    steps = helpers.trace_mixed(reqs, seed=5, max_live=4)
    s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True, state_slots=4)
    got = run(m, s, steps, reqs, dtype, "mixed")
    s.cache.manager.check()
    if dtype == "float32":
        alone = helpers.trace_session(m.folder, dtype, 128)
        for rid, ids in reqs[:3]:
            one = helpers.replay(alone, helpers.trace_whole(rid, ids))[rid]
            scale = float(np.sqrt((one.astype(np.float64) ** 2).mean()))
            assert np.abs(one.astype(np.float64) - got[rid]).max() <= 2e-5 * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, dtype):
    """Three hundred tokens one by one beside a neighbour that comes and goes, in a model whose layers use all of their
    experts (nothing hangs on a choice) and whose scan's decays are slow, so that the state remembers hundreds of
    tokens."""
    helpers.skip_in_simulation_if(True)
    cfg = {"architecture": "Pedatar", "vocab": 90, "width": 40, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.5},
           "layers": [scan_layer(scan(56, 8, 4, 3), moe(2, 2, 24, shared=8)),
                      att_layer(latent(2, 8, 16, 8, 16, 24, 0.3, 10000.0), moe(3, 3, 16)),
                      scan_layer(scan(56, 8, 4, 3), moe(2, 2, 24, shared=8), weights_of=0)]}
    m = make_model(tmp_path / "m", cfg, 31)
    ids, other = m.prompt(310, salt=20), m.prompt(60, salt=21)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:10], "want": list(range(10))}], "end": []}]
    for i in range(10, len(ids)):
        entries = [{"id": "a", "tokens": [ids[i]], "want": [0]}]
        j = i - 50
        if 0 <= j < len(other):
            entries.append({"id": "b", "tokens": [other[j]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["b"] if j == len(other) - 1 else []})
    steps[-1]["end"].append("a")
    s = helpers.trace_session(m.folder, dtype, 448, poison_freed=True, state_slots=2)
    got = helpers.replay(s, steps)
    check(m, got, {}, [("a", ids), ("b", other)], dtype, "long decode")


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_engine(pmodels, name, dtype):
    """The engine's own entry point and scheduler: several prompts at once over a pool that forces portions, with
    recorded decode steps and steps launched ahead.  Every generated token must be (nearly) the best under the plain
    model given the tokens before it; in 32-bit, where a choice of experts cannot flip, it is the plain model's token."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = pmodels[name]
    prompts = [m.prompt(n, salt=30 + n) for n in (5, 33, 70, 2)]
    model = AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=512, max_num_seqs=3,
                                                 max_batch_tokens=48, max_chunk=32)
    outs = model.generate(prompts, GeneratorParameters(max_tokens=24, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.finish_reason == "length" and len(out.generated_tokens) == 24
        ids = list(prompt) + list(out.generated_tokens)
        ref = m.plain_logits(ids)
        margins = P.forward(m.plain_cfg, m.W, ids, with_margins=True)[1]
        for k, t in enumerate(out.generated_tokens):
            row = ref[len(prompt) + k - 1]
            if dtype == "float32":
                assert t == int(np.argmax(row)) or row[t] >= row.max() - 1e-4
            elif margins > 0.05:                      # no choice of experts hangs on a hair in this sequence
                assert row[t] >= row.max() - 2 * 5e-2 * float(np.sqrt((row ** 2).mean()))


# ------------------------------------------------------------------------------------------ random configurations
def random_config(seed):
    """Sizes drawn at random, among them what the kernels take only on their plain paths (widths and ranks that are no
    multiple of 8, rows that the matrix-core attention does not take), one expert, as many experts a token as there
    are, one tap, layers on another layer's weights in any order."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    width = pick(40, 50, 64, 100, 72, 36)
    layers = []
    for i in range(int(rng.integers(1, 5))):
        n = pick(1, 2, 5, 9)
        mlp = pick(None, "moe", "moe", "moe")
        if mlp == "moe":
            mlp = moe(n, pick(1, n, max(1, n // 2)), pick(8, 20, 32), pick(None, 8, 24))
        same = [j for j, L in enumerate(layers) if "weights_of" not in L]
        if same and rng.random() < 0.3:
            j = same[int(rng.integers(0, len(same)))]
            layers.append(dict(layers[j], weights_of=j))
        elif rng.random() < 0.5:
            dr = pick(2, 8, 16, 24)
            layers.append(att_layer(latent(pick(1, 2, 3, 6), pick(8, 16, 20, 32), dr, pick(8, 16, 40), pick(8, 12, 32), pick(8, 24, 30, 64),
                                           float(pick(0.1, 0.25, 0.4)), float(pick(100.0, 10000.0, 1e6)), dims=pick(dr, dr, 2, 0)), mlp))
        else:
            layers.append(scan_layer(scan(pick(24, 50, 64, 128), pick(1, 4, 16, 33), pick(1, 3, 8), pick(1, 2, 4, 6)), mlp))
    return {"architecture": "Pedatar", "vocab": pick(50, 130, 257), "width": width, "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))},
            "embedding": {"scale": float(pick(1.0, 0.5, 4.0))}, "layers": layers}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(14))
def test_random_configurations(tmp_path, seed, dtype):
    m = make_model(tmp_path / "m", random_config(seed), 100 + seed)
    ids = m.prompt(45, salt=seed)
    s = helpers.trace_session(m.folder, dtype, 128, poison_freed=True, state_slots=2)
    run(m, s, helpers.trace_whole("w", ids), [("w", ids)], dtype, f"seed {seed} whole")
    run(m, s, helpers.trace_portions("p", ids, (5, 2, 17, 1, 1, 9)), [("p", ids)], dtype, f"seed {seed} portions")
