"""Pedatar without a GPU: its configuration, run order and shared weights, tensor declarations, the random-weights
mode, what its mixers ask of the cache, and the plain implementation against other ways of writing the same
formulas."""
import json

import numpy as np
import pytest
import torch

import plain_pedatar as P
from pedatar_models import CONFIG_P, CONFIG_Q, CONFIG_R


def test_config_reads_every_size_and_constant():
    from deliverance_amd.config import ConfigError, PedatarConfig
    from deliverance_amd.config.specs import ExpertsFeedForwardSpec, LatentAttentionSpec, SelectiveScanSpec
    mc = PedatarConfig.from_dict(CONFIG_Q).to_model_config()
    assert (mc.vocab_size, mc.width, mc.embed_scale) == (CONFIG_Q["vocab"], CONFIG_Q["width"], CONFIG_Q["embedding"]["scale"])
    assert mc.final_norm.kind == "rmsnorm" and mc.final_norm.gain_offset == 0.0 and mc.final_norm.eps == CONFIG_Q["norm"]["eps"]
    assert not mc.tie_word_embeddings and mc.embed_position.kind == "none"
    for spec, raw in zip(mc.layers, CONFIG_Q["layers"]):
        m, a = raw["mixer"], spec.mixer
        assert spec.pre_mixer_norm is not None and spec.post_mixer_norm is None and spec.post_ff_norm is None
        if raw["type"] == "latent_attention":
            assert isinstance(a, LatentAttentionSpec)
            assert (a.n_heads, a.head_dim, a.rot_dim, a.v_head_dim, a.q_rank, a.kv_rank, a.scale) == \
                (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"], m["scale"])
            assert (a.rotary.dims, a.rotary.base, a.rotary.interleaved, a.norm_eps) == (m["rot"]["dims"], m["rot"]["base"], True, CONFIG_Q["norm"]["eps"])
        else:
            assert isinstance(a, SelectiveScanSpec)
            assert (a.inner, a.state, a.dt_rank, a.conv_taps) == (m["inner"], m["state"], m["dt_rank"], m["conv"])
        if raw["mlp"] is None:
            assert spec.feed_forward is None and spec.pre_ff_norm is None
        else:
            f = spec.feed_forward
            assert isinstance(f, ExpertsFeedForwardSpec) and f.router == "logistic_top" and not f.gated
            assert f.weight_on == "input" and not f.renormalize and f.activation == "relu2"
            assert (f.inner, f.n_experts, f.top) == (raw["mlp"]["expert"]["ff"], raw["mlp"]["router"]["experts"], raw["mlp"]["router"]["top"])
            assert f.shared_inner == (raw["mlp"]["shared"]["ff"] if raw["mlp"]["shared"] else 0)
    # what is missing is named, all of it at once
    broken = json.loads(json.dumps(CONFIG_Q))
    del broken["embedding"]["scale"], broken["layers"][1]["mixer"]["rot"]["base"], broken["layers"][0]["mixer"]["conv"]
    del broken["layers"][2]["mlp"]["router"]["top"]
    with pytest.raises(ConfigError) as e:
        PedatarConfig.from_dict(broken)
    for key in ("embedding.scale", "layers[1].mixer.rot.base", "layers[0].mixer.conv", "layers[2].mlp.router.top"):
        assert key in str(e.value)
    other = json.loads(json.dumps(CONFIG_Q))
    other["layers"][0]["type"] = "attention"
    with pytest.raises(ConfigError, match="attention"):
        PedatarConfig.from_dict(other)
    other = json.loads(json.dumps(CONFIG_Q))
    other["layers"][1]["mixer"]["rot"]["dims"] = 14
    with pytest.raises(ConfigError, match="rot.dims"):
        PedatarConfig.from_dict(other)


def test_layers_on_another_layers_weights_keep_a_cache_of_their_own():
    from deliverance_amd.config import ConfigError, PedatarConfig
    mc = PedatarConfig.from_dict(CONFIG_P).to_model_config()
    assert len(mc.layers) == 2 and [s.weight_prefix for s in mc.layers] == ["l0.", "l1."]
    assert [(c.layer, c.cache, c.write) for c in mc.schedule] == [(0, 0, True), (1, 1, True), (0, 2, True), (1, 3, True)]
    assert mc.n_cache_slots == 4
    assert [p for _, p in P.layer_runs(CONFIG_P)] == [mc.layers[c.layer].weight_prefix for c in mc.schedule]
    # a layer in the middle may lend its weights to one in front of it, and borrowed weights may be lent on
    cfg = json.loads(json.dumps(CONFIG_P))
    cfg["layers"] = [dict(cfg["layers"][1], weights_of=3), cfg["layers"][0], dict(cfg["layers"][0], weights_of=1),
                     {k: v for k, v in cfg["layers"][1].items() if k != "weights_of"}, dict(cfg["layers"][1], weights_of=0)]
    mc = PedatarConfig.from_dict(cfg).to_model_config()
    assert [s.weight_prefix for s in mc.layers] == ["l1.", "l3."]
    assert [(c.layer, c.cache) for c in mc.schedule] == [(1, 0), (0, 1), (0, 2), (1, 3), (1, 4)]
    bad = json.loads(json.dumps(CONFIG_P))
    bad["layers"][2]["mixer"]["vdim"] += 8
    with pytest.raises(ConfigError, match="differs"):
        PedatarConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIG_P))
    bad["layers"][2]["weights_of"] = 2
    with pytest.raises(ConfigError, match="weights_of"):
        PedatarConfig.from_dict(bad)
    bad["layers"][2]["weights_of"], bad["layers"][0]["weights_of"] = 0, 2
    with pytest.raises(ConfigError, match="circle"):
        PedatarConfig.from_dict(bad)


@pytest.mark.parametrize("cfg", [CONFIG_P, CONFIG_Q, CONFIG_R])
def test_random_model_goes_through_the_loader_and_the_registry(tmp_path, cfg):
    from deliverance_amd.models.causal_lm import load_model
    from deliverance_amd.parts import KVNeed, StateNeed
    from deliverance_amd.random_model import random_model
    from deliverance_amd.registry import ModelSupport, read_config_json
    from deliverance_amd.weights.loader import WeightError
    folder = random_model(str(tmp_path / "m"), cfg, 3)
    assert ModelSupport.detect(read_config_json(folder)).name == "Pedatar"
    model = load_model(folder, torch.float32, "cpu")
    needs = model.cache_needs()
    assert sorted(needs) == list(range(len(cfg["layers"])))
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] == "latent_attention":           # one row a token: the latent and the key piece, nothing per head
            assert needs[i] == KVNeed(1, m["kv_rank"] + m["rot_dim"], None, m["kv_rank"], values_in_keys=True)
        else:
            assert needs[i] == StateNeed(m["inner"] * m["state"] + (m["conv"] - 1) * m["inner"])
    assert model.graph_safe
    # the stored tensors are the design's names, none more and none less
    cfg_read, W = P.read_model_folder(folder)
    own = [i for i, L in enumerate(cfg["layers"]) if "weights_of" not in L]
    assert {n.split(".")[0] for n in W} == {"embed", "head", "final"} | {f"l{i}" for i in own}
    from safetensors.torch import load_file, save_file
    t = load_file(str(tmp_path / "m" / "model.safetensors"))
    t["l0.extra"] = torch.zeros(3)
    del t["final.norm"]
    save_file(t, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_model(folder, torch.float32, "cpu")
    assert "final.norm" in str(e.value) and "l0.extra" in str(e.value)


def test_cache_bytes_count_a_latent_row_once():
    from deliverance_amd.engine.device_cache import DeviceCache
    from deliverance_amd.parts import KVNeed, StateNeed
    needs = {0: KVNeed(1, 48, None, 40, values_in_keys=True), 1: StateNeed(100), 2: KVNeed(1, 48, None, 40, values_in_keys=True),
             3: KVNeed(2, 16)}
    cache = DeviceCache(needs, torch.bfloat16, "cpu", 16, 64, n_state_slots=3)
    assert cache.bytes_per_token() == 2 * 48 * 2 + 2 * 2 * 16 * 2
    assert tuple(cache.kv[0].shape) == (4, 16 * 48) and tuple(cache.kv[3].shape) == (4, 2, 2, 16, 16)
    assert cache.group_of_slot[0] == cache.group_of_slot[2] != cache.group_of_slot[3]
    assert tuple(cache.state[1].shape) == (3, 100) and cache.state[1].dtype == torch.float32
    assert DeviceCache.tokens_for_budget(needs, torch.bfloat16, 3 * 400 + 10 * (2 * 96 + 128), 3) == 10


# ------------------------------------------------------------------------------------------ the plain model itself
def test_plain_latent_attention_equals_the_folded_form():
    """Scores against the unfolded keys equal the folded queries against the cached rows; the values' map can be
    applied to the weighted sum of latents."""
    rng = np.random.default_rng(0)
    m = {"heads": 3, "dim": 8, "rot_dim": 6, "vdim": 10, "q_rank": 7, "kv_rank": 12, "scale": 0.3, "rot": {"base": 50.0, "dims": 4}}
    E, T, H = 20, 9, 3
    W = {"mix.dq": rng.normal(size=(7, E)), "mix.dq.norm": rng.normal(size=7), "mix.uq": rng.normal(size=(H * 14, 7)),
         "mix.dkv": rng.normal(size=(18, E)), "mix.dkv.norm": rng.normal(size=12), "mix.uk": rng.normal(size=(H * 8, 12)),
         "mix.uv": rng.normal(size=(H * 10, 12)), "mix.o": rng.normal(size=(E, H * 10))}
    h = rng.normal(size=(T, E))
    want = P.latent_attention(W, "", m, h, 1e-5)
    cq = P.unit_rms(h @ W["mix.dq"].T, W["mix.dq.norm"], 1e-5)
    q = (cq @ W["mix.uq"].T).reshape(T, H, 14)
    down = h @ W["mix.dkv"].T
    rows = np.concatenate([P.unit_rms(down[:, :12], W["mix.dkv.norm"], 1e-5), P.turn_pairs(down[:, 12:], np.arange(T), 4, 50.0)], axis=1)
    out = np.zeros((T, H, 10))
    for head in range(H):
        fold = np.concatenate([q[:, head, :8] @ W["mix.uk"][head * 8:head * 8 + 8], P.turn_pairs(q[:, head, 8:], np.arange(T), 4, 50.0)], axis=1)
        for t in range(T):
            s = fold[t] @ rows[:t + 1].T * 0.3
            w = np.exp(s - s.max())
            out[t, head] = W["mix.uv"][head * 10:head * 10 + 10] @ ((w / w.sum()) @ rows[:t + 1, :12])
    assert np.abs(out.reshape(T, -1) @ W["mix.o"].T - want).max() < 1e-9


def test_plain_scan_in_two_halves_and_filter_by_hand():
    rng = np.random.default_rng(1)
    T, I, N = 11, 5, 3
    x, step = rng.normal(size=(T, I)), np.abs(rng.normal(size=(T, I)))
    A, B, C, D = -np.abs(rng.normal(size=(I, N))), rng.normal(size=(T, N)), rng.normal(size=(T, N)), rng.normal(size=I)
    y = P.selective_scan(x, step, A, B, C, D)
    # the closed form of the last output: every input's contribution decays by the step sizes behind it
    last = D * x[-1]
    for t in range(T):
        decay = np.exp(A * step[t + 1:].sum(axis=0)[:, None])
        last = last + (decay * (step[t] * x[t])[:, None] * B[t][None, :]) @ C[-1]
    assert np.abs(y[-1] - last).max() < 1e-9
    taps, bias = rng.normal(size=(I, 4)), rng.normal(size=I)
    f = P.short_filter(x, taps, bias)
    assert np.allclose(f[0], bias + taps[:, 3] * x[0]) and np.allclose(f[5], bias + (taps * x[2:6].T).sum(axis=1))


def test_plain_routing_weights_the_input_and_follows_a_given_choice_only_when_it_is_close():
    rng = np.random.default_rng(2)
    E = 6
    W = {"mlp.router": np.array([[1.0] + [0] * 5, [0.99] + [0] * 5, [-1.0] + [0] * 5])}
    for e in range(3):
        W[f"mlp.e{e}.up"], W[f"mlp.e{e}.down"] = rng.normal(size=(4, E)), rng.normal(size=(E, 4))
    mlp = {"router": {"experts": 3, "top": 1}, "shared": None}
    h = np.array([[2.0, 1, 0, -1, 3, 0.5]])
    s = P.logistic(2.0)
    assert np.allclose(P.routed_ff(W, "", mlp, h), W["mlp.e0.down"] @ np.square(np.maximum(W["mlp.e0.up"] @ (s * h[0]), 0)))
    # the square of the ramp makes the weight on the input a squared weight on the output
    assert np.allclose(P.routed_ff(W, "", mlp, h), s * s * P.small_ff(W, "mlp.e0.", h))
    s1 = P.logistic(1.98)
    assert np.allclose(P.routed_ff(W, "", mlp, h, given=[[1]], slack=0.05), s1 * s1 * P.small_ff(W, "mlp.e1.", h))
    with pytest.raises(P.FarChoice):
        P.routed_ff(W, "", mlp, h, given=[[1]], slack=0.001)
    with pytest.raises(P.FarChoice):
        P.routed_ff(W, "", mlp, h, given=[[2]], slack=0.05)
    assert abs(P.router_margin(W, "", mlp, h)[0] - (s - s1)) < 1e-12
