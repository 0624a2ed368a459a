"""The Podurax design without a GPU: its configuration, its plan, the tensors it declares, the cache's kept first pages
against the plain cache manager, and the plain implementation's own mechanisms against independent formulas."""
import math
import random

import numpy as np
import pytest

import plain_cache_manager as plain_cm
import plain_podurax as pp
import podurax_models as pm
from inferflux_amd.cache import CacheManager, GroupSpec
from inferflux_amd.cache.storage import plan_groups
from inferflux_amd.config import ConfigError, PoduraxConfig, config_from_dict, load_config, plan_for
from inferflux_amd.engine.model import Model


def test_config_reads_every_layer_and_roundtrips(tmp_path):
    for name in pm.CONFIGS:
        d = pm.config(name)
        cfg = config_from_dict(d)
        assert isinstance(cfg, PoduraxConfig) and (cfg.vocab, cfg.width) == (d["vocab"], d["width"])
        assert (cfg.norm_eps, cfg.embedding_scale, cfg.residual_mult) == (d["norm"]["eps"], d["embedding"]["scale"], d["residual_mult"])
        for L, want in zip(cfg.layers, d["layers"]):
            m = want["mixer"]
            assert L.type == want["type"] and (L.mlp is None) == (want["mlp"] is None)
            if L.type == "attention":
                mask = m.get("mask") or {}
                assert (L.mixer.heads, L.mixer.kv_heads, L.mixer.dim, L.mixer.vdim, L.mixer.scale, L.mixer.v_mix) == \
                       (m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], m["v_mix"])
                assert (L.mixer.window, L.mixer.keep_first) == (mask.get("size"), mask.get("keep_first", 0))
                assert (L.mixer.rot_base, L.mixer.rot_dims) == (m["rot"]["base"], m["rot"]["dims"])
                assert (L.mixer.rot_scaling is None) == ("scaling" not in m["rot"])
            else:
                assert (L.mixer.inner, L.mixer.state, L.mixer.dt_rank, L.mixer.conv) == (m["inner"], m["state"], m["dt_rank"], m["conv"])
        cfg.save(str(tmp_path / name))
        assert load_config(str(tmp_path / name)) == cfg


@pytest.mark.parametrize("path,value,match", [
    (("layers", 0, "mixer", "heads"), None, r"layers\[0\]\.mixer\.heads"),
    (("layers", 0, "mixer", "kv_heads"), 3, "multiple"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "even"),
    (("layers", 0, "mixer", "rot", "dims"), 64, "within"),
    (("layers", 0, "mixer", "rot", "scaling", "factor"), 0.0, "positive"),
    (("layers", 0, "mixer", "mask", "size"), 0, "positive"),
    (("layers", 0, "mixer", "mask", "keep_first"), -1, "negative"),
    (("layers", 2, "mixer", "vdim"), 16, "agree"),
    (("layers", 1, "mixer", "conv"), 17, "taps"),
    (("layers", 1, "mixer", "state"), 0, "positive"),
    (("layers", 0, "mlp", "kind"), "moe", "not supported"),
    (("layers", 0, "type"), "mamba9", "known mixer"),
    (("norm",), None, "norm"),
    (("residual_mult",), "half", "residual_mult"),
    (("layers",), [], "non-empty"),
])
def test_bad_configs_name_the_key(path, value, match):
    d = pm.config("A")
    node = d
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ConfigError, match=match):
        config_from_dict(d)


def test_plan_builds_every_layer_from_its_own_entry():
    cfg = config_from_dict(pm.config("A"))
    plan = plan_for(cfg)
    kinds = [L.mixer.kind for L in plan.layers]
    assert kinds == ["paged_attention", "selective_ssm", "paged_attention", "paged_attention", "paged_attention"]
    assert [L.block.args["residual_scale"] for L in plan.layers] == [0.5] * 5 and plan.embedding.args["scale"] == 2.0
    assert [L.ffn is None for L in plan.layers] == [False, False, True, False, False]
    # the first layer that mixes values hands them on, the later ones mix them in, a layer that does not mix does neither
    assert [L.mixer.args.get("value_mix") for L in plan.layers] == ["source", None, "mix", None, "mix"]
    a0 = plan.layers[0].mixer.args
    assert (a0["window"], a0["keep_first"], a0["sink"], a0["unit_norm_eps"], a0["output_gate"]) == (20, 3, 0.0, 1e-5, True)
    assert a0["position"].args["scaling"] == {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    model = Model(cfg)
    names = set(model.param_specs())
    assert {"embed", "final.norm", "head", "l0.mix.q.b", "l0.mix.vmix", "l0.mix.g", "l1.mix.A_log", "l1.mix.conv.b", "l1.mix.dt.b",
            "l2.mix.vmix", "l4.mlp.down"} <= names
    assert "l2.norm2" not in names and "l3.mix.vmix" not in names and not any(n.startswith("l2.mlp") for n in names)
    assert model.param_specs()["l1.mix.x"].shape == (5 + 2 * 6, 96) and model.param_specs()["l0.mix.vmix"].shape == ()
    # cache groups: everything kept, and the two windows with their kept first tokens; the recurrence owns state, no pages
    groups, entry_group = plan_groups(plan.schedule, model.schedule_mixers())
    assert [(g.window, g.keep_first, g.entries) for g in groups] == [(None, 0, (3,)), (20, 3, (0,)), (33, 5, (2, 4))]
    assert 1 not in entry_group and model.schedule_mixers()[1].cache_spec() is None
    assert model.schedule_mixers()[1].state_spec().shape == (96 * 3 + 96 * 6,)
    assert model.graph_safe


def _both(pages, window, keep, slots=4, page_size=16):
    spec = [GroupSpec(None, (0,)), GroupSpec(window, (1,), keep)]
    return CacheManager(spec, page_size, pages, slots), plain_cm.CacheManager([plain_cm.GroupSpec(None, (0,)), plain_cm.GroupSpec(window, (1,), keep)],
                                                                            page_size, pages, slots)


def test_kept_first_pages_stay_while_the_window_moves_on():
    m, _ = _both(pages=20, window=40, keep=20)
    m.add("a")
    for n in (30, 1, 1, 70, 16, 1, 100):
        m.reserve("a", n)
        m.commit("a", n)
        m.check()
    length = m.length("a")
    table = m.block_table("a", 1)
    first_needed = (length - 40 + 1) // 16
    assert table[0] >= 0 and table[1] >= 0                                   # positions 0..19 live in blocks 0 and 1
    assert all(p < 0 for p in table[2:first_needed]) and all(p >= 0 for p in table[first_needed:])
    assert all(p >= 0 for p in m.block_table("a", 0))
    m.free("a")
    assert m.free_pages() == [20, 20]


@pytest.mark.parametrize("seed", range(6))
def test_native_manager_follows_the_plain_one_with_kept_first_pages(seed):
    rng = random.Random(300 + seed)
    m, p = _both(pages=rng.choice([8, 12, 17]), window=rng.choice([24, 40, 7]), keep=rng.choice([1, 6, 16, 17, 50]))
    live, next_id = [], 0
    for _ in range(400):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            m.add(next_id); p.add(next_id); live.append(next_id); next_id += 1
        elif op < 0.85 and live:
            rid, n = rng.choice(live), rng.choice([1, 1, 1, 2, 5, 16, 31, 70])
            assert m.pages_needed(rid, n) == p.pages_needed(rid, n)
            outcome = []
            for mgr, exc in ((m, Exception), (p, Exception)):
                try:
                    mgr.reserve(rid, n)
                    outcome.append("ok")
                except exc as e:
                    outcome.append((e.group, e.needed, e.free))
            assert outcome[0] == outcome[1]
            if outcome[0] == "ok":
                m.commit(rid, n); p.commit(rid, n)
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.free(rid); p.free(rid)
        m.check(); p.check()
        for rid in live:
            a, b = m.get(rid), p.get(rid)
            assert (a.length, a.reserved, a.tables) == (b.length, b.reserved, b.tables), rid


# ---- the plain implementation's own mechanisms against independent formulas -------------------------------
def test_visibility_is_causal_windowed_and_keeps_the_first():
    see = lambda i, size, keep: [j for j in range(i + 3) if pp.visible(i, j, size, keep)]
    assert see(5, None, 0) == [0, 1, 2, 3, 4, 5]
    assert see(9, 4, 0) == [6, 7, 8, 9]
    assert see(9, 4, 2) == [0, 1, 6, 7, 8, 9]
    assert see(3, 4, 2) == [0, 1, 2, 3] and see(9, 4, 8) == [0, 1, 2, 3, 4, 5, 6, 7, 8, 9] and see(0, 1, 0) == [0]


def test_sink_softmax_is_a_softmax_over_the_keys_and_a_zero():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(7, 2, 6)), rng.normal(size=(7, 1, 6)), rng.normal(size=(7, 1, 5))
    out = pp.sink_softmax_attention(q, k, v, 0.7, 3, 1)
    for i in (0, 2, 6):
        for h in range(2):
            js = [j for j in range(7) if pp.visible(i, j, 3, 1)]
            s = np.array([0.0] + [0.7 * float(q[i, h] @ k[j, 0]) for j in js])       # the sink's score first
            w = np.exp(s) / np.exp(s).sum()
            assert np.allclose(out[i, h], sum(w[1 + n] * v[j, 0] for n, j in enumerate(js)))
            assert 0 < w[0] < 1
    # position 0 alone: its own value times exp(s) / (1 + exp(s))
    s0 = 0.7 * float(q[0, 0] @ k[0, 0])
    assert np.allclose(out[0, 0], v[0, 0] * math.exp(s0) / (1 + math.exp(s0)))


def test_stretched_frequencies_keep_the_fast_pairs_and_stretch_the_slow():
    f, mag = pp.yarn_frequencies(24, 5e5, {"factor": 6.0, "original": 2048, "fast": 24.0, "slow": 1.0})
    plain_f, one = pp.yarn_frequencies(24, 5e5, None)
    assert one == 1.0 and np.allclose(plain_f, [5e5 ** (-2 * i / 24) for i in range(12)])
    assert np.isclose(mag, 0.1 * math.log(6.0) + 1.0)
    assert np.allclose(f[0], plain_f[0]) and np.allclose(f[-1], plain_f[-1] / 6.0)          # the ends of the ramp
    assert all(b / 6.0 - 1e-18 <= a <= b + 1e-18 for a, b in zip(f, plain_f)) and list(f) == sorted(f, reverse=True)
    x = np.random.default_rng(1).normal(size=(3, 2, 30))
    y = pp.rotate(x, np.array([0, 5, 900]), 24, 5e5, {"factor": 6.0, "original": 2048, "fast": 24.0, "slow": 1.0})
    assert np.allclose(y[..., 24:], x[..., 24:])                                             # the rest passes unchanged
    assert np.allclose((y[..., :24] ** 2).sum(-1), mag ** 2 * (x[..., :24] ** 2).sum(-1))    # a rotation, lengthened by the factor


def test_the_recurrence_cut_anywhere_carries_on_from_its_state():
    rng = np.random.default_rng(2)
    T, C, N = 23, 5, 3
    x, dt, B, Cm = rng.normal(size=(T, C)), np.abs(rng.normal(size=(T, C))) * 0.3, rng.normal(size=(T, N)), rng.normal(size=(T, N))
    A, D = -np.abs(rng.normal(size=(C, N))) - 0.1, rng.normal(size=C)
    y = pp.selective_scan(x, dt, A, B, Cm, D)
    # by the closed form: S_t = sum_{s <= t} exp(A * sum_{s < r <= t} dt_r) dt_s x_s B_s
    t = 17
    S = np.zeros((C, N))
    for s in range(t + 1):
        S += np.exp(A * dt[s + 1:t + 1].sum(0)[:, None]) * (dt[s] * x[s])[:, None] * B[s][None, :]
    assert np.allclose(y[t], S @ Cm[t] + D * x[t])
    conv = pp.causal_conv(x, rng.normal(size=(C, 4)), np.zeros(C))
    assert conv.shape == (T, C)
    w = rng.normal(size=(C, 4))
    full = pp.causal_conv(x, w, np.ones(C))
    assert np.allclose(full[0], 1.0 + w[:, 3] * x[0]) and np.allclose(full[5], 1.0 + sum(w[:, j] * x[5 - 3 + j] for j in range(4)))


def test_the_whole_model_changes_when_a_mechanism_is_left_out(tmp_path):
    """What the engine's tests rely on: every mechanism moves the plain model's logits by far more than rounding."""
    folder = pm.write_model(str(tmp_path / "m"), pm.config("A"), 5, gain=2.0)
    cfg, W = pm.load_plain(folder)
    ids = list(np.random.default_rng(3).integers(0, 300, size=60))
    base = pp.forward(cfg, W, ids)
    scale = np.abs(base).max()

    def changed(edit):
        c2 = pm.config("A")
        edit(c2)
        return np.abs(pp.forward(c2, W, ids) - base).max() / scale

    assert changed(lambda c: c["layers"][0]["mixer"]["mask"].update(size=21)) > 1e-3
    assert changed(lambda c: c["layers"][0]["mixer"]["mask"].update(keep_first=4)) > 1e-3
    assert changed(lambda c: c["layers"][2]["mixer"].update(v_mix=False)) > 1e-3
    assert changed(lambda c: c["layers"][0]["mixer"]["rot"].pop("scaling")) > 1e-3
    assert changed(lambda c: c.update(residual_mult=0.51)) > 1e-3
    assert changed(lambda c: c["embedding"].update(scale=2.1)) > 1e-3
    W2 = dict(W)
    W2["l1.mix.A_log"] = W["l1.mix.A_log"] + 0.5
    assert np.abs(pp.forward(cfg, W2, ids) - base).max() / scale > 1e-3


def test_random_weights_folder_roundtrips_with_its_scalar_tensors(tmp_path):
    """The seeded random-weights mode writes every tensor the plan declares, the scalar mixing weights among them, with
    decays and step-size biases in the range a recurrence needs; the folder reads back equal and its config reloads."""
    import torch
    from safetensors.torch import load_file
    from inferflux_amd.weights import write_random_model
    from inferflux_amd.weights.safetensors_io import open_model_files
    cfg = config_from_dict(pm.config("A"))
    folder = str(tmp_path / "m")
    write_random_model(folder, cfg, seed=3)
    assert load_config(folder) == cfg
    t = load_file(folder + "/model.safetensors")
    assert set(t) == set(Model(cfg).param_specs())
    assert t["l0.mix.vmix"].shape == () and 0.2 <= float(t["l2.mix.vmix"]) <= 0.8
    assert float(t["l1.mix.A_log"].float().exp().min()) >= 0.99 and float(t["l1.mix.dt.b"].float().max()) <= -0.99
    files = open_model_files(folder)
    mine = files[0].tensor("l2.mix.vmix") if hasattr(files[0], "tensor") else None
    if mine is not None:
        assert torch.equal(mine, t["l2.mix.vmix"])
    write_random_model(str(tmp_path / "again"), cfg, seed=3)
    assert all(torch.equal(v, load_file(str(tmp_path / "again") + "/model.safetensors")[k]) for k, v in t.items())
