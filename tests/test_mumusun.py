"""The Mumusun design without a GPU: its configuration, its plan, the tensors it declares, and the plain
implementation's own mechanisms against independent formulas."""
import copy
import math

import pytest
import torch

import mumusun_models as mm
import plain_mumusun as pm
from inferflux_amd.cache.storage import plan_groups
from inferflux_amd.config import ConfigError, MumusunConfig, config_from_dict, load_config, plan_for
from inferflux_amd.engine.model import Model


def test_config_reads_every_layer_and_roundtrips(tmp_path):
    for name in mm.CONFIGS:
        d = mm.config(name)
        cfg = config_from_dict(d)
        assert isinstance(cfg, MumusunConfig) and cfg.vocab == d["vocab"] and cfg.width == d["width"]
        assert cfg.norm_eps == d["norm"]["eps"] and len(cfg.layers) == len(d["layers"])
        for L, want in zip(cfg.layers, d["layers"]):
            m = want["mixer"]
            assert (L.mixer.heads, L.mixer.dim, L.mixer.rot_dim, L.mixer.vdim, L.mixer.q_rank, L.mixer.kv_rank) == \
                   (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"])
            assert L.mixer.scale == m["scale"] and L.mixer.rot_base == m["rot"]["base"] and L.mixer.rot_dims == m["rot"]["dims"]
            assert L.mixer.window == (m.get("mask") or {}).get("size")
            if want["mlp"] is None:
                assert L.mlp is None
            else:
                r = want["mlp"]["router"]
                assert (L.mlp.ff, L.mlp.experts, L.mlp.top, L.mlp.groups, L.mlp.keep_groups) == \
                       (want["mlp"]["expert"]["ff"], r["experts"], r["top"], r["groups"]["count"], r["groups"]["keep"])
        cfg.save(str(tmp_path / name))
        assert load_config(str(tmp_path / name)) == cfg


@pytest.mark.parametrize("path,value,match", [
    (("layers", 0, "mixer", "heads"), None, r"layers\[0\]\.mixer\.heads"),
    (("layers", 1, "mixer", "rot", "dims"), 7, "even"),
    (("layers", 0, "mixer", "rot", "dims"), 64, "within"),
    (("layers", 0, "mixer", "mask", "size"), 0, "positive"),
    (("layers", 0, "mlp", "router", "top"), 7, "exceeds"),
    (("layers", 0, "mlp", "router", "groups", "count"), 3, "multiple"),
    (("layers", 0, "mlp", "kind"), "dense", "not supported"),
    (("layers", 0, "type"), "recurrent", "known mixer"),
    (("norm",), None, "norm"),
    (("width",), "64", "width"),
    (("layers",), [], "non-empty"),
])
def test_bad_configs_name_the_key(path, value, match):
    d = mm.config("P")
    node = d
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    with pytest.raises(ConfigError, match=match):
        config_from_dict(d)


def test_plan_builds_each_layer_from_its_own_entry():
    cfg = config_from_dict(mm.config("P"))
    plan = plan_for(cfg)
    assert [l.block.kind for l in plan.layers] == ["outnorm"] * 3
    assert [l.mixer.args["window"] for l in plan.layers] == [20, 33, None]
    assert plan.layers[1].ffn is None and plan.layers[1].norm_post is None
    assert plan.layers[1].mixer.args["position"].args == {"head_dim": 16, "rotary_dim": 8, "theta": 500.0, "style": "split_half"}
    assert plan.layers[0].ffn.args["groups"] == 4 and plan.layers[0].ffn.args["keep_groups"] == 2
    model = Model(cfg)
    groups, entry_group = plan_groups(plan.schedule, model.schedule_mixers())
    assert [g.window for g in groups] == [None, 20, 33] and entry_group == {2: 0, 0: 1, 1: 2}
    spec = model.schedule_mixers()[0].cache_spec()
    assert (spec.n_kv_heads, spec.k_dim, spec.v_dim, spec.window) == (1, 32 + 8, 32, 20)     # the latent and the shared rotated part
    assert model.graph_safe


def test_declared_tensors():
    specs = Model.param_specs_for(config_from_dict(mm.config("Q")))
    assert specs["embed"].shape == (131, 88) and specs["head"].shape == (131, 88) and specs["final.norm"].shape == (88,)
    assert specs["l0.mix.dq"].shape == (36, 88) and specs["l0.mix.dq.norm"].shape == (36,)
    assert specs["l0.mix.uq"].shape == (1 * (20 + 12), 36) and specs["l0.mix.dkv"].shape == (44 + 12, 88)
    assert specs["l0.mix.uk"].shape == (20, 44) and specs["l0.mix.uv"].shape == (28, 44) and specs["l0.mix.o"].shape == (88, 28)
    assert specs["l1.mlp.router"].shape == (4, 88) and specs["l1.mlp.e3.down"].shape == (88, 24)
    assert "l0.mlp.e9.gate" not in specs and "l0.mlp.e8.gate" in specs
    assert len(specs) == 3 + 2 * 10 + 1 + 27 + 1 + 12


# ---- the plain implementation's mechanisms against other formulas -------------------------------
def test_plain_norms():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 37, generator=g, dtype=torch.float64) + 2.0, torch.randn(37, generator=g, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (37,), w, None, 1e-3)
    assert torch.allclose(pm.layer_norm(x, w, 1e-3), want, atol=1e-12)
    r = pm.rms_norm(x, w, 1e-3)
    assert torch.allclose(r[2], x[2] * w / math.sqrt(float((x[2] ** 2).mean()) + 1e-3), atol=1e-12)


def test_plain_rotation_turns_pairs_and_leaves_the_rest():
    x = torch.arange(2 * 1 * 10, dtype=torch.float64).view(2, 1, 10) + 1
    y = pm.rotate(x, [0, 3], 6, 100.0)
    assert torch.equal(y[0], x[0]) and torch.equal(y[1, 0, 6:], x[1, 0, 6:])
    for i in range(3):
        a = 3 * 100.0 ** (-2 * i / 6)
        u, v = float(x[1, 0, i]), float(x[1, 0, i + 3])
        assert abs(float(y[1, 0, i]) - (u * math.cos(a) - v * math.sin(a))) < 1e-12
        assert abs(float(y[1, 0, i + 3]) - (v * math.cos(a) + u * math.sin(a))) < 1e-12
    # a rotation of q and k by their positions leaves a score that depends on the distance alone
    q, k = torch.randn(1, 1, 6, dtype=torch.float64), torch.randn(1, 1, 6, dtype=torch.float64)
    s1 = (pm.rotate(q, [9], 6, 50.0) * pm.rotate(k, [4], 6, 50.0)).sum()
    s2 = (pm.rotate(q, [105], 6, 50.0) * pm.rotate(k, [100], 6, 50.0)).sum()
    assert abs(float(s1 - s2)) < 1e-9


def test_plain_window():
    ok = pm.visible(list(range(10)), 4)
    assert ok[9].tolist() == [False] * 6 + [True] * 4 and ok[2].tolist() == [True] * 3 + [False] * 7
    assert pm.visible(list(range(5)), None)[4].all()


def test_plain_route_keeps_to_the_best_groups():
    w = torch.eye(8, dtype=torch.float64)
    r = {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}
    # groups (0,1) (2,3) (4,5) (6,7): the highest single score sits in group 3, but groups 0 and 1 have the best pairs
    h = torch.tensor([[2.0, 1.9, 1.5, 1.6, -3.0, -3.0, 5.0, -9.0]], dtype=torch.float64)
    chosen, s = pm.route(h, w, r)
    assert chosen.tolist() == [[0, 1, 3]]
    assert torch.allclose(s, torch.sigmoid(h))
    r["groups"] = {"count": 1, "keep": 1}
    assert pm.route(h, w, r)[0].tolist() == [[6, 0, 1]]


def test_plain_model_is_causal_and_windowed(tmp_path):
    folder = mm.write_model(str(tmp_path / "m"), mm.config("Q"), 3)
    cfg, W = pm.load_folder(folder)
    ids = [int(t) for t in torch.randint(0, 131, (60,), generator=torch.Generator().manual_seed(4))]
    a = pm.forward(cfg, W, ids)
    assert torch.allclose(a[:25], pm.forward(cfg, W, ids[:25]), atol=1e-10)
    # both layers see at most 40 positions back, so after two layers a change 80 or more back cannot show
    other = list(ids)
    other[0] = (ids[0] + 1) % 131
    b = pm.forward(cfg, W, other)
    assert (a[0] - b[0]).abs().max() > 1e-3 and torch.allclose(a[-1], b[-1], atol=1e-10)
    streams = []
    pm.forward(cfg, W, ids[:9], streams)
    assert len(streams) == 2 and streams[0].shape == (9, 88)


def test_command_line_writes_and_inspects_a_model(tmp_path, capsys):
    import json
    from inferflux_amd import cli
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(mm.config("Q")))
    out = str(tmp_path / "model")
    assert cli.main(["random-weights", "--config", str(cfg_file), "--out", out, "--seed", "3"]) == 0
    capsys.readouterr()
    assert cli.main(["inspect", "--model", out]) == 0
    report = json.loads(capsys.readouterr().out)
    assert report["missing"] == [] and report["unexpected"] == [] and report["tensors_expected"] == report["tensors_in_file"]
    assert report["config"]["architecture"] == "Mumusun" and report["config"]["layers"][1]["mixer"]["rot"]["dims"] == 4
    cfg, W = pm.load_folder(out)                      # the plain implementation reads what the package wrote
    assert pm.forward(cfg, W, [1, 2, 3]).shape == (3, 131)
