"""The Mumusun design on the GPU: every mechanism's kernel alone against the plain implementation's function, then the
model through the engine's step function, its replay tool and its generation loop, under every way of cutting and
batching, in 32-bit and in bfloat16."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import mumusun_models as mm
import plain_mumusun as pm
import traces
from conftest import ROOT, rel_err

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd import SamplingParams
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepContext, StepEntry
    from inferflux_amd.engine.engine import Engine
    from inferflux_amd.kernels import ops
    from inferflux_amd.kernels.attention import paged_attention
    from inferflux_amd.parts.base import LayerCache

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# Largest difference of a logit from the plain model's, relative to the largest logit.  32-bit: rounding over a few
# hundred operations.  bfloat16: the models' attention is peaked on purpose, which multiplies what the rounding of
# scores and activations to 8 bits of mantissa does (query/key gain 1 / 2 / 4: worst row 1.4 / 4.3 / 5.7 %, median
# 0.5 / 0.9 / 1.1 %); the bfloat16 models take gain 2 and the bound is the worst seen and half as much again.  A key,
# a window's edge or an expert that is wrong moves a row by 30-100 %.
TOL = {"float32": 3e-5, "bfloat16": 6.5e-2}
GAIN = {"float32": 4.0, "bfloat16": 2.0}
DEV = "cuda"


def rnd(seed, *shape, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def ids_of(seed, n, vocab):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """(configuration, precision) -> model folder.  The 32-bit runs take routers with random weights; the bfloat16
    runs take models in which no choice of experts is a close call (``write_model``), because a choice that
    rounding flips changes a row's logits altogether and says nothing about the kernels."""
    out = {}
    for i, n in enumerate(mm.CONFIGS):
        for dtype in DT:
            out[n, dtype] = mm.write_model(str(tmp_path_factory.mktemp(f"mumusun{n}{dtype}")), mm.config(n), 40 + i, gain=GAIN[dtype],
                                           decisive_router=dtype == "bfloat16")
    return out


_PLAIN = {}


def plain(folder, ids, streams=None):
    if folder not in _PLAIN:
        _PLAIN[folder] = pm.load_folder(folder)
    key = (folder, tuple(ids))
    if key not in _PLAIN or streams is not None:
        _PLAIN[key] = pm.forward(*_PLAIN[folder], list(ids), streams)
    return _PLAIN[key]


def run_whole(runner, rid, ids, want=None):
    runner.add_request(rid)
    out = runner.step([StepEntry(rid, ids, list(range(len(ids))) if want is None else want)]).cpu()
    runner.free_request(rid)
    return out


# ---- each mechanism's kernel alone ------------------------------------------------------------
@pytest.mark.parametrize("H", [24, 200, 1000, 5000])
def test_layer_norm_kernels(H):
    x, d, w = rnd(1, 7, H) + 0.5, rnd(2, 7, H, scale=3.0) - 1.0, rnd(3, H)
    xs, ws = x.float().to(DEV), w.float().to(DEV)
    got = ops.layernorm(xs.clone(), None, ws, 1e-5, torch.float32).cpu()
    assert rel_err(got, pm.layer_norm(x.float().double(), w.float().double(), 1e-5)) < 1e-5
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    got = ops.layernorm(xs.clone(), None, ws, 1e-5, torch.bfloat16, rows).cpu()
    assert rel_err(got, pm.layer_norm(x.float().double(), w.float().double(), 1e-5)[[5, 0, 5]]) < 1e-2
    # on a sub-block's output: stream += norm(delta), and the new stream rounded beside it
    for dd in (torch.float32, torch.bfloat16):
        stream, delta = xs.clone(), d.to(dd).to(DEV)
        wd = w.to(dd).to(DEV)
        cast = ops.add_layernorm(stream, delta, wd, 1e-5, torch.bfloat16)
        want = x.float().double() + pm.layer_norm(delta.cpu().double(), wd.cpu().double(), 1e-5)
        assert rel_err(stream.cpu(), want) < 1e-5
        assert torch.equal(cast, stream.to(torch.bfloat16))
    # the delta as partial sums of a product cut into slices
    parts = torch.stack([d.float() * 0.25, d.float() * 0.5, d.float() * 0.25]).to(DEV)
    stream = xs.clone()
    assert ops.add_layernorm(stream, ops.SliceSums(parts, torch.bfloat16), ws, 1e-5, torch.float32) is stream
    assert rel_err(stream.cpu(), x.float().double() + pm.layer_norm(parts.sum(0).cpu().double(), w.float().double(), 1e-5)) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("wide_values", [False, True])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim,rot_dims", [(40, 32, 8, 8), (16, 48, 16, 8), (300, 130, 6, 2), (0, 20, 4, 4)])
def test_latent_finish_norms_rotates_and_writes_the_cache(dtype, q_rank, kv_rank, rot_dim, rot_dims, wide_values):
    T, P, pages, base = 21, 16, 9, 777.0
    dt = DT[dtype]
    y = rnd(4, T, q_rank + kv_rank + rot_dim, scale=2.0).to(dt)
    wq, wkv = (rnd(5, q_rank) + 1).to(dt), (rnd(6, kv_rank) + 1).to(dt)
    positions = torch.tensor([3 + 7 * t for t in range(T)], dtype=torch.int32)
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(7))[:T].to(torch.int32)
    inv = torch.tensor([base ** (-2.0 * i / rot_dims) for i in range(rot_dims // 2)], dtype=torch.float32, device=DEV)
    cos, sin = ops.rope_table(positions.to(DEV), inv)
    k = torch.zeros((pages, 1, P, kv_rank + rot_dim), dtype=dt, device=DEV)
    v_rows = kv_rank + rot_dim if wide_values else kv_rank       # (values as wide as keys hold the key part as well)
    v = torch.zeros((pages, 1, v_rows, P), dtype=dt, device=DEV)
    cq = ops.latent_finish(y.to(DEV), wq.to(DEV) if q_rank else None, wkv.to(DEV), 1e-5, cos, sin, rot_dims, slots.to(DEV), q_rank,
                           kv_rank, rot_dim, k, v, P, dt)
    tol = 1e-5 if dtype == "float32" else 1e-2
    yd = y.double()
    if q_rank:
        assert rel_err(cq.cpu(), pm.rms_norm(yd[:, :q_rank], wq.double(), 1e-5)) < tol
    else:
        assert cq is None
    c = pm.rms_norm(yd[:, q_rank:q_rank + kv_rank], wkv.double(), 1e-5)
    kr = pm.rotate(yd[:, None, q_rank + kv_rank:], positions.tolist(), rot_dims, base)[:, 0]
    k_rows = k.cpu().view(pages * P, -1)[slots.long()]
    assert rel_err(k_rows[:, :kv_rank], c) < tol and rel_err(k_rows[:, kv_rank:], kr) < tol
    v_cols = v.cpu()[:, 0].permute(0, 2, 1).reshape(pages * P, v_rows)[slots.long()]
    assert torch.equal(v_cols, k_rows[:, :v_rows])                       # the same numbers in both layouts
    untouched = torch.ones(pages * P, dtype=torch.bool)
    untouched[slots.long()] = False
    assert not k.cpu().view(pages * P, -1)[untouched].any()
    # partial sums of a sliced product give the same as their sum
    if dtype == "float32":
        parts = torch.stack([y * 0.5, y * 0.25, y * 0.25]).to(DEV)
        k2, v2 = torch.zeros_like(k), torch.zeros_like(v)
        cq2 = ops.latent_finish(ops.SliceSums(parts, dt), wq.to(DEV) if q_rank else None, wkv.to(DEV), 1e-5, cos, sin, rot_dims,
                                slots.to(DEV), q_rank, kv_rank, rot_dim, k2, v2, P, dt)
        assert rel_err(k2.cpu(), k.cpu().double()) < 1e-6 and (not q_rank or rel_err(cq2.cpu(), cq.cpu().double()) < 1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,K,N,tail,rot", [(1, 3, 16, 32, 8, 8), (37, 2, 8, 48, 16, 8), (130, 5, 70, 9, 0, 0), (16, 1, 20, 44, 12, 12),
                                              (65, 4, 128, 200, 6, 2)])
def test_headwise_product_with_rotated_tail(dtype, T, H, K, N, tail, rot):
    dt = DT[dtype]
    x, w = rnd(8, T, H * (K + tail) + 3).to(dt), rnd(9, H, N, K, scale=K ** -0.5).to(dt)
    positions = torch.arange(T, dtype=torch.int32) * 3 + 1
    cos = sin = None
    if rot:
        inv = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV)
        cos, sin = ops.rope_table(positions.to(DEV), inv)
    got = ops.headwise(x.to(DEV), w.to(DEV), H, K + tail, tail, cos, sin, rot).cpu()
    xh = x.double()[:, :H * (K + tail)].view(T, H, K + tail)
    want = torch.einsum("thk,hnk->thn", xh[..., :K], w.double())
    if tail:
        t = xh[..., K:]
        want = torch.cat([want, pm.rotate(t, positions.tolist(), rot, 50.0) if rot else t], dim=-1)
    assert got.shape == (T, H, N + tail)
    assert rel_err(got, want) < (1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("E,top,count,keep", [(8, 3, 4, 2), (10, 3, 2, 1), (6, 1, 1, 1), (9, 2, 3, 1), (4, 4, 2, 2), (16, 2, 16, 5), (64, 6, 8, 3)])
def test_router_scores_groups_and_choice(E, top, count, keep):
    T, K = 50, 72
    h, w = rnd(10, T, K), rnd(11, E, K, scale=0.4)
    for dtype in ("float32", "bfloat16"):
        hd, wd = h.to(DT[dtype]), w.to(DT[dtype])
        ids, weights = ops.moe_route(hd.to(DEV), wd.to(DEV), top, count, keep, 2)
        chosen, s = pm.route(hd.double(), wd.double(), {"experts": E, "top": top, "groups": {"count": count, "keep": keep}})
        assert ids.cpu().tolist() == chosen.tolist()                               # (in descending order of score)
        assert rel_err(weights.cpu(), torch.gather(s, 1, chosen)) < 1e-5           # the scores as they are
    # other routers a design may ask of the same kernel: a softmax, weights that sum to one, a scale
    ids, weights = ops.moe_route(h.float().to(DEV), w.float().to(DEV), top, 1, 1, 2, softmax=True, renormalize=True, scale=2.5)
    p = torch.softmax(h.float().double() @ w.float().double().T, -1)
    best = p.topk(top, -1)
    assert ids.cpu().tolist() == best.indices.tolist()
    assert rel_err(weights.cpu(), best.values / best.values.sum(-1, keepdim=True) * 2.5) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,ff,E,top", [(1, 64, 48, 8, 3), (33, 88, 56, 9, 2), (200, 128, 64, 8, 2), (5, 40, 130, 3, 3)])
def test_experts_weighted_sum(dtype, T, K, ff, E, top):
    dt = DT[dtype]
    h = rnd(12, T, K).to(dt)
    gate, up, down = rnd(13, E, ff, K, scale=K ** -0.5).to(dt), rnd(14, E, ff, K, scale=K ** -0.5).to(dt), rnd(15, E, K, ff, scale=ff ** -0.5).to(dt)
    g = torch.Generator().manual_seed(16)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    weights = torch.rand(T, top, generator=g)
    got = ops.moe_experts(h.to(DEV), gate.to(DEV), up.to(DEV), down.to(DEV), ids.to(DEV), weights.to(DEV)).cpu()
    want = torch.zeros(T, K, dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            want[t] += weights[t, j].double() * pm.expert(h[t].double(), gate[e].double(), up[e].double(), down[e].double())
    assert rel_err(got, want) < (1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("T,K,ff,E,top,N", [(200, 128, 64, 8, 2, 128), (33, 88, 48, 9, 2, 88), (700, 64, 96, 12, 4, 72), (64, 192, 16, 3, 1, 50),
                                              (16, 40, 32, 40, 4, 40), (130, 96, 160, 5, 5, 200)])
def test_experts_on_the_matrix_cores(T, K, ff, E, top, N):
    """Many rows: items ordered by expert, tiles of one expert's items against its weights.  Experts nobody chose,
    experts with several tiles, tiles that are not full; the choices come back as partial sums in choice order."""
    h = rnd(17, T, K).bfloat16()
    gate, up = rnd(18, E, ff, K, scale=K ** -0.5).bfloat16(), rnd(19, E, ff, K, scale=K ** -0.5).bfloat16()
    down = rnd(20, E, N, ff, scale=ff ** -0.5).bfloat16()
    g = torch.Generator().manual_seed(21)
    popular = torch.randperm(E, generator=g)[:max(top, E // 2)]                  # the other experts get nothing
    ids = torch.stack([popular[torch.randperm(popular.numel(), generator=g)[:top]] for _ in range(T)]).to(torch.int32)
    weights = torch.rand(T, top, generator=g)
    pairs = ops.pair_gate_up(gate.to(DEV), up.to(DEV))
    got = ops.moe_experts_grouped(h.to(DEV), pairs, down.to(DEV), ids.to(DEV), weights.to(DEV))
    assert tuple(got.parts.shape) == (top, T, N) and got.parts.dtype == torch.float32
    want = torch.zeros(top, T, N, dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            want[j, t] = weights[t, j].double() * pm.expert(h[t].double(), gate[e].double(), up[e].double(), down[e].double())
    assert rel_err(got.parts.cpu(), want) < 2e-2
    rows = ops.moe_experts(h.to(DEV), pairs, None, down.to(DEV), ids.to(DEV), weights.to(DEV)).cpu()      # row by row from the same tensor
    assert rel_err(rows, want.sum(0)) < 2e-2
    stream = torch.zeros(T, N, device=DEV)                           # the kernel that takes the partial sums adds them up
    ops.add_layernorm(stream, got, torch.ones(N, device=DEV), 1e-5, None)
    assert rel_err(stream.cpu(), pm.layer_norm(want.sum(0), torch.ones(N, dtype=torch.float64), 1e-5)) < 2e-2


@pytest.mark.parametrize("T,H,K,N,tail,rot", [(32, 3, 32, 96, 32, 32), (100, 6, 16, 40, 8, 4), (257, 2, 96, 24, 0, 0), (64, 1, 128, 130, 16, 16)])
def test_headwise_product_on_the_matrix_cores(T, H, K, N, tail, rot):
    x, w = rnd(22, T, H * (K + tail)).bfloat16(), rnd(23, H, N, K, scale=K ** -0.5).bfloat16()
    positions = torch.arange(T, dtype=torch.int32) * 2 + 5
    cos = sin = None
    if rot:
        inv = torch.tensor([30.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV)
        cos, sin = ops.rope_table(positions.to(DEV), inv)
    assert T >= ops.HEADWISE_GROUPED_MIN_ROWS
    got = ops.headwise(x.to(DEV), w.to(DEV), H, K + tail, tail, cos, sin, rot).cpu()
    few = torch.cat([ops.headwise(x[i:i + 8].to(DEV), w.to(DEV), H, K + tail, tail, None if cos is None else cos[i:i + 8].contiguous(),
                                  None if sin is None else sin[i:i + 8].contiguous(), rot).cpu() for i in range(0, T, 8)])
    xh = x.double().view(T, H, K + tail)
    want = torch.einsum("thk,hnk->thn", xh[..., :K], w.double())
    if tail:
        want = torch.cat([want, pm.rotate(xh[..., K:], positions.tolist(), rot, 30.0) if rot else xh[..., K:]], dim=-1)
    assert rel_err(got, want) < 1e-2 and rel_err(few, want) < 1e-2
    assert torch.equal(got[..., N:], few[..., N:])


def _paged_case(dtype, n, window, d, dv, nH, P=16, seed=20):
    """One request of n positions whose rows are all queried at once, its pages scattered over the pool; every query
    is aimed at two keys, the one on the window's inner edge and, twice as hard, the one just outside it, so that a
    window one position too wide or too narrow changes which value a head returns."""
    dt = DT[dtype]
    pages = -(-n // P) + 3
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed))[:-(-n // P)]
    k, v = rnd(seed + 1, n, d, scale=0.05), rnd(seed + 2, n, dv)
    q = rnd(seed + 3, n, nH, d, scale=0.05)
    marks = d - 1
    for j in range(n):
        k[j, j % marks] += 1.0
    for p in range(n):
        inner = p - (window - 1) if window else 0
        if inner >= 0:
            q[p, :, inner % marks] += 12.0
        if inner - 1 >= 0:
            q[p, :, (inner - 1) % marks] += 24.0
    k, v, q = k.to(dt), v.to(dt), q.to(dt)
    kc = torch.zeros((pages, 1, P, d), dtype=dt)
    vc = torch.zeros((pages, 1, dv, P), dtype=dt)
    for j in range(n):
        kc[order[j // P], 0, j % P] = k[j]
        vc[order[j // P], 0, :, j % P] = v[j]
    pos = torch.arange(n)
    s = torch.einsum("ihd,jd->hij", q.double(), k.double())
    s = s.masked_fill(~pm.visible(pos.tolist(), window), -math.inf)
    want = torch.einsum("hij,jd->ihd", torch.softmax(s, -1), v.double()).reshape(n, nH * dv)
    table = torch.full((1, pages), -1, dtype=torch.int32)
    table[0, :order.numel()] = order.to(torch.int32)
    return q, kc, vc, table, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,window,d,dv,nH", [(70, 20, 40, 32, 3), (150, 33, 64, 48, 2), (40, 7, 56, 44, 1), (200, 64, 48, 32, 4),
                                              (130, None, 44, 40, 4), (100, 16, 64, 48, 16), (530, 90, 120, 88, 5)])
def test_attention_over_a_latent_cache_at_the_windows_edges(dtype, n, window, d, dv, nH):
    """Keys as wide as latent + rotated part, values as wide as the latent, one shared kv head."""
    q, kc, vc, table, want = _paged_case(dtype, n, window, d, dv, nH)
    row_req, pos = torch.zeros(n, dtype=torch.int32, device=DEV), torch.arange(n, dtype=torch.int32, device=DEV)
    got = ops.attention_plain(q.to(DEV), kc.to(DEV), vc.to(DEV), row_req, pos, table.to(DEV), window, 1.0).cpu()
    assert rel_err(got, want) < (2e-5 if dtype == "float32" else 2e-2)
    if window and window < min(n, d - 1):      # the aim works (where the marks do not repeat within a window): the inner edge's value, not the outer's
        p = n - 1
        v_in = vc.double()[table[0, (p - window + 1) // 16], 0, :, (p - window + 1) % 16]
        assert (want[p, :dv] - v_in).abs().max() < 0.05 * v_in.abs().max()


@pytest.mark.parametrize("n,window,d,dv,nH", [(70, 20, 40, 32, 3), (150, 33, 64, 48, 2), (200, 64, 48, 32, 4), (130, None, 56, 48, 20),
                                              (100, 16, 64, 48, 16), (300, 80, 576, 512, 16), (530, 100, 136, 96, 33)])
def test_wide_attention_on_the_matrix_cores(n, window, d, dv, nH):
    """The same cases through the kernel for one shared kv head of any width, with the keys cut into splits of several
    lengths (a split's edge inside a page, inside the window, past the end)."""
    q, kc, vc, table, want = _paged_case("bfloat16", n, window, d, dv, nH)
    row_req, pos = torch.zeros(n, dtype=torch.int32, device=DEV), torch.arange(n, dtype=torch.int32, device=DEV)
    bound = table.shape[1] * 16
    for chunk in (32, 96, 64 * -(-bound // 64)):
        got = ops.attention_wide(q.to(DEV), kc.to(DEV), vc.to(DEV), row_req, pos, table.to(DEV), window, 1.0, chunk, -(-bound // chunk)).cpu()
        assert rel_err(got, want) < 2e-2, chunk
    chunk, splits = ops.wide_launch_shape(n, nH, bound)
    assert chunk % 32 == 0 and chunk * splits >= bound


# ---- the model through the step function ----------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(mm.CONFIGS))
def test_whole_prompts(name, dtype, folders):
    folder = folders[name, dtype]
    runner = load_runner(folder, DT[dtype], num_pages=48, max_requests=4)
    vocab = mm.CONFIGS[name]["vocab"]
    for n in (1, 2, 17, 130, 600):
        ids = ids_of(n, n, vocab)
        got = run_whole(runner, "a", ids)
        assert rel_err(got, plain(folder, ids)) < TOL[dtype], (name, n)
    runner.manager.check()
    assert runner.manager.free_pages() == [48] * len(runner.manager.groups)


def test_stream_after_every_layer(folders):
    folder = folders["P", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    ids = ids_of(3, 50, 300)
    streams = []
    plain(folder, ids, streams)
    runner.add_request("p")
    runner.manager.reserve("p", len(ids))
    ctx = StepContext([StepEntry("p", ids, [0])], runner.manager, torch.float32, runner.device)
    model = runner.model
    x, pending = model.embedding.forward(ctx), None
    for i, e in enumerate(model.plan.schedule):
        x, pending = model.blocks[e.layer].forward(x, pending, ctx, runner.storage.binding(i))
        assert rel_err(x.cpu(), streams[i]) < 1e-5, i


def test_first_tokens(folders):
    """Position 0 sees itself alone: its logits are a function of the token."""
    folder = folders["Q", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    for tok in (0, 77, 130):
        a, b = run_whole(runner, "x", [tok]), run_whole(runner, "y", [tok, 5, 9, 2])
        assert rel_err(a, plain(folder, [tok])) < TOL["float32"] and torch.equal(a[0], b[0])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_prefill_against_decoding_and_portions(name, dtype, folders):
    folder, vocab = folders[name, dtype], mm.CONFIGS[name]["vocab"]
    runner = load_runner(folder, DT[dtype], num_pages=24, max_requests=4)
    ids = ids_of(31, 170, vocab)
    want = plain(folder, ids)
    whole = run_whole(runner, "w", ids)
    runner.add_request("d")                                      # token by token from the first
    single = torch.cat([runner.step([StepEntry("d", [t], [0])]).cpu() for t in ids])
    runner.free_request("d")
    runner.add_request("c")                                      # portions of changing size, down to two tokens and one
    rows, p = [], 0
    for m in [2, 3, 16, 2, 1, 31, 2, 64, 17, 2, 30]:
        rows.append(runner.step([StepEntry("c", ids[p:p + m], list(range(m)))]).cpu())
        p += m
    runner.free_request("c")
    assert p == len(ids)
    for got in (whole, single, torch.cat(rows)):
        assert rel_err(got, want) < TOL[dtype]
    if dtype == "float32":       # in 32-bit a row's arithmetic does not depend on the cutting at all
        assert torch.equal(single, whole) and torch.equal(torch.cat(rows), whole)
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch_against_each_alone(dtype, folders):
    folder = folders["P", dtype]
    runner = load_runner(folder, DT[dtype], num_pages=40, max_requests=4)
    seqs = {"a": ids_of(41, 90, 300), "b": ids_of(42, 23, 300), "c": ids_of(43, 140, 300), "d": ids_of(44, 2, 300)}
    for r in seqs:
        runner.add_request(r)
    at = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    plan = [{"a": 30, "b": 2, "c": 64, "d": 1}, {"a": 1, "c": 40, "d": 1}, {"a": 17, "b": 20, "c": 1}, {"a": 1, "b": 1, "c": 1},
            {"a": 41, "c": 34}]
    for step in plan:
        entries = [StepEntry(r, seqs[r][at[r]:at[r] + m], list(range(m))) for r, m in step.items()]
        out = runner.step(entries).cpu()
        o = 0
        for r, m in step.items():
            got[r].append(out[o:o + m]); o += m; at[r] += m
    for r, ids in seqs.items():
        assert at[r] == len(ids)
        assert rel_err(torch.cat(got[r]), plain(folder, ids)) < TOL[dtype], r
        if dtype == "float32":
            runner.free_request(r)
            assert torch.equal(torch.cat(got[r]), run_whole(runner, r + "'", ids)), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_gives_pages_back_as_the_windows_pass(dtype, folders):
    folder = folders["P", dtype]
    runner = load_runner(folder, DT[dtype], num_pages=30, max_requests=2)
    ids = ids_of(51, 420, 300)
    want = plain(folder, ids)
    runner.add_request("d")
    got = [runner.step([StepEntry("d", ids[:9], [8])]).cpu()[0]]
    for p in range(9, len(ids)):
        got.append(runner.step([StepEntry("d", [ids[p]], [0])]).cpu()[0])
    assert rel_err(torch.stack(got), want[8:]) < TOL[dtype]
    runner.manager.check()
    windows = [g.window for g in runner.manager.groups]
    assert windows == [None, 20, 33]
    held = [sum(1 for p in runner.manager.block_table("d", g) if p >= 0) for g in range(3)]
    assert held[0] == -(-420 // 16) and held[1] <= 20 // 16 + 2 and held[2] <= 33 // 16 + 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_replay_of_traces_with_pages_and_slots_used_again(name, dtype, folders, tmp_path):
    """Through bin/trace_run as a user would: whole, prefill then decode, portions, and mixed steps of up to four live
    requests, one process, a pool so small that pages and slots are used again."""
    folder, vocab = folders[name, dtype], mm.CONFIGS[name]["vocab"]
    seqs = {f"r{i}": ids_of(60 + i, n, vocab) for i, n in enumerate([45, 150, 1, 96, 33, 260, 64])}
    all_steps, expected, offset = [], {}, 0
    for build in (traces.whole, traces.prefill_then_decode, traces.portions, lambda s: traces.mixed(s, seed=7)):
        steps, exp = build(seqs)
        for s in steps:
            s["step"] += offset
        expected.update({k + offset: v for k, v in exp.items()})
        all_steps += steps
        offset += len(steps)
    out = str(tmp_path / "out")
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
                             "--max-tokens", str(traces.peak_tokens(all_steps))], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in all_steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {s['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    assert sorted(int(f[:-4]) for f in os.listdir(out)) == sorted(expected)
    for step, rows in expected.items():
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(len(rows), vocab))
        want = torch.stack([plain(folder, seqs[rid])[p] for rid, p in rows])
        assert rel_err(got, want) < TOL[dtype], (step, rows[:3])


def _drawn_config(seed):
    """A configuration drawn from sizes of every kind: latents that the matrix-core attention kernels take whole (a multiple of
    16 up to 128), that the kernel for one shared kv head takes, and that only the plain kernel takes; more heads than a matrix
    tile has columns; layers with and without window and feed-forward; routers with and without groups."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 72, 96, 160])
    layers = []
    for _ in range(rng.choice([1, 2, 3])):
        kv_rank, rot_dim = rng.choice([(16, 16), (48, 16), (64, 16), (96, 32), (96, 16), (32, 8), (80, 24), (20, 6), (136, 8)])
        dims = rng.choice([rot_dim, max(2, rot_dim // 2 // 2 * 2)])
        mixer = mm._mixer(rng.choice([1, 2, 5, 8, 20]), rng.choice([8, 12, 16, 40]), rot_dim, rng.choice([8, 10, 24, 48]), rng.choice([16, 24, 52]),
                          kv_rank, rng.choice([0.1, 0.17, 0.3]), rng.choice([100.0, 10000.0, 1e6]), dims, rng.choice([None, 5, 16, 17, 64, 100]))
        count = rng.choice([1, 2, 3, 4])
        per = rng.choice([1, 2, 3])
        keep = rng.randint(1, count)
        mlp = rng.choice([None, mm._moe(count * per, rng.randint(1, keep * per), rng.choice([16, 24, 48, 80]), count, keep)])
        layers.append(mm._layer(mixer, mlp))
    return {"architecture": "Mumusun", "vocab": rng.choice([61, 128, 500]), "width": width, "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
            "layers": layers}


@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations(seed, tmp_path):
    """Whole prompts, portions and decoding of drawn configurations against the plain implementation, both precisions."""
    cfg = _drawn_config(seed)
    for dtype in ("float32", "bfloat16"):
        folder = mm.write_model(str(tmp_path / dtype), cfg, 80 + seed, gain=GAIN[dtype], decisive_router=dtype == "bfloat16")
        runner = load_runner(folder, DT[dtype], num_pages=24, max_requests=3)
        ids = ids_of(seed, 150, cfg["vocab"])
        want = plain(folder, ids)
        assert rel_err(run_whole(runner, "w", ids), want) < TOL[dtype], (seed, dtype, cfg)
        runner.add_request("c")
        runner.add_request("other")
        rows, p = [], 0
        for m in [33, 2, 64, 1, 1, 17, 1, 1, 1, 29]:
            out = runner.step([StepEntry("other", ids_of(p, 3, cfg["vocab"]), []), StepEntry("c", ids[p:p + m], list(range(m)))]).cpu()
            rows.append(out)
            p += m
        assert p == len(ids) and rel_err(torch.cat(rows), want) < TOL[dtype], (seed, dtype, cfg)
        runner.manager.check()


# ---- generation through the engine's own entry point and scheduler ------------------------------
@pytest.mark.parametrize("name", ["P", "R"])
def test_greedy_generation_through_the_engine(name, folders):
    folder, vocab = folders[name, "float32"], mm.CONFIGS[name]["vocab"]
    cfg, W = pm.load_folder(folder)
    prompts = [ids_of(70 + i, n, vocab) for i, n in enumerate([5, 40, 1, 77, 19, 130])]
    want = [pm.greedy_generate(cfg, W, p, 12) for p in prompts]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32, prefill_tokens_alone=48)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    assert [o.token_ids for o in outs] == want
    assert engine.runner.graph_replays > 0                       # decode steps ran as replayed graphs
    folder = folders[name, "bfloat16"]
    cfg, W = pm.load_folder(folder)
    engine = Engine.load(folder, dtype="bfloat16", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):        # bfloat16 may pick another token where two logits nearly tie
        full = pm.forward(cfg, W, p + o.token_ids)
        for i, tok in enumerate(o.token_ids):
            row = full[len(p) - 1 + i]
            assert row[tok] >= row.max() - 0.06 * row.abs().max(), (name, i)


def test_completion_from_the_command_line(folders, capsys):
    from inferflux_amd import cli
    folder = folders["Q", "float32"]
    cfg, W = pm.load_folder(folder)
    prompt = ids_of(90, 21, 131)
    assert cli.main(["completion", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "7", "--temperature", "0",
                     "--ignore-eos", "--dtype", "float32", "--kv-pages", "32", "--max-parallel-sequences", "2"]) == 0
    said = capsys.readouterr().out
    want = pm.greedy_generate(cfg, W, prompt, 7)
    assert str(want)[1:-1].replace(" ", "") in said.replace(" ", ""), (want, said)
