"""The Podurax design on the GPU: every mechanism's kernel alone against the plain implementation's function, then the
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

import plain_podurax as pp
import podurax_models as pm
import traces
from conftest import ROOT, rel_err

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd import SamplingParams
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepContext, StepEntry
    from inferflux_amd.engine.engine import Engine
    from inferflux_amd.kernels import ops
    from inferflux_amd.parts.position import RotaryPosition

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# Largest difference of a logit from the plain model's, relative to the largest logit.  32-bit: rounding over a few hundred
# operations.  bfloat16: the worst seen over all of these tests and half as much again (0.9 % where attention runs on the
# plain kernel, 3 % on the matrix cores, whose second product takes the softmax's weights rounded to bfloat16); a key, a
# window's edge, a state or a sink that is wrong moves a row by 20-100 % (the kernels' own tests aim queries at the edges
# so that it does).
TOL = {"float32": 5e-6, "bfloat16": 4.5e-2}
GAIN = {"float32": 2.0, "bfloat16": 1.0}
DEV = "cuda"


def rnd(seed, *shape, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def ids_of(seed, n, vocab):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def T64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for i, n in enumerate(pm.CONFIGS):
        for dtype in DT:
            out[n, dtype] = pm.write_model(str(tmp_path_factory.mktemp(f"podurax{n}{dtype}")), pm.config(n), 40 + i, gain=GAIN[dtype])
    return out


_PLAIN = {}


def plain(folder, ids, layers=False):
    if folder not in _PLAIN:
        _PLAIN[folder] = pm.load_plain(folder)
    key = (folder, tuple(ids), layers)
    if key not in _PLAIN:
        out = pp.forward(*_PLAIN[folder], list(ids), return_layers=layers)
        _PLAIN[key] = (T64(out[0]), T64(out[1])) if layers else T64(out)
    return _PLAIN[key]


def run_whole(runner, rid, ids, want=None):
    runner.add_request(rid)
    out = runner.step([StepEntry(rid, ids, list(range(len(ids))) if want is None else want)]).cpu()
    runner.free_request(rid)
    return out


# ---- each mechanism's kernel alone ------------------------------------------------------------
@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (4.0, 64, 8.0, 1.0)), (24, 5e5, (6.0, 2048, 24.0, 1.0)), (6, 300.0, None),
                                               (32, 5e5, (2.5, 4096, 16.0, 0.25)), (4, 50.0, (16.0, 32, 2.0, 1.5))])
def test_rotation_table_with_stretched_frequencies(dims, base, scaling):
    sc = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    part = RotaryPosition(head_dim=dims + 4, theta=base, rotary_dim=dims, scaling=sc)
    f, mag = pp.yarn_frequencies(dims, base, sc)
    assert rel_err(part.frequencies(), T64(f)) < 1e-12 and abs(part.magnitude - mag) < 1e-12
    if sc:          # the slow pairs are stretched, the fast ones are not, and what is turned grows a little
        plain_f = base ** (-2.0 * np.arange(dims // 2) / dims)
        assert f[-1] <= plain_f[-1] and f[0] <= plain_f[0] and mag > 1.0 or sc["factor"] <= 1.0
    positions = torch.tensor([0, 1, 2, 77, 1000, 40000], dtype=torch.int32, device=DEV)
    cos, sin = ops.rope_table(positions, part.inv_freq(DEV), part.magnitude)
    a = positions.cpu().double()[:, None] * T64(f)[None, :]
    assert (cos.cpu().double() - torch.cos(a) * mag).abs().max() < 5e-3 * max(1.0, 40000 * float(f[0]) * 1e-4)
    small = slice(0, 3)     # (float32 angles lose digits at large positions: the first positions pin the table itself)
    assert (cos.cpu().double()[small] - (torch.cos(a) * mag)[small]).abs().max() < 2e-6
    assert (sin.cpu().double()[small] - (torch.sin(a) * mag)[small]).abs().max() < 2e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [37, 300])       # (many rows of sizes in sixteens take the kernel that works in 16-byte pieces)
@pytest.mark.parametrize("nH,nKV,d,dv,dims,style", [(4, 2, 16, 24, 8, "mix"), (3, 3, 12, 12, 12, "source"), (2, 1, 32, 8, 4, None),
                                                    (8, 2, 64, 64, 16, "mix"), (3, 1, 10, 14, 6, "mix"), (5, 5, 130, 70, 100, "source"),
                                                    (4, 2, 32, 32, 16, "source"), (8, 8, 128, 128, 64, "mix"), (8, 2, 64, 48, 32, "mix"),
                                                    (16, 2, 128, 128, 128, None), (8, 1, 16, 16, 16, "mix")])
def test_row_kernel_biases_rotation_unit_norms_gate_value_mixing_and_cache(dtype, T, nH, nKV, d, dv, dims, style):
    P, pages, eps, lam = 16, -(-T // 16) + 4, 1e-5, 0.3125
    dt = DT[dtype]
    width = (nH + nKV) * d + nKV * dv + nH
    qkv, bias = rnd(1, T, width, scale=1.5).to(dt), rnd(2, width, scale=0.5).to(dt)
    bias[-nH:] = 0
    v_first = rnd(3, T, nKV * dv).to(dt)
    positions = torch.tensor([5 + 3 * t for t in range(T)], dtype=torch.int32)
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(4))[:T].to(torch.int32)
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    part = RotaryPosition(head_dim=d, theta=1000.0, rotary_dim=dims, scaling=sc)
    cos, sin = ops.rope_table(positions.to(DEV), part.inv_freq(DEV), part.magnitude)
    k = torch.zeros((pages, nKV, P, d), dtype=dt, device=DEV)
    v = torch.zeros((pages, nKV, dv, P), dtype=dt, device=DEV)
    gate = torch.empty((T, nH), dtype=torch.float32, device=DEV)
    v_out = torch.empty((T, nKV * dv), dtype=dt, device=DEV) if style == "source" else None
    q = ops.rope_append(qkv.to(DEV), bias.to(DEV), slots.to(DEV), cos, sin, ops.ROPE_SPLIT_HALF, dims, nH, nKV, d, k, v, P, dv, eps, gate,
                        v_first.to(DEV) if style == "mix" else None, lam, v_out)
    x = (qkv.double() + bias.double()).numpy()
    pos = positions.numpy()
    # (32-bit: the engine forms angles in float, position times frequency, which at position p is off by up to p * 6e-8)
    tol = 1e-5 + 1e-7 * int(positions.max()) if dtype == "float32" else 1e-2
    want_q = pp.rms(pp.rotate(x[:, :nH * d].reshape(T, nH, d), pos, dims, 1000.0, sc), eps)
    assert rel_err(q.cpu(), T64(want_q)) < tol
    want_k = pp.rms(pp.rotate(x[:, nH * d:(nH + nKV) * d].reshape(T, nKV, d), pos, dims, 1000.0, sc), eps)
    got_k = k.cpu().permute(0, 2, 1, 3).reshape(pages * P, nKV, d)[slots.long()]
    assert rel_err(got_k, T64(want_k)) < tol
    want_v = x[:, (nH + nKV) * d:(nH + nKV) * d + nKV * dv]
    if style == "source":
        assert rel_err(v_out.cpu(), T64(want_v)) < tol
    if style == "mix":
        want_v = (1.0 - lam) * want_v + lam * v_first.double().numpy()
    got_v = v.cpu().permute(0, 3, 1, 2).reshape(pages * P, nKV * dv)[slots.long()]
    assert rel_err(got_v, T64(want_v)) < tol
    assert rel_err(gate.cpu(), T64(pp.sigmoid(x[:, -nH:]))) < 1e-5
    untouched = torch.ones(pages * P, dtype=torch.bool)
    untouched[slots.long()] = False
    assert not k.cpu().permute(0, 2, 1, 3).reshape(pages * P, -1)[untouched].any()
    if dtype == "float32":       # partial sums of a sliced product give the same as their sum
        parts = torch.stack([qkv * 0.5, qkv * 0.25, qkv * 0.25]).to(DEV)
        k2, v2, g2 = torch.zeros_like(k), torch.zeros_like(v), torch.empty_like(gate)
        q2 = ops.rope_append(ops.SliceSums(parts, dt), bias.to(DEV), slots.to(DEV), cos, sin, ops.ROPE_SPLIT_HALF, dims, nH, nKV, d, k2, v2, P,
                             dv, eps, g2, v_first.to(DEV) if style == "mix" else None, lam, None)
        assert rel_err(q2.cpu(), q.cpu()) < 1e-6 and rel_err(k2.cpu(), k.cpu()) < 1e-6 and rel_err(v2.cpu(), v.cpu()) < 1e-6


def _paged_case(dtype, n, window, keep, d, dv, nH, nKV, P=16, seed=20):
    """One request of n positions whose rows are all queried at once, its pages scattered over the pool.  Every key carries
    a mark of its own and every query is aimed, hard, at four keys: the one on the window's inner edge and the one just
    outside it, the last kept first token and the one after it, so that a window or a kept range one position off
    changes which values a head returns.  Unit-length directions and a scale keep the scores within what a softmax with
    a sink makes interesting."""
    dt = DT[dtype]
    pages = -(-n // P) + 3
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed))[:-(-n // P)]
    k, v = rnd(seed + 1, n, nKV, d, scale=0.05), rnd(seed + 2, n, nKV, dv)
    q = rnd(seed + 3, n, nH, d, scale=0.05)
    marks = d - 1
    for j in range(n):
        k[j, :, j % marks] += 1.0
    for p in range(n):
        inner = p - (window - 1) if window else 0
        for j, w in ((inner, 3.0), (inner - 1, 5.0), (keep - 1, 4.0), (keep, 6.0)):
            if 0 <= j <= p + 2:
                q[p, :, j % marks] += w
    k, v, q = k.to(dt), v.to(dt), q.to(dt)
    kc = torch.zeros((pages, nKV, P, d), dtype=dt)
    vc = torch.zeros((pages, nKV, dv, P), dtype=dt)
    for j in range(n):
        kc[order[j // P], :, j % P] = k[j]
        vc[order[j // P], :, :, j % P] = v[j]
    table = torch.full((1, pages), -1, dtype=torch.int32)
    table[0, :order.numel()] = order.to(torch.int32)
    return q, k, v, kc, vc, table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,window,keep,d,dv,nH,nKV", [(70, 20, 3, 16, 24, 4, 2), (150, 33, 5, 64, 48, 2, 1), (40, 7, 0, 56, 44, 1, 1),
                                                       (200, 64, 1, 48, 32, 4, 4), (130, None, 9, 44, 40, 4, 2), (100, 16, 16, 64, 64, 16, 2),
                                                       (300, 9, 40, 32, 32, 3, 1), (530, 90, 17, 120, 88, 6, 3), (260, 80, 7, 64, 64, 8, 4)])
def test_attention_window_kept_first_tokens_sink_and_gate(dtype, n, window, keep, d, dv, nH, nKV):
    q, k, v, kc, vc, table = _paged_case(dtype, n, window, keep, d, dv, nH, nKV)
    gate = torch.rand(n, nH, generator=torch.Generator().manual_seed(5))
    row_req, pos = torch.zeros(n, dtype=torch.int32, device=DEV), torch.arange(n, dtype=torch.int32, device=DEV)
    tol = 2e-5 if dtype == "float32" else 2e-2
    for sink, use_gate in ((0.0, True), (None, False), (1.5, False)):
        got = ops.attention_plain(q.to(DEV), kc.to(DEV), vc.to(DEV), row_req, pos, table.to(DEV), window, 2.0, keep, sink,
                                  gate.to(DEV) if use_gate else None).cpu()
        kk = k.double().numpy()
        if sink not in (None, 0.0):       # a sink of another score is a sink of score 0 with every score lowered by it
            want = pp.sink_softmax_attention(q.double().numpy(), kk, v.double().numpy(), 2.0, window, keep, sink=False)
            s_shift = True
        else:
            want = pp.sink_softmax_attention(q.double().numpy(), kk, v.double().numpy(), 2.0, window, keep, sink=sink is not None)
            s_shift = False
        if s_shift:
            # exp(s) / (exp(c) + sum exp(s)): from the plain softmax o and its denominator Z, o * Z / (Z + exp(c))
            H, G = nH, nKV
            for h in range(H):
                s = (q.double().numpy()[:, h] @ kk[:, h // (H // G)].T) * 2.0
                mask = np.array([[pp.visible(i, j, window, keep) for j in range(n)] for i in range(n)])
                Z = np.where(mask, np.exp(s), 0.0).sum(1)
                want[:, h] *= (Z / (Z + math.exp(sink)))[:, None]
        if use_gate:
            want = want * gate.double().numpy()[:, :, None]
        assert rel_err(got, T64(want).reshape(n, nH * dv)) < tol, (sink, use_gate)


@pytest.mark.parametrize("n,window,keep,d,nH,nKV", [(70, 20, 3, 16, 4, 2), (150, 33, 5, 64, 2, 1), (200, 64, 1, 48, 4, 4), (100, 16, 16, 64, 16, 2),
                                                    (300, 9, 40, 32, 3, 1), (530, 90, 17, 128, 6, 3), (260, 80, 7, 64, 8, 4), (400, 70, 70, 32, 20, 1),
                                                    (330, 100, 130, 16, 2, 2)])
def test_matrix_core_attention_with_kept_first_tokens_sink_and_gate(n, window, keep, d, nH, nKV):
    """The same function on the matrix-core kernels (bfloat16, values as wide as keys): single rows in splits of the keys
    with the merge launch and whole in one workgroup, tiles of 64 and 128 rows whole and with their keys in splits, a
    portion behind a past."""
    q, k, v, kc, vc, table = _paged_case("bfloat16", n, window, keep, d, d, nH, nKV)
    gate = torch.rand(n, nH, generator=torch.Generator().manual_seed(5))
    want = pp.sink_softmax_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 2.0, window, keep)
    want = T64(want * gate.double().numpy()[:, :, None]).reshape(n, nH * d)
    row_req, pos = torch.zeros(n, dtype=torch.int32, device=DEV), torch.arange(n, dtype=torch.int32, device=DEV)
    qd, kd, vd, td, gd = q.to(DEV), kc.to(DEV), vc.to(DEV), table.to(DEV), gate.to(DEV)
    for chunk, waves in ((32, 0), (128, 0), (128, 1), (128, 4)):
        if waves and ops.row_waves_fit(nH, nKV, d, waves) != waves:
            continue
        out = torch.zeros(n, nH * d, dtype=torch.bfloat16, device=DEV)
        ops.attention_rows(qd, kd, vd, out, None, n, row_req, pos, td, window, 2.0, chunk, -(-n // chunk) + 1, waves, False, keep, 0.0, gd)
        assert rel_err(out.cpu(), want) < 2e-2, (chunk, waves)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    for qt in (1, 2):
        rows_per = ops.attention_tile_rows(d, qt)
        for first in (0, n - 70 if n > 100 else 0):            # the whole prompt, and its last rows behind the others as a past
            m = n - first
            tiles = list(range(0, m, rows_per))
            for split_chunk in (0, 64, 192):
                splits = {}
                if split_chunk:
                    splits = dict(chunk=split_chunk, max_splits=-(-n // split_chunk), rows=torch.arange(m, dtype=torch.int32, device=DEV),
                                  row_req=row_req[:m], positions=pos[first:].contiguous())
                out = torch.zeros(m, nH * d, dtype=torch.bfloat16, device=DEV)
                ops.attention_tiles(qd[first:].contiguous(), kd, vd, out, dev([0] * len(tiles)), dev(tiles), dev([0]), dev([m]), dev([n]), td,
                                    window, 2.0, qt, **splits, keep_first=keep, sink=0.0, gate=gd[first:].contiguous())
                assert rel_err(out.cpu(), want[first:]) < 2e-2, (qt, first, split_chunk)


def test_the_aim_of_the_attention_case_shows_an_edge_one_off():
    """What the case above is built for: moving the window or the kept range by one changes rows by tens of percent."""
    n, window, keep, d, dv = 150, 33, 5, 64, 48
    q, k, v, _, _, _ = _paged_case("float32", n, window, keep, d, dv, 2, 1)
    a = pp.sink_softmax_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 2.0, window, keep)
    for w2, k2 in ((window + 1, keep), (window - 1, keep), (window, keep + 1), (window, keep - 1)):
        b = pp.sink_softmax_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 2.0, w2, k2)
        assert np.abs(a - b).max() > 0.2 * np.abs(a).max(), (w2, k2)
    b = pp.sink_softmax_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), 2.0, window, keep, sink=False)
    assert np.abs(a - b).max() > 0.05 * np.abs(a).max()


def _step_arrays(lens):
    q_len = torch.tensor(lens, dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0).to(torch.int32) - q_len
    row_req = torch.repeat_interleave(torch.arange(len(lens), dtype=torch.int32), q_len.long())
    return q_start, q_len, row_req


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C,taps,extra", [(96, 4, 96), (40, 2, 0), (56, 1, 8), (300, 7, 21), (50, 3, 50)])
def test_causal_convolution_carries_its_last_inputs_from_step_to_step(dtype, C, taps, extra):
    """Three requests in slots 2, 0 and 3 of 4, fed in unequal portions (down to one token, fewer than the taps) in shared
    steps; each must come out as the convolution of its whole sequence."""
    dt = DT[dtype]
    lens_total = [29, 11, 40]
    slots = torch.tensor([2, 0, 3], dtype=torch.int32)
    xs = [rnd(10 + i, n, C + extra).to(dt) for i, n in enumerate(lens_total)]
    w, b = rnd(20, C, taps, scale=0.6).to(dt), rnd(21, C, scale=0.3).to(dt)
    state = torch.zeros((4, C * (taps - 1) + 13), dtype=torch.float32, device=DEV)
    state[1] = 7.0                                               # somebody else's slot: must come out untouched
    got = [[] for _ in lens_total]
    at = [0, 0, 0]
    for step in ([5, 1, 17], [1, 2, 1], [2, 1, 2], [20, 7, 19], [1, 0, 1]):
        live = [i for i, m in enumerate(step) if m]
        x = torch.cat([xs[i][at[i]:at[i] + step[i]] for i in live])
        q_start, q_len, row_req = _step_arrays([step[i] for i in live])
        out = ops.causal_conv_silu(x.to(DEV), C, w.to(DEV), b.to(DEV), state, row_req.to(DEV), q_start.to(DEV), q_len.to(DEV),
                                   slots[live].to(DEV)).cpu()
        o = 0
        for i in live:
            got[i].append(out[o:o + step[i]]); o += step[i]; at[i] += step[i]
    assert at == lens_total
    for i, x in enumerate(xs):
        want = pp.silu(pp.causal_conv(x.double().numpy()[:, :C], w.double().numpy(), b.double().numpy()))
        assert rel_err(torch.cat(got[i]), T64(want)) < (1e-5 if dtype == "float32" else 1e-2), i
    assert torch.all(state[1] == 7.0) and torch.all(state[:, C * (taps - 1):][[0, 2, 3]] == 0)


@pytest.mark.parametrize("taps", [2, 3, 4, 5])
def test_causal_convolution_of_many_rows(taps):
    """Steps of many rows in bfloat16 take the kernel that works in 16-byte pieces (2 to 4 taps): two requests, the second
    continued from its slot, then single rows behind them."""
    C, lens = 2048, [[300, 260], [270, 1], [1, 2]]
    totals = [sum(step[i] for step in lens) for i in range(2)]
    xs = [rnd(80 + i, n, 2 * C).to(torch.bfloat16) for i, n in enumerate(totals)]
    w, b = rnd(82, C, taps, scale=0.6).to(torch.bfloat16), rnd(83, C, scale=0.3).to(torch.bfloat16)
    state = torch.zeros((3, C * (taps - 1)), dtype=torch.float32, device=DEV)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    got, at = [[], []], [0, 0]
    for step in lens:
        x = torch.cat([xs[i][at[i]:at[i] + step[i]] for i in range(2)])
        q_start, q_len, row_req = _step_arrays(step)
        out = ops.causal_conv_silu(x.to(DEV), C, w.to(DEV), b.to(DEV), state, row_req.to(DEV), q_start.to(DEV), q_len.to(DEV), slots).cpu()
        got[0].append(out[:step[0]]); got[1].append(out[step[0]:])
        at = [at[i] + step[i] for i in range(2)]
    for i in range(2):
        want = pp.silu(pp.causal_conv(xs[i].double().numpy()[:, :C], w.double().numpy(), b.double().numpy()))
        assert rel_err(torch.cat(got[i]), T64(want)) < 1e-2, i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C,N", [(96, 6), (40, 17), (56, 4), (256, 16), (50, 5), (24, 1), (32, 33), (16, 128)])
def test_selective_scan_carries_its_state_from_step_to_step(dtype, C, N):
    dt = DT[dtype]
    lens_total = [33, 9, 50]
    slots = torch.tensor([1, 3, 0], dtype=torch.int32)
    offset = 11
    u = [rnd(30 + i, n, C).to(dt) for i, n in enumerate(lens_total)]
    z = [rnd(33 + i, n, 2 * C + 3).to(dt) for i, n in enumerate(lens_total)]        # the gate's input is a view of wider rows
    bc = [rnd(36 + i, n, 2 * N + 2).to(dt) for i, n in enumerate(lens_total)]
    dt_raw = [rnd(39 + i, n, C, scale=2.0).float() for i, n in enumerate(lens_total)]
    dt_b, D = (rnd(42, C) - 2.0).to(dt), (rnd(43, C, scale=0.5) + 1.0).to(dt)
    A = -torch.exp(torch.log(1.0 + 15.0 * torch.rand(C, N, generator=torch.Generator().manual_seed(44)))).float()
    state = torch.zeros((5, offset + C * N + 4), dtype=torch.float32, device=DEV)
    got = [[] for _ in lens_total]
    at = [0, 0, 0]
    for step in ([7, 1, 30], [1, 1, 1], [2, 0, 3], [20, 5, 15], [3, 2, 1]):
        live = [i for i, m in enumerate(step) if m]
        cat = lambda xs: torch.cat([xs[i][at[i]:at[i] + step[i]] for i in live])
        q_start, q_len, _ = _step_arrays([step[i] for i in live])
        zz = cat(z).to(DEV)
        out = ops.selective_scan(cat(u).to(DEV), cat(dt_raw).to(DEV), dt_b.to(DEV), A.to(DEV), cat(bc).to(DEV), D.to(DEV), zz[:, 3:3 + C],
                                 state, offset, q_start.to(DEV), q_len.to(DEV), slots[live].to(DEV)).cpu()
        o = 0
        for i in live:
            got[i].append(out[o:o + step[i]]); o += step[i]; at[i] += step[i]
    assert at == lens_total
    for i in range(3):
        step_size = pp.softplus(dt_raw[i].double().numpy() + dt_b.double().numpy())
        y = pp.selective_scan(u[i].double().numpy(), step_size, A.double().numpy(), bc[i].double().numpy()[:, :N],
                              bc[i].double().numpy()[:, N:2 * N], D.double().numpy())
        want = y * pp.silu(z[i].double().numpy()[:, 3:3 + C])
        assert rel_err(torch.cat(got[i]), T64(want)) < (2e-5 if dtype == "float32" else 1e-2), i
    s = state.cpu()
    assert not s[[2, 4]].any() and not s[:, :offset].any() and not s[:, offset + C * N:].any()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("C,N,chunk", [(96, 6, 64), (40, 17, 16), (256, 16, 64), (50, 5, 7), (24, 1, 200)])
def test_selective_scan_in_chunks_side_by_side(dtype, C, N, chunk):
    """Long portions cut into chunks that first run from zero and then from what the chunks before them leave: the same
    outputs and the same final state as the walk in one piece, for requests of unequal length that start from a state."""
    dt = DT[dtype]
    lens = [300, 1, 70, 129]
    T = sum(lens)
    u, z, bc = rnd(70, T, C).to(dt), rnd(71, T, C).to(dt), rnd(72, T, 2 * N).to(dt)
    dt_raw = rnd(73, T, C, scale=2.0).float()
    dt_b, D = (rnd(74, C) - 2.0).to(dt), (rnd(75, C, scale=0.5) + 1.0).to(dt)
    A = -torch.exp(torch.log(1.0 + 15.0 * torch.rand(C, N, generator=torch.Generator().manual_seed(76)))).float()
    q_start, q_len, _ = _step_arrays(lens)
    slots = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    start = rnd(77, 4, C * N).float()
    outs, states = [], []
    for chunks in (None, ops.scan_chunks(q_start.numpy(), q_len.numpy(), chunk, DEV)):
        state = start.clone().to(DEV)
        outs.append(ops.selective_scan(u.to(DEV), dt_raw.to(DEV), dt_b.to(DEV), A.to(DEV), bc.to(DEV), D.to(DEV), z.to(DEV), state, 0,
                                       q_start.to(DEV), q_len.to(DEV), slots.to(DEV), chunks).cpu())
        states.append(state.cpu())
    assert rel_err(outs[1], outs[0]) < (2e-5 if dtype == "float32" else 1e-2)
    assert rel_err(states[1], states[0]) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M", [1, 7, 16, 40, 100, 300])
@pytest.mark.parametrize("K,ff", [(64, 96), (256, 384), (100, 50)])
def test_gated_feed_forward_with_the_tanh_form_of_gelu(dtype, M, K, ff):
    dt = DT[dtype]
    x, g, u = rnd(50, M, K).to(dt), rnd(51, ff, K, scale=2.0 * K ** -0.5).to(dt), rnd(52, ff, K, scale=K ** -0.5).to(dt)
    pairs = ops.prepare_linear(torch.stack([g, u], dim=1).reshape(2 * ff, K).contiguous().to(DEV))
    want = pp.gelu_tanh(x.double().numpy() @ g.double().numpy().T) * (x.double().numpy() @ u.double().numpy().T)
    got = ops.linear_swiglu(x.to(DEV), pairs, ops.ACT_GELU_TANH).cpu()
    assert rel_err(got, T64(want)) < (1e-5 if dtype == "float32" else 1.5e-2)
    silu = ops.linear_swiglu(x.to(DEV), pairs).cpu()                 # the default is still silu
    assert rel_err(silu, T64(pp.silu(x.double().numpy() @ g.double().numpy().T) * (x.double().numpy() @ u.double().numpy().T))) < (1e-5 if dtype == "float32" else 1.5e-2)
    z = torch.linspace(-6, 6, 4001, dtype=torch.float32)
    both = torch.stack([z, torch.ones_like(z)], dim=1).reshape(1, -1).contiguous()
    assert rel_err(ops.swiglu(both.to(DEV), interleaved=True, act=ops.ACT_GELU_TANH).cpu()[0], T64(pp.gelu_tanh(z.double().numpy()))) < 1e-6


@pytest.mark.parametrize("H", [64, 100, 384, 5000])
def test_stream_add_with_a_factor_and_scaled_embedding(H):
    T, eps, m = 9, 1e-5, 0.625
    x, d, w = rnd(60, T, H).float(), rnd(61, T, H, scale=3.0), rnd(62, H) + 1.0
    want_x = x.double() + m * d.float().double()
    want = T64(pp.rms_norm(want_x.numpy(), w.float().double().numpy(), eps))
    for delta in (d.float().to(DEV), ops.ScaledDelta(d.float().to(DEV) * 2.0, m / 2.0),
                  ops.ScaledDelta(ops.SliceSums(torch.stack([d.float() * 0.25, d.float() * 0.75]).to(DEV), torch.float32), m)):
        res = x.clone().to(DEV)
        out = ops.add_rmsnorm(res, delta, w.float().to(DEV), eps, torch.float32, delta_scale=m if torch.is_tensor(delta) else 1.0)
        assert rel_err(res.cpu(), want_x) < 1e-6 and rel_err(out.cpu(), want) < 1e-5
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=DEV)       # picked rows: nothing is written back
    res = x.clone().to(DEV)
    out = ops.add_rmsnorm(res, ops.ScaledDelta(d.float().to(DEV), m), w.float().to(DEV), eps, torch.float32, rows)
    assert torch.equal(res.cpu(), x) and rel_err(out.cpu(), want[[4, 0, 4]]) < 1e-5
    table = rnd(63, 50, H).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    assert torch.equal(ops.embedding(ids.to(DEV), table.to(DEV), 0.375).cpu(), table[ids.long()].float() * 0.375)
    if H % 8 == 0 and H <= 4096:          # a product of few rows that adds itself to the stream takes the factor too
        K = 72
        a, wo = rnd(64, T, K).to(torch.bfloat16), rnd(65, H, K, scale=K ** -0.5).to(torch.bfloat16)
        lw = ops.prepare_linear(wo.to(DEV))
        nw = (rnd(66, H) + 1.0).to(torch.bfloat16)
        if ops.adds_into_stream(T, lw, nw.to(DEV)):
            res = x.clone().to(DEV)
            rows_out = ops.linear_into_stream(a.to(DEV), lw, res, nw.to(DEV), eps, m)
            want_x = x.double() + m * (a.double() @ wo.double().T)
            assert rel_err(res.cpu(), want_x) < 1e-5
            nxt = ops.linear(rows_out, ops.prepare_linear(torch.eye(H, dtype=torch.bfloat16, device=DEV)), out_dtype=torch.float32)
            assert rel_err(nxt.cpu(), T64(pp.rms_norm(want_x.numpy(), nw.double().numpy(), eps))) < 1e-2


# ---- the model through the engine -----------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(pm.CONFIGS))
def test_whole_prompts(name, dtype, folders):
    folder, vocab = folders[name, dtype], pm.CONFIGS[name]["vocab"]
    runner = load_runner(folder, DT[dtype], num_pages=32, max_requests=2)
    for seed, n in ((1, 1), (2, 2), (3, 37), (4, 200)):
        ids = ids_of(seed, n, vocab)
        assert rel_err(run_whole(runner, "w", ids), plain(folder, ids)) < TOL[dtype], (name, n)
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["recurrent_only", "no_windows", "one_attention"])
def test_models_without_pages_or_without_windows(kind, dtype, tmp_path):
    """A model of recurrences alone keeps no pages at all; attention without a window keeps everything (kept first tokens
    then mean nothing); a single attention layer that mixes values has nobody to mix with."""
    layers = {
        "recurrent_only": [pm.layer(pm.mamba1(48, 8, 4, 3), 40), pm.layer(pm.mamba1(32, 3, 2, 4), None)],
        "no_windows": [pm.layer(pm.attention(4, 1, 16, 16, 0.5, 10000.0, 16, window=None, keep_first=9), 40),
                       pm.layer(pm.attention(2, 2, 32, 16, 0.4, 500.0, 8, v_mix=False), 24)],
        "one_attention": [pm.layer(pm.attention(4, 4, 64, 64, 0.2, 5e5, 32, window=70, keep_first=9, scaling=(6.0, 2048, 24.0, 1.0)), 64)],
    }[kind]
    cfg = pm.model(150, 64, 1e-5, 0.5, 0.5, layers)
    folder = pm.write_model(str(tmp_path / "m"), cfg, 9, gain=GAIN[dtype])
    runner = load_runner(folder, DT[dtype], num_pages=20, max_requests=3)
    assert len(runner.manager.groups) == {"recurrent_only": 0, "no_windows": 1, "one_attention": 1}[kind]
    ids = ids_of(8, 230, 150)
    want = plain(folder, ids)
    assert rel_err(run_whole(runner, "w", ids), want) < TOL[dtype]
    runner.add_request("c")
    runner.add_request("o")
    rows, p = [], 0
    for m in [2, 100, 1, 1, 64, 3, 1, 58]:
        rows.append(runner.step([StepEntry("o", ids_of(p, 2, 150), []), StepEntry("c", ids[p:p + m], list(range(m)))]).cpu())
        p += m
    assert p == len(ids) and rel_err(torch.cat(rows), want) < TOL[dtype]
    runner.manager.check()


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_stream_after_every_layer(name, folders):
    folder = folders[name, "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    ids = ids_of(3, 50, pm.CONFIGS[name]["vocab"])
    _, streams = plain(folder, ids, layers=True)
    runner.add_request("p")
    runner.manager.reserve("p", len(ids))
    ctx = StepContext([StepEntry("p", ids, [0])], runner.manager, torch.float32, runner.device)
    model = runner.model
    x, pending = model.embedding.forward(ctx), None
    for i, e in enumerate(model.plan.schedule):
        x, pending = model.blocks[e.layer].forward(x, pending, ctx, runner.storage.binding(i))
        after = x + pending.tensor() if isinstance(pending, ops.ScaledDelta) else x + (pending.sum(torch.float32) if hasattr(pending, "parts") else pending.float())
        assert rel_err(after.cpu(), streams[i]) < 1e-5, i


def test_first_tokens(folders):
    """Position 0 sees itself (and the sink) alone: its logits are a function of the token; the first tokens of a sequence
    see no window's edge, no kept range and a zero state."""
    folder = folders["D", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    for tok in (0, 77, 98):
        a, b = run_whole(runner, "x", [tok]), run_whole(runner, "y", [tok, 5, 9, 2])
        assert rel_err(a, plain(folder, [tok])) < TOL["float32"] and torch.equal(a[0], b[0])
        assert rel_err(b, plain(folder, [tok, 5, 9, 2])) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D", "E"])
def test_prefill_against_decoding_and_portions(name, dtype, folders):
    folder, vocab = folders[name, dtype], pm.CONFIGS[name]["vocab"]
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
@pytest.mark.parametrize("name", ["A", "C"])
def test_unequal_requests_in_one_batch_against_each_alone(name, dtype, folders):
    folder, vocab = folders[name, dtype], pm.CONFIGS[name]["vocab"]
    runner = load_runner(folder, DT[dtype], num_pages=40, max_requests=4)
    seqs = {"a": ids_of(41, 90, vocab), "b": ids_of(42, 23, vocab), "c": ids_of(43, 140, vocab), "d": ids_of(44, 2, vocab)}
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
def test_long_decoding_gives_pages_back_but_keeps_the_first(dtype, folders):
    folder = folders["A", dtype]
    runner = load_runner(folder, DT[dtype], num_pages=30, max_requests=2)
    ids = ids_of(51, 420, 300)
    want = plain(folder, ids)
    runner.add_request("d")
    got = [runner.step([StepEntry("d", ids[:9], [8])]).cpu()[0]]
    for p in range(9, len(ids)):
        got.append(runner.step([StepEntry("d", [ids[p]], [0])]).cpu()[0])
    assert rel_err(torch.stack(got), want[8:]) < TOL[dtype]
    runner.manager.check()
    assert [(g.window, g.keep_first) for g in runner.manager.groups] == [(None, 0), (20, 3), (33, 5)]
    tables = [runner.manager.block_table("d", g) for g in range(3)]
    held = [sum(1 for p in t if p >= 0) for t in tables]
    assert held[0] == -(-420 // 16) and held[1] <= 20 // 16 + 3 and held[2] <= 33 // 16 + 3
    assert tables[1][0] >= 0 and tables[2][0] >= 0 and tables[1][1] < 0          # the page of the kept first tokens stays
    assert runner.graph_replays > 0          # decode steps of a model with state of its own are replayed graphs too


def test_a_freed_slot_starts_from_zero_state(folders):
    """The same prompt gives the same logits in a slot and pages that another request has just used."""
    folder = folders["B", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=6, max_requests=1)
    a, b = ids_of(52, 80, 131), ids_of(53, 61, 131)
    first = run_whole(runner, "a", a)
    run_whole(runner, "b", b)
    assert torch.equal(run_whole(runner, "a2", a), first)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(pm.CONFIGS))
def test_replay_of_traces_with_pages_and_slots_used_again(name, dtype, folders, tmp_path):
    """Through bin/trace_run as a user would: whole, prefill then decode, portions, and mixed steps of up to four live
    requests, one process, a pool so small that pages and slots are used again."""
    folder, vocab = folders[name, dtype], pm.CONFIGS[name]["vocab"]
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


def test_replay_takes_a_file_with_tensors_nobody_reads(folders, tmp_path):
    """A model file may hold more than the model reads (a second norm in a layer without feed-forward) and less where a
    tensor is read by nobody (the first mixing layer's weight): the replay tool lists the former and goes on, unless told to
    be strict; the logits are the same."""
    from safetensors.torch import load_file, save_file
    import shutil
    src = folders["B", "float32"]
    folder = str(tmp_path / "m")
    shutil.copytree(src, folder)
    t = load_file(os.path.join(folder, "model.safetensors"))
    t["l2.norm2"] = torch.ones(88, dtype=torch.bfloat16)           # layer 2 has no feed-forward
    del t["l1.mix.vmix"]                                           # the one mixing layer hands its values on and mixes nothing
    save_file(t, os.path.join(folder, "model.safetensors"))
    ids = ids_of(95, 40, 131)
    step = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": ids, "want": [39]}], "end": ["a"]}) + "\n"
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--max-tokens", "64"]
    ok = subprocess.run(cmd + ["--out", str(tmp_path / "o1")], input=step, capture_output=True, text=True, timeout=120)
    assert ok.returncode == 0 and "done 0" in ok.stdout and "l2.norm2" in ok.stderr
    got = torch.from_numpy(np.fromfile(str(tmp_path / "o1" / "0.f32"), dtype="<f4"))
    assert rel_err(got[None], plain(src, ids)[39:40]) < TOL["float32"]
    strict = subprocess.run(cmd + ["--out", str(tmp_path / "o2"), "--strict-weights"], input=step, capture_output=True, text=True, timeout=120)
    assert strict.returncode != 0 and "l2.norm2" in strict.stderr


def _drawn_config(seed):
    """A configuration drawn from sizes of every kind: heads the matrix-core kernels take and heads only the plain kernel
    takes, grouped and ungrouped, values wider and narrower than keys, windows around a page's size with and without
    kept first tokens, recurrences of few and many states, layers in any order with and without feed-forward."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 72, 96, 160])
    layers, mixing = [], None
    for _ in range(rng.choice([1, 2, 3, 4])):
        if rng.random() < 0.4:
            mixer = pm.mamba1(rng.choice([24, 64, 100, 192]), rng.choice([1, 4, 7, 16, 24]), rng.choice([1, 4, 8, 10]), rng.choice([1, 2, 4, 5]))
        else:
            kv = rng.choice([1, 2, 3])
            dim, vdim = rng.choice([8, 12, 16, 32, 48, 64, 96, 128]), rng.choice([8, 10, 16, 32, 64])
            if rng.random() < 0.5:
                vdim = dim                                  # (values as wide as keys: the matrix-core kernels where the size allows)
            v_mix = rng.random() < 0.7
            if v_mix:
                mixing = mixing or (kv, vdim)
                kv, vdim = mixing
            dims = rng.choice([dim, max(2, dim // 2 // 2 * 2), 2])
            window = rng.choice([None, 5, 16, 17, 64, 100])
            mixer = pm.attention(kv * rng.choice([1, 2, 4]), kv, dim, vdim, rng.choice([1.0, 2.0, 4.0]) / dim ** 0.5 * 2.0, rng.choice([100.0, 10000.0, 1e6]),
                                 dims, window, rng.choice([0, 1, 4, 16, 30]) if window else 0, v_mix,
                                 rng.choice([None, (4.0, 64, 8.0, 1.0), (6.0, 2048, 24.0, 1.0)]))
        layers.append(pm.layer(mixer, rng.choice([None, 24, 56, 80])))
    return pm.model(rng.choice([61, 128, 500]), width, rng.choice([1e-5, 1e-6, 1e-3]), rng.choice([1.0, 0.5, 3.0]), rng.choice([1.0, 0.5, 0.3]), layers)


@pytest.mark.parametrize("seed", range(14))
def test_drawn_configurations(seed, tmp_path):
    """Whole prompts, portions and decoding of drawn configurations against the plain implementation, both precisions."""
    cfg = _drawn_config(seed)
    for dtype in ("float32", "bfloat16"):
        folder = pm.write_model(str(tmp_path / dtype), cfg, 80 + seed, gain=GAIN[dtype])
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
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_engine(name, folders):
    folder, vocab = folders[name, "float32"], pm.CONFIGS[name]["vocab"]
    cfg, W = pm.load_plain(folder)
    prompts = [ids_of(70 + i, n, vocab) for i, n in enumerate([5, 40, 1, 77, 19, 130])]
    want = [pp.greedy_generate(cfg, W, p, 10) for p in prompts]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32, prefill_tokens_alone=48)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert [o.token_ids for o in outs] == want
    assert engine.runner.graph_replays > 0                       # decode steps ran as replayed graphs
    folder = folders[name, "bfloat16"]
    cfg, W = pm.load_plain(folder)
    engine = Engine.load(folder, dtype="bfloat16", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for p, o in zip(prompts, outs):        # bfloat16 may pick another token where two logits nearly tie
        full = pp.forward(cfg, W, p + o.token_ids)
        for i, tok in enumerate(o.token_ids):
            row = full[len(p) - 1 + i]
            assert row[tok] >= row.max() - 0.06 * np.abs(row).max(), (name, i)


def test_completion_from_the_command_line(folders, capsys):
    from inferflux_amd import cli
    folder = folders["B", "float32"]
    cfg, W = pm.load_plain(folder)
    prompt = ids_of(90, 21, 131)
    assert cli.main(["completion", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "7", "--temperature", "0",
                     "--ignore-eos", "--dtype", "float32", "--kv-pages", "32", "--max-parallel-sequences", "2"]) == 0
    said = capsys.readouterr().out
    want = pp.greedy_generate(cfg, W, prompt, 7)
    assert str(want)[1:-1].replace(" ", "") in said.replace(" ", ""), (want, said)
