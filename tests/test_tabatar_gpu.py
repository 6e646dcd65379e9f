"""The Tabatar design on the GPU: every mechanism's kernel alone against the plain implementation's function, then the
model through the engine's step function, its replay tool and its generation loop, under every way of cutting and
batching, in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_tabatar as pt
import tabatar_models as tm
import traces
from conftest import ROOT, rel_err

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd import SamplingParams
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepContext, StepEntry
    from inferflux_amd.engine.engine import Engine
    from inferflux_amd.kernels import ops
    from inferflux_amd.parts import block as blk
    from inferflux_amd.parts.position import RotaryPosition

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# Largest difference of a logit from the plain model's, relative to the largest logit.  32-bit: rounding over a few hundred
# operations.  bfloat16: the worst seen over these tests and half as much again; a key, a window's edge, a state, a bias or a
# stream that is wrong moves a row by 10-100 % (the kernels' own tests aim queries at the edges so that it does).  The rows of
# a sequence's first positions get more in bfloat16: a recurrent head's output is normed, so while its state holds one or a
# few outer products the output's direction hangs on single q . k products, which rounding q and k to bfloat16 moves by a
# large fraction wherever they happen to be small (32-bit pins these rows).
TOL = {"float32": 1e-5, "bfloat16": 5e-2}
TOL_FIRST = {"float32": 1e-5, "bfloat16": 1.6e-1}
FIRST = 16
GAIN = {"float32": 2.0, "bfloat16": 1.0}
DEV = "cuda"


def rnd(seed, *shape, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


def ids_of(seed, n, vocab):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def T64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


def N64(t):
    return t.double().cpu().numpy()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """(configuration, precision) -> model folder.  The 32-bit runs take routers with random weights and biases; the bfloat16
    runs take models in which no choice of experts is a close call (``write_model``)."""
    out = {}
    for i, n in enumerate(tm.CONFIGS):
        for dtype in DT:
            out[n, dtype] = tm.write_model(str(tmp_path_factory.mktemp(f"tabatar{n}{dtype}")), tm.config(n), 40 + i, gain=GAIN[dtype],
                                           decisive_router=dtype == "bfloat16")
    return out


_PLAIN = {}


def plain(folder, ids, layers=False):
    if folder not in _PLAIN:
        _PLAIN[folder] = tm.load_plain(folder)
    key = (folder, tuple(ids), layers)
    if key not in _PLAIN:
        out = pt.forward(*_PLAIN[folder], list(ids), return_layers=layers)
        _PLAIN[key] = (T64(out[0]), T64(out[1])) if layers else T64(out)
    return _PLAIN[key]


def off(got, want, dtype, positions=None):
    """The rows' largest differences from ``want`` (relative to its largest entry) over what their positions allow: below 1 is
    within tolerance.  ``positions``: each row's place in its sequence (by default row i is position i)."""
    want = want.double()
    err = (got.double() - want).abs().amax(dim=1) / want.abs().max()
    positions = torch.arange(len(err)) if positions is None else torch.as_tensor(list(positions))
    allowed = torch.where(positions < FIRST, TOL_FIRST[dtype], TOL[dtype])
    rel_err(got, want)
    return float((err / allowed).max())


def run_whole(runner, rid, ids, want=None):
    runner.add_request(rid)
    out = runner.step([StepEntry(rid, ids, list(range(len(ids))) if want is None else want)]).cpu()
    runner.free_request(rid)
    return out


def _step_arrays(lens):
    q_len = torch.tensor(lens, dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0).to(torch.int32) - q_len
    return q_start, q_len


# ---- each mechanism's kernel alone ------------------------------------------------------------
@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (4.0, 1.0, 4.0, 64)), (24, 5e5, (8.0, 1.0, 4.0, 8192)), (6, 300.0, None),
                                               (32, 5e5, (2.5, 0.5, 16.0, 4096)), (4, 50.0, (16.0, 2.0, 3.0, 32)), (64, 1e4, (32.0, 1.0, 4.0, 16))])
def test_rotation_table_with_frequencies_scaled_in_bands(dims, base, scaling):
    sc = dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None
    part = RotaryPosition(head_dim=dims + 4, theta=base, rotary_dim=dims, scaling=sc)
    f = pt.banded_frequencies(dims, base, sc)
    assert rel_err(part.frequencies(), T64(f)) < 1e-12 and part.magnitude == 1.0
    positions = torch.tensor([0, 1, 2, 77, 1000, 40000], dtype=torch.int32, device=DEV)
    cos, sin = ops.rope_table(positions, part.inv_freq(DEV), part.magnitude)
    a = positions.cpu().double()[:, None] * T64(f)[None, :]
    small = slice(0, 3)     # (float32 angles lose digits at large positions: the first positions pin the table itself)
    assert (cos.cpu().double()[small] - torch.cos(a)[small]).abs().max() < 2e-6
    assert (sin.cpu().double()[small] - torch.sin(a)[small]).abs().max() < 2e-6
    assert (cos.cpu().double() - torch.cos(a)).abs().max() < 5e-3 * max(1.0, 40000 * float(f[0]) * 1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [37, 300])
@pytest.mark.parametrize("nH,nKV,d,dv,dims", [(4, 2, 16, 24, 8), (3, 3, 12, 12, 12), (2, 1, 20, 20, 20), (8, 2, 64, 64, 32), (3, 1, 10, 14, 6),
                                              (16, 2, 48, 96, 48), (8, 2, 96, 96, 32), (4, 4, 128, 128, 64), (5, 5, 130, 70, 100)])
def test_row_kernel_norms_heads_with_a_weight_before_it_turns_them(dtype, T, nH, nKV, d, dv, dims):
    """q and k heads normed with a weight each (one for all q heads, one for all k heads), then turned; values written as they
    are; the gate's columns behind them left alone."""
    P, pages, eps = 16, -(-T // 16) + 4, 1e-5
    dt = DT[dtype]
    gate_cols = nH * dv
    width = (nH + nKV) * d + nKV * dv + gate_cols
    qkv = rnd(1, T, width, scale=1.5).to(dt)
    qw, kw = (rnd(2, d, scale=0.3) + 1.0).to(dt), (rnd(3, d, scale=0.3) + 1.0).to(dt)
    positions = torch.tensor([5 + 3 * t for t in range(T)], dtype=torch.int32)
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(4))[:T].to(torch.int32)
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    part = RotaryPosition(head_dim=d, theta=1000.0, rotary_dim=dims, scaling=sc)
    cos, sin = ops.rope_table(positions.to(DEV), part.inv_freq(DEV), part.magnitude)
    k = torch.zeros((pages, nKV, P, d), dtype=dt, device=DEV)
    v = torch.zeros((pages, nKV, dv, P), dtype=dt, device=DEV)
    q = ops.rope_append(qkv.to(DEV), None, slots.to(DEV), cos, sin, ops.ROPE_SPLIT_HALF, dims, nH, nKV, d, k, v, P, dv,
                        qk_norm=(qw.to(DEV), kw.to(DEV), eps), extra_cols=gate_cols)
    x, pos = N64(qkv), positions.numpy()
    tol = 1e-5 + 1e-7 * int(positions.max()) if dtype == "float32" else 1e-2
    want_q = pt.rotate(pt.rms_norm(x[:, :nH * d].reshape(T, nH, d), N64(qw), eps), pos, dims, 1000.0, sc)
    assert rel_err(q.cpu(), T64(want_q)) < tol
    want_k = pt.rotate(pt.rms_norm(x[:, nH * d:(nH + nKV) * d].reshape(T, nKV, d), N64(kw), eps), pos, dims, 1000.0, sc)
    got_k = k.cpu().permute(0, 2, 1, 3).reshape(pages * P, nKV, d)[slots.long()]
    assert rel_err(got_k, T64(want_k)) < tol
    got_v = v.cpu().permute(0, 3, 1, 2).reshape(pages * P, nKV * dv)[slots.long()]
    assert rel_err(got_v, qkv[:, (nH + nKV) * d:(nH + nKV) * d + nKV * dv]) < tol
    untouched = torch.ones(pages * P, dtype=torch.bool)
    untouched[slots.long()] = False
    assert not k.cpu().permute(0, 2, 1, 3).reshape(pages * P, -1)[untouched].any()
    if dtype == "float32":       # partial sums of a sliced product give the same as their sum
        parts = torch.stack([qkv * 0.5, qkv * 0.25, qkv * 0.25]).to(DEV)
        k2, v2 = torch.zeros_like(k), torch.zeros_like(v)
        q2 = ops.rope_append(ops.SliceSums(parts, dt), None, slots.to(DEV), cos, sin, ops.ROPE_SPLIT_HALF, dims, nH, nKV, d, k2, v2, P, dv,
                             qk_norm=(qw.to(DEV), kw.to(DEV), eps), extra_cols=gate_cols)
        assert rel_err(q2.cpu(), q.cpu()) < 1e-6 and rel_err(k2.cpu(), k.cpu()) < 1e-6 and rel_err(v2.cpu(), v.cpu()) < 1e-6


def _paged_case(dtype, n, window, d, dv, nH, nKV, P=16, seed=20):
    """One request of n positions whose rows are all queried at once, its pages scattered over the pool.  Every key carries a
    mark of its own and every query is aimed, hard, at the key on the window's inner edge and, harder, at the one just outside
    it, so that a window one position off changes which values a head returns."""
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
        for j, w in ((inner, 3.0), (inner - 1, 5.0)):
            if 0 <= j:
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
@pytest.mark.parametrize("n,window,d,dv,nH,nKV", [(70, 20, 16, 24, 4, 2), (150, 33, 48, 48, 8, 2), (40, 7, 20, 20, 2, 1), (200, 64, 48, 96, 4, 4),
                                                  (130, None, 44, 40, 4, 2), (100, 16, 64, 64, 16, 2), (300, 40, 96, 96, 3, 1), (90, 1, 12, 12, 3, 3)])
def test_attention_sees_exactly_its_window_with_an_ordinary_softmax(dtype, n, window, d, dv, nH, nKV):
    q, k, v, kc, vc, table = _paged_case(dtype, n, window, d, dv, nH, nKV)
    row_req, pos = torch.zeros(n, dtype=torch.int32, device=DEV), torch.arange(n, dtype=torch.int32, device=DEV)
    got = ops.attention_plain(q.to(DEV), kc.to(DEV), vc.to(DEV), row_req, pos, table.to(DEV), window, 2.0, 0, None, None).cpu()
    want = pt.window_attention(N64(q), N64(k), N64(v), 2.0, window)
    assert rel_err(got.reshape(n, nH, dv), T64(want)) < (2e-5 if dtype == "float32" else 2e-2)
    if window and window > 1:       # the aim works: a window one longer or one shorter gives other rows
        for other in (window + 1, window - 1):
            assert rel_err(T64(pt.window_attention(N64(q), N64(k), N64(v), 2.0, other)), T64(want)) > 0.2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,C,ld,col", [(1, 24, 60, 36), (37, 96, 200, 100), (300, 384, 900, 512), (5, 7, 7, 0)])
def test_elementwise_sigmoid_gate_from_the_projected_rows(dtype, T, C, ld, col):
    dt = DT[dtype]
    x, rows = rnd(5, T, C).to(dt), rnd(6, T, ld, scale=2.0).to(dt)
    got = ops.sigmoid_gate(x.to(DEV), rows.to(DEV), col).cpu()
    want = N64(x) * pt.sigmoid(N64(rows)[:, col:col + C])
    assert rel_err(got, T64(want)) < (1e-6 if dtype == "float32" else 6e-3)
    if dtype == "float32":
        parts = torch.stack([rows * 0.75, rows * 0.25]).to(DEV)
        assert rel_err(ops.sigmoid_gate(x.to(DEV), ops.SliceSums(parts, dt), col).cpu(), T64(want)) < 1e-6


GLA_SHAPES = [(2, 16, 24, 8.0), (3, 8, 16, 3.0), (1, 32, 8, 20.0), (2, 12, 12, 1.0), (4, 64, 64, 16.0), (3, 10, 14, 5.0), (4, 128, 128, 16.0),
              (8, 32, 96, 4.0), (2, 48, 256, 2.0), (1, 200, 16, 9.0), (2, 128, 256, 16.0), (3, 128, 8, 1.0), (1, 300, 4, 2.0),
              (2, 192, 192, 4.0), (1, 256, 256, 8.0), (1, 96, 512, 2.0)]       # (the last three: several columns of S a thread)


def _gla_inputs(seed, T, H, d, dv, dt, extra=5):
    """Rows [T, q | k | pad | v | g] of the activation type, the decays' logits in float, their bias and the norm's weight."""
    HD, HV = H * d, H * dv
    rows = rnd(seed, T, 2 * HD + extra + 2 * HV).to(dt)
    rows[:, HD:2 * HD] *= d ** -0.5
    z = rnd(seed + 1, T, HD, scale=1.5).float()
    bias = (torch.rand(HD, generator=torch.Generator().manual_seed(seed + 2)) * 7.0 - 1.0).float()
    w = (rnd(seed + 3, dv, scale=0.3) + 1.0).to(dt)
    return rows, (0, HD, 2 * HD + extra, 2 * HD + extra + HV), z, bias, w


def _gla_plain(rows, cols, z, bias, w, H, d, dv, tau, eps, S0=None):
    x = N64(rows)
    T = x.shape[0]
    q = x[:, cols[0]:cols[0] + H * d].reshape(T, H, d) * d ** -0.5
    k = x[:, cols[1]:cols[1] + H * d].reshape(T, H, d)
    v = x[:, cols[2]:cols[2] + H * dv].reshape(T, H, dv)
    g = x[:, cols[3]:cols[3] + H * dv]
    alpha = (pt.sigmoid(N64(z) + N64(bias)) ** (1.0 / tau)).reshape(T, H, d)
    o, S = pt.gla_recurrence(q, k, v, alpha, S0)
    return pt.rms_norm(o, N64(w), eps).reshape(T, H * dv) * pt.silu(g), S


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,d,dv,tau", GLA_SHAPES)
def test_gated_linear_attention_over_steps_with_state_in_slots(dtype, H, d, dv, tau):
    """Three requests of unequal length fed in unequal portions, single tokens among them, some left out of a step, their
    states in slots of a wider state row: every request's outputs are those of the recurrence over its whole sequence."""
    dt, eps = DT[dtype], 1e-5
    lens_total = [41, 9, 50]
    inputs = [_gla_inputs(10 * i + 1, n, H, d, dv, dt) for i, n in enumerate(lens_total)]
    cols, bias, w = inputs[0][1], inputs[0][3], inputs[0][4]
    offset, n_state = 8, ops.gla_state_floats(H, d, dv)
    state = torch.zeros((5, offset + n_state + 4), dtype=torch.float32, device=DEV)
    slots = torch.tensor([3, 0, 1], dtype=torch.int32)
    got, at = [[] for _ in lens_total], [0, 0, 0]
    for step in ([7, 1, 30], [1, 1, 1], [2, 0, 3], [20, 5, 15], [11, 2, 1]):
        live = [i for i, m in enumerate(step) if m]
        rows = torch.cat([inputs[i][0][at[i]:at[i] + step[i]] for i in live])
        z = torch.cat([inputs[i][2][at[i]:at[i] + step[i]] for i in live])
        q_start, q_len = _step_arrays([step[i] for i in live])
        out = ops.gla_scan(rows.to(DEV), cols, z.to(DEV), bias.to(DEV), tau, d ** -0.5, w.to(DEV), eps, H, d, dv, state, offset,
                           q_start.to(DEV), q_len.to(DEV), slots[live].to(DEV)).cpu()
        o = 0
        for i in live:
            got[i].append(out[o:o + step[i]]); o += step[i]; at[i] += step[i]
    assert at == lens_total
    for i in range(3):
        want, _ = _gla_plain(inputs[i][0], cols, inputs[i][2], bias, w, H, d, dv, tau, eps)
        assert rel_err(torch.cat(got[i]), T64(want)) < (3e-5 if dtype == "float32" else 1.5e-2), i
    s = state.cpu()
    assert not s[[2, 4]].any() and not s[:, :offset].any() and not s[:, offset + n_state:].any()
    # the state holds S itself: its sum of squares is that of the plain recurrence's last S (whatever the layout, padding is zero)
    _, S = _gla_plain(inputs[1][0], cols, inputs[1][2], bias, w, H, d, dv, tau, eps)
    assert abs(float((s[0, offset:offset + n_state].double() ** 2).sum()) / float((S ** 2).sum()) - 1.0) < 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,d,dv,tau,chunk", [(2, 16, 24, 8.0, 64), (3, 8, 16, 3.0, 16), (4, 64, 64, 16.0, 64), (3, 10, 14, 5.0, 7), (2, 128, 128, 16.0, 64),
                                             (1, 32, 8, 20.0, 200), (1, 192, 192, 8.0, 32), (1, 256, 256, 4.0, 64)])
def test_gated_linear_attention_in_chunks_side_by_side(dtype, H, d, dv, tau, chunk):
    """Long portions cut into chunks that first run from zero and then from what the chunks before them leave: the same
    outputs and the same final state as the walk in one piece, for requests of unequal length that start from a state."""
    dt, eps = DT[dtype], 1e-6
    lens = [300, 1, 70, 129]
    T = sum(lens)
    rows, cols, z, bias, w = _gla_inputs(70, T, H, d, dv, dt, extra=0)
    q_start, q_len = _step_arrays(lens)
    slots = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    n_state = ops.gla_state_floats(H, d, dv)
    warm = torch.zeros((4, n_state), dtype=torch.float32, device=DEV)          # a state of the kernel's own making to start from
    r0, _, z0, _, _ = _gla_inputs(80, 12, H, d, dv, dt, extra=0)
    s4, l4 = _step_arrays([3, 3, 3, 3])
    ops.gla_scan(r0.to(DEV), cols, z0.to(DEV), bias.to(DEV), tau, d ** -0.5, w.to(DEV), eps, H, d, dv, warm, 0, s4.to(DEV), l4.to(DEV), slots.to(DEV))
    outs, states = [], []
    for chunks in (None, ops.scan_chunks(q_start.numpy(), q_len.numpy(), chunk, DEV)):
        state = warm.clone()
        outs.append(ops.gla_scan(rows.to(DEV), cols, z.to(DEV), bias.to(DEV), tau, d ** -0.5, w.to(DEV), eps, H, d, dv, state, 0,
                                 q_start.to(DEV), q_len.to(DEV), slots.to(DEV), chunks).cpu())
        states.append(state.cpu())
    assert rel_err(outs[1], outs[0]) < (5e-5 if dtype == "float32" else 1.5e-2)
    assert rel_err(states[1], states[0]) < 5e-5
    assert warm.cpu().abs().max() > 0 and not torch.equal(states[0], warm.cpu())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunked", [False, True])
def test_a_key_far_back_is_still_in_the_state(dtype, chunked):
    """One channel of one head never decays; the key at position 3 is written on it and the query at the last position reads
    it, after hundreds of tokens fed in portions: the head returns that token's value.  A lost or reset state returns noise."""
    dt, eps, H, d, dv, tau, n = DT[dtype], 1e-6, 2, 16, 24, 4.0, 700
    rows, cols, z, bias, w = _gla_inputs(90, n, H, d, dv, dt, extra=0)
    HD = H * d
    ch = d + 5                                   # head 1, channel 5
    z[:, ch], bias[ch] = 40.0, 0.0               # alpha = 1 there, to float's last digit
    rows[:, HD + ch] = 0.0                       # nobody else writes on the channel
    rows[3, HD + ch] = 8.0
    rows[-1, d:2 * d] = 0.0
    rows[-1, ch] = 16.0                          # the last query reads that channel alone (head 1)
    state = torch.zeros((2, ops.gla_state_floats(H, d, dv)), dtype=torch.float32, device=DEV)
    slot = torch.tensor([1], dtype=torch.int32, device=DEV)
    outs, p = [], 0
    for m in [2, 300, 1, 1, 133, 2, 260, 1]:
        q_start, q_len = _step_arrays([m])
        chunks = ops.scan_chunks(q_start.numpy(), q_len.numpy(), 64, DEV) if chunked and m > 64 else None
        outs.append(ops.gla_scan(rows[p:p + m].to(DEV), cols, z[p:p + m].to(DEV), bias.to(DEV), tau, d ** -0.5, w.to(DEV), eps, H, d, dv, state, 0,
                                 q_start.to(DEV), q_len.to(DEV), slot, chunks).cpu())
        p += m
    assert p == n
    want, _ = _gla_plain(rows, cols, z, bias, w, H, d, dv, tau, eps)
    assert rel_err(torch.cat(outs), T64(want)) < (3e-5 if dtype == "float32" else 1.5e-2)
    v3 = N64(rows)[3, cols[2] + dv:cols[2] + 2 * dv]
    o_last = v3 * 8.0 * 16.0 * d ** -0.5
    head1 = pt.rms_norm(o_last, N64(w), eps) * pt.silu(N64(rows)[-1, cols[3] + dv:cols[3] + 2 * dv])
    assert rel_err(torch.cat(outs)[-1, dv:], T64(head1)) < (1e-4 if dtype == "float32" else 1.5e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("S", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("T,H", [(1, 64), (9, 100), (70, 384), (3, 5000), (5, 99), (2, 2050)])
def test_hyper_connections_read_and_update_all_streams_at_once(dtype, S, T, H):
    dt, eps = DT[dtype], 1e-5
    g = torch.Generator().manual_seed(S * 100 + T)
    x0 = rnd(1, T, H).float()
    y1, y2 = rnd(2, T, H, scale=3.0).to(dt), rnd(3, T, H, scale=3.0).to(dt)
    W = {f"{q}.{k}": torch.rand(shape, generator=g) + 0.1 for q in ("a", "b") for k, shape in (("in", (S,)), ("out", (S,)), ("mix", (S, S)))}
    Wn = {k: N64(v) for k, v in W.items()}
    nw = (rnd(4, H, scale=0.3) + 1.0).to(dt)
    dev = lambda k: W[k].to(DEV)
    # the first read: S copies of the one stream, nothing pending
    streams, rows = ops.hyper_step(x0.to(DEV), S, None, None, None, dev("a.in"), nw.to(DEV), eps, dt)
    xs = np.stack([N64(x0)] * S)
    assert torch.equal(streams.cpu(), x0[:, None, :].expand(T, S, H))
    tol = 1e-5 if dtype == "float32" else 6e-3
    assert rel_err(rows.cpu(), T64(pt.rms_norm(np.einsum("s,stw->tw", Wn["a.in"], xs), N64(nw), eps))) < tol
    # the first sub-block's output changes the streams as the second reads them
    streams2, rows = ops.hyper_step(streams, S, y1.to(DEV), dev("a.mix"), dev("a.out"), dev("b.in"), nw.to(DEV), eps, dt)
    assert streams2.data_ptr() == streams.data_ptr()
    xs = pt.hyper_step(xs, {"in": Wn["a.in"], "out": Wn["a.out"], "mix": Wn["a.mix"]}, "", lambda u: N64(y1))
    assert rel_err(streams2.cpu().permute(1, 0, 2), T64(xs)) < 1e-6
    assert rel_err(rows.cpu(), T64(pt.rms_norm(np.einsum("s,stw->tw", Wn["b.in"], xs), N64(nw), eps))) < tol
    # the last update (a product left as partial sums) and the sum of the streams
    parts = torch.stack([y2.float() * 0.25, y2.float() * 0.75]).to(DEV)
    _, total = ops.hyper_step(streams2, S, ops.SliceSums(parts, dt), dev("b.mix"), dev("b.out"), torch.ones(S, device=DEV))
    xs = pt.hyper_step(xs, {"in": Wn["b.in"], "out": Wn["b.out"], "mix": Wn["b.mix"]}, "", lambda u: N64(y2))
    assert total.dtype == torch.float32 and rel_err(total.cpu(), T64(xs.sum(0))) < 1e-6
    if S > 1:       # the matrix is indexed [from, to]: its transpose gives other streams
        wrong = pt.hyper_step(np.stack([N64(x0)] * S) * np.arange(1, S + 1)[:, None, None], {"in": Wn["a.in"], "out": Wn["a.out"], "mix": Wn["a.mix"].T},
                              "", lambda u: N64(y1))
        right = pt.hyper_step(np.stack([N64(x0)] * S) * np.arange(1, S + 1)[:, None, None], {"in": Wn["a.in"], "out": Wn["a.out"], "mix": Wn["a.mix"]},
                              "", lambda u: N64(y1))
        assert np.abs(wrong - right).max() > 1e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M", [1, 7, 16, 40, 300])
@pytest.mark.parametrize("K,ff", [(64, 96), (256, 384), (100, 50)])
def test_feed_forward_without_a_gate(dtype, M, K, ff):
    dt = DT[dtype]
    x, up = rnd(50, M, K).to(dt), rnd(51, ff, K, scale=2.0 * K ** -0.5).to(dt)
    got = ops.linear_act(x.to(DEV), ops.prepare_linear(up.to(DEV)), ops.ACT_GELU_TANH).cpu()
    assert rel_err(got, T64(pt.gelu_tanh(N64(x) @ N64(up).T))) < (1e-5 if dtype == "float32" else 1.5e-2)
    pre = N64(x) @ N64(up).T                                        # a product left as partial sums is added up on the way
    parts = ops.SliceSums(torch.stack([T64(pre * 0.25), T64(pre * 0.5), T64(pre * 0.25)]).float().to(DEV), dt)
    got = ops.activation(parts, ops.ACT_GELU_TANH)
    assert got.dtype == dt and rel_err(got.cpu(), T64(pt.gelu_tanh(pre))) < (1e-5 if dtype == "float32" else 6e-3)
    z = torch.linspace(-6, 6, 4001, dtype=torch.float32)
    assert rel_err(ops.activation(z.to(DEV), ops.ACT_GELU_TANH).cpu(), T64(pt.gelu_tanh(N64(z)))) < 1e-6
    assert rel_err(ops.activation(z.to(DEV), ops.ACT_SILU).cpu(), T64(pt.silu(N64(z)))) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [1, 5, 16, 17, 90])
@pytest.mark.parametrize("E,top,K", [(8, 2, 64), (6, 3, 100), (4, 1, 88), (5, 5, 100), (32, 6, 512), (16, 4, 128)])
def test_router_with_a_bias_and_a_softmax_over_the_chosen(dtype, T, E, top, K):
    dt = DT[dtype]
    h, w = rnd(60, T, K).to(dt), rnd(61, E, K, scale=2.0 * K ** -0.5).to(dt)
    bias = rnd(62, E, scale=1.5).float()
    ids, weights = ops.moe_route(h.to(DEV), w.to(DEV), top, softmax=True, renormalize=True, bias=bias.to(DEV))
    W = {"router": N64(w), "router.b": N64(bias)}
    want_ids, want_w = pt.route(N64(h), W, "", top)
    z = N64(h) @ N64(w).T + N64(bias)
    ids, weights = ids.cpu().long().numpy(), N64(weights)
    for t in range(T):
        order = np.argsort(ids[t])
        zs = np.sort(z[t])[::-1]
        if top < E and zs[top - 1] - zs[top] < 1e-3:        # a close call: either expert may be taken
            continue
        assert sorted(ids[t]) == sorted(want_ids[t]), t
        by_id = dict(zip(want_ids[t], want_w[t]))
        assert np.allclose(weights[t][order], [by_id[e] for e in ids[t][order]], atol=1e-5 if dtype == "float32" else 2e-3), t
    # without its bias the router chooses otherwise: the bias counts
    ids0, _ = ops.moe_route(h.to(DEV), w.to(DEV), top, softmax=True, renormalize=True)
    if top < E and T >= 16:
        assert not np.array_equal(np.sort(ids0.cpu().numpy(), 1), np.sort(ids, 1))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,N", [(1, 64, 64), (9, 100, 100), (70, 512, 512), (300, 88, 88)])
def test_shared_expert_joins_through_a_gate_of_one_number_per_row(dtype, T, K, N):
    dt = DT[dtype]
    base, extra, h = rnd(70, T, N).to(dt), rnd(71, T, N).to(dt), rnd(72, T, K).to(dt)
    gw = rnd(73, K, scale=2.0 * K ** -0.5).to(dt)
    want = N64(base) + pt.sigmoid(N64(h) @ N64(gw))[:, None] * N64(extra)
    got = ops.gated_add(base.to(DEV), extra.to(DEV), h.to(DEV), gw.to(DEV)).cpu()
    assert rel_err(got, T64(want)) < (1e-5 if dtype == "float32" else 6e-3)
    parts = ops.SliceSums(torch.stack([base.float() * 0.5, base.float() * 0.5]).to(DEV), dt)
    eparts = ops.SliceSums(torch.stack([extra.float() * 0.25, extra.float() * 0.75]).to(DEV), dt)
    assert rel_err(ops.gated_add(parts, eparts, h.to(DEV), gw.to(DEV)).cpu(), T64(want)) < (1e-5 if dtype == "float32" else 6e-3)


def test_logits_scaled_and_capped():
    x = rnd(80, 7, 333, scale=20.0).float()
    for scale, cap in ((2.0, 30.0), (1.0, 5.0), (0.5, None), (1.0, None)):
        want = N64(x) * scale
        if cap:
            want = cap * np.tanh(want / cap)
        assert rel_err(ops.scale_softcap(x.clone().to(DEV), scale, cap).cpu(), T64(want)) < 1e-6
    assert float(ops.scale_softcap(x.clone().to(DEV), 2.0, 30.0).abs().max()) <= 30.0


# ---- the model through the engine -----------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(tm.CONFIGS))
def test_whole_prompts(name, dtype, folders):
    folder, vocab = folders[name, dtype], tm.CONFIGS[name]["vocab"]
    runner = load_runner(folder, DT[dtype], num_pages=32, max_requests=2)
    for seed, n in ((1, 1), (2, 2), (3, 37), (4, 200)):
        ids = ids_of(seed, n, vocab)
        assert off(run_whole(runner, "w", ids), plain(folder, ids), dtype) < 1, (name, n)
    runner.manager.check()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_stream_after_every_layer(name, folders):
    folder = folders[name, "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    ids = ids_of(3, 50, tm.CONFIGS[name]["vocab"])
    _, streams = plain(folder, ids, layers=True)
    runner.add_request("p")
    runner.manager.reserve("p", len(ids))
    ctx = StepContext([StepEntry("p", ids, [0])], runner.manager, torch.float32, runner.device)
    model = runner.model
    assert len(model.plan.schedule) == streams.shape[0]
    x, pending = model.embedding.forward(ctx), None
    for i, e in enumerate(model.plan.schedule):
        block = model.blocks[e.layer]
        x, pending = block.forward(x, pending, ctx, runner.storage.binding(i))
        if isinstance(x, blk.HyperStreams):       # the pending update on a copy, then the sum of the streams
            _, after = ops.hyper_step(x.data.clone(), block.streams, pending.y, pending.mix, pending.out, block.ones)
        else:
            after = x + (pending.sum(torch.float32) if hasattr(pending, "parts") else pending.float())
        assert rel_err(after.cpu(), streams[i]) < 1e-5, i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["recurrent_only", "no_windows", "one_of_each_plain"])
def test_models_without_pages_or_without_windows(kind, dtype, tmp_path):
    """A model of recurrences alone keeps no pages at all; attention without a window keeps everything; one stream without
    connections, no cap, no loop."""
    layers = {
        "recurrent_only": [tm.layer(tm.gla(2, 16, 16, 4.0, 4), tm.dense(40)), tm.layer(tm.gla(1, 24, 40, 9.0, 3), None)],
        "no_windows": [tm.layer(tm.attention(4, 1, 16, 16, 0.5, 10000.0, 16), tm.moe(4, 2, 24, shared=16)),
                       tm.layer(tm.attention(2, 2, 32, 16, 0.4, 500.0, 8), tm.dense(24))],
        "one_of_each_plain": [tm.layer(tm.attention(4, 4, 64, 64, 0.2, 5e5, 32, window=70, scaling=(8.0, 1.0, 4.0, 2048)), tm.dense(64)),
                              tm.layer(tm.gla(2, 32, 32, 16.0, 8), tm.moe(8, 8, 16))],
    }[kind]
    cfg = tm.model(150, 64, 1e-5, layers, emb_scale=0.5, streams=None if kind == "one_of_each_plain" else 2,
                   loop=(0, 2, 2) if kind == "recurrent_only" else None)
    folder = tm.write_model(str(tmp_path / "m"), cfg, 9, gain=GAIN[dtype], decisive_router=dtype == "bfloat16")
    runner = load_runner(folder, DT[dtype], num_pages=20, max_requests=3)
    assert len(runner.manager.groups) == {"recurrent_only": 0, "no_windows": 1, "one_of_each_plain": 1}[kind]
    ids = ids_of(8, 230, 150)
    want = plain(folder, ids)
    assert off(run_whole(runner, "w", ids), want, dtype) < 1
    runner.add_request("c")
    runner.add_request("o")
    rows, p = [], 0
    for m in [2, 100, 1, 1, 64, 3, 1, 58]:
        rows.append(runner.step([StepEntry("o", ids_of(p, 2, 150), []), StepEntry("c", ids[p:p + m], list(range(m)))]).cpu())
        p += m
    assert p == len(ids) and off(torch.cat(rows), want, dtype) < 1
    runner.manager.check()


def test_first_tokens(folders):
    """Position 0 sees itself alone and a zero state: its logits are a function of the token."""
    folder = folders["D", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    for tok in (0, 77, 98):
        a, b = run_whole(runner, "x", [tok]), run_whole(runner, "y", [tok, 5, 9, 2])
        assert rel_err(a, plain(folder, [tok])) < TOL["float32"] and torch.equal(a[0], b[0])
        assert rel_err(b, plain(folder, [tok, 5, 9, 2])) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(tm.CONFIGS))
def test_prefill_against_decoding_and_portions(name, dtype, folders):
    folder, vocab = folders[name, dtype], tm.CONFIGS[name]["vocab"]
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
        assert off(got, want, dtype) < 1
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_run_in_chunks_and_carry_on(dtype, folders):
    """Portions long enough that the recurrence is cut into chunks running side by side, beside a request that decodes."""
    folder = folders["C", dtype]
    runner = load_runner(folder, DT[dtype], num_pages=64, max_requests=3)
    ids, other = ids_of(33, 700, 512), ids_of(34, 40, 512)
    want, want_o = plain(folder, ids), plain(folder, other)
    runner.add_request("a")
    runner.add_request("o")
    got, got_o, p = [], [], 0
    for i, m in enumerate([300, 1, 129, 2, 268]):
        out = runner.step([StepEntry("o", other[i * 8:i * 8 + 8] if i == 0 else [other[7 + i]], [0]), StepEntry("a", ids[p:p + m], list(range(m)))]).cpu()
        got_o.append(out[0]); got.append(out[1:]); p += m
    assert p == len(ids) and off(torch.cat(got), want, dtype) < 1
    assert off(torch.stack(got_o), want_o[[0, 8, 9, 10, 11]], dtype, [0, 8, 9, 10, 11]) < 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_unequal_requests_in_one_batch_against_each_alone(name, dtype, folders):
    folder, vocab = folders[name, dtype], tm.CONFIGS[name]["vocab"]
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
        assert off(torch.cat(got[r]), plain(folder, ids), dtype) < 1, r
        if dtype == "float32":      # in 32-bit a row's arithmetic depends neither on the cutting nor on its neighbours, beyond rounding
            runner.free_request(r)
            assert rel_err(torch.cat(got[r]), run_whole(runner, r + "'", ids)) < 2e-6, r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_gives_pages_back_and_keeps_its_state(dtype, folders):
    folder = folders["A", dtype]
    runner = load_runner(folder, DT[dtype], num_pages=30, max_requests=2)
    ids = ids_of(51, 420, 300)
    want = plain(folder, ids)
    runner.add_request("d")
    got = [runner.step([StepEntry("d", ids[:9], [8])]).cpu()[0]]
    for p in range(9, len(ids)):
        got.append(runner.step([StepEntry("d", [ids[p]], [0])]).cpu()[0])
    assert off(torch.stack(got), want[8:], dtype, range(8, len(ids))) < 1
    runner.manager.check()
    assert [g.window for g in runner.manager.groups] == [20, 33]
    held = [sum(1 for p in runner.manager.block_table("d", g) if p >= 0) for g in range(2)]
    assert held[0] <= 20 // 16 + 2 and held[1] <= 33 // 16 + 2
    assert runner.graph_replays > 0          # decode steps of a model with state of its own are replayed graphs too


def test_a_freed_slot_starts_from_zero_state(folders):
    """The same prompt gives the same logits in a slot and pages that another request has just used."""
    folder = folders["B", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=6, max_requests=1)
    a, b = ids_of(52, 80, 131), ids_of(53, 61, 131)
    first = run_whole(runner, "a", a)
    run_whole(runner, "b", b)
    assert torch.equal(run_whole(runner, "a2", a), first)
    folder = folders["A", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=12, max_requests=2)
    a, b = ids_of(54, 80, 300), ids_of(55, 61, 300)
    first = run_whole(runner, "a", a)
    runner.add_request("b")
    runner.step([StepEntry("b", b, [])])
    runner.add_request("a2")
    out = runner.step([StepEntry("a2", a, list(range(len(a))))]).cpu()
    runner.free_request("b")
    assert rel_err(out, first) < 2e-6 and rel_err(run_whole(runner, "a3", a), first) < 2e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(tm.CONFIGS))
def test_replay_of_traces_with_pages_and_slots_used_again(name, dtype, folders, tmp_path):
    """Through bin/trace_run as a user would: whole, prefill then decode, portions, and mixed steps of up to four live
    requests, one process, a pool so small that pages and slots are used again."""
    folder, vocab = folders[name, dtype], tm.CONFIGS[name]["vocab"]
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
        assert off(got, want, dtype, [p for _, p in rows]) < 1, (step, rows[:3])


def _drawn_config(seed):
    """A configuration drawn from sizes of every kind: heads the matrix-core kernels take and heads only the plain kernel
    takes, grouped and ungrouped, values wider and narrower than keys, windows around a page's size, recurrences of few and
    many channels, both feed-forwards, layers in any order with and without feed-forward, streams, loops."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 72, 96, 160])
    layers = []
    for _ in range(rng.choice([1, 2, 3, 4])):
        if rng.random() < 0.5:
            mixer = tm.gla(rng.choice([1, 2, 3, 4]), rng.choice([8, 10, 16, 32, 48, 64, 128]), rng.choice([8, 14, 16, 32, 64, 128]),
                           rng.choice([1.0, 4.0, 16.0]), rng.choice([1, 4, 10, 16]))
        else:
            kv = rng.choice([1, 2, 3])
            dim, vdim = rng.choice([8, 12, 16, 32, 48, 64, 96, 128]), rng.choice([8, 10, 16, 32, 64])
            if rng.random() < 0.5:
                vdim = dim
            dims = rng.choice([dim, max(2, dim // 2 // 2 * 2), 2])
            mixer = tm.attention(kv * rng.choice([1, 2, 4]), kv, dim, vdim, rng.choice([1.0, 2.0, 4.0]) / dim ** 0.5 * 2.0, rng.choice([100.0, 10000.0, 1e6]),
                                 dims, rng.choice([None, 1, 5, 16, 17, 64, 100]), rng.choice([None, (4.0, 1.0, 4.0, 64), (8.0, 1.0, 4.0, 8192), (2.0, 0.5, 2.0, 16)]))
        mlp = rng.choice([None, tm.dense(56), tm.dense(24), tm.moe(4, 2, 24), tm.moe(8, 3, 16, shared=24), tm.moe(3, 1, 40, shared=8), tm.moe(2, 2, 8)])
        layers.append(tm.layer(mixer, mlp))
    n = len(layers)
    loop = None
    if rng.random() < 0.5:
        start = rng.randrange(n)
        loop = (start, rng.randrange(start + 1, n + 1), rng.choice([1, 2, 3]))
    return tm.model(rng.choice([61, 128, 500]), width, rng.choice([1e-5, 1e-6, 1e-3]), layers, emb_scale=rng.choice([1.0, 0.5, 3.0]),
                    streams=rng.choice([None, 1, 2, 4, 6]), logit_scale=rng.choice([1.0, 0.5, 2.0]), softcap=rng.choice([None, 10.0, 30.0]), loop=loop)


@pytest.mark.parametrize("seed", range(14))
def test_drawn_configurations(seed, tmp_path):
    """Whole prompts, portions and decoding of drawn configurations against the plain implementation, both precisions."""
    cfg = _drawn_config(seed)
    for dtype in ("float32", "bfloat16"):
        folder = tm.write_model(str(tmp_path / dtype), cfg, 80 + seed, gain=GAIN[dtype], decisive_router=dtype == "bfloat16")
        runner = load_runner(folder, DT[dtype], num_pages=24, max_requests=3)
        ids = ids_of(seed, 150, cfg["vocab"])
        want = plain(folder, ids)
        assert off(run_whole(runner, "w", ids), want, dtype) < 1, (seed, dtype, cfg)
        runner.add_request("c")
        runner.add_request("other")
        rows, p = [], 0
        for m in [33, 2, 64, 1, 1, 17, 1, 1, 1, 29]:
            out = runner.step([StepEntry("other", ids_of(p, 3, cfg["vocab"]), []), StepEntry("c", ids[p:p + m], list(range(m)))]).cpu()
            rows.append(out)
            p += m
        assert p == len(ids) and off(torch.cat(rows), want, dtype) < 1, (seed, dtype, cfg)
        runner.manager.check()


# ---- generation through the engine's own entry point and scheduler ------------------------------
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_engine(name, folders):
    folder, vocab = folders[name, "float32"], tm.CONFIGS[name]["vocab"]
    cfg, W = tm.load_plain(folder)
    prompts = [ids_of(70 + i, n, vocab) for i, n in enumerate([5, 40, 1, 77, 19, 130])]
    want = [pt.greedy_generate(cfg, W, p, 10) for p in prompts]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32, prefill_tokens_alone=48)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert [o.token_ids for o in outs] == want
    assert engine.runner.graph_replays > 0                       # decode steps ran as replayed graphs
    folder = folders[name, "bfloat16"]
    cfg, W = tm.load_plain(folder)
    engine = Engine.load(folder, dtype="bfloat16", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for p, o in zip(prompts, outs):        # bfloat16 may pick another token where two logits nearly tie
        full = pt.forward(cfg, W, p + o.token_ids)
        for i, tok in enumerate(o.token_ids):
            row = full[len(p) - 1 + i]
            assert row[tok] >= row.max() - 0.06 * np.abs(row).max(), (name, i)


def test_completion_from_the_command_line(folders, capsys):
    from inferflux_amd import cli
    folder = folders["B", "float32"]
    cfg, W = tm.load_plain(folder)
    prompt = ids_of(90, 21, 131)
    assert cli.main(["completion", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "7", "--temperature", "0",
                     "--ignore-eos", "--dtype", "float32", "--kv-pages", "32", "--max-parallel-sequences", "2"]) == 0
    said = capsys.readouterr().out
    want = pt.greedy_generate(cfg, W, prompt, 7)
    assert str(want)[1:-1].replace(" ", "") in said.replace(" ", ""), (want, said)
