"""The Vavadra design on the GPU: every mechanism's kernel alone against the plain implementation's function, then the
model through the engine's step function, its replay tool and its generation loop, under every way of cutting and
batching, in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_vavadra as pv
import traces
import vavadra_models as vm
from conftest import ROOT, rel_err

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd import SamplingParams
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepContext, StepEntry
    from inferflux_amd.engine.engine import Engine
    from inferflux_amd.kernels import ops

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# Largest difference of a logit from the plain model's, relative to the largest logit.  32-bit: rounding over a few hundred
# operations.  bfloat16: the worst seen over these tests and half as much again; a key, a block's or a window's edge, a
# state, a sink or a pass's input that is wrong moves a row by 10-100 %.  The rows of a sequence's first positions get more
# in bfloat16: a recurrent head's output is normed, so while its state holds one or a few outer products the output's
# direction hangs on single q . k products, which rounding q and k moves by a large fraction where they happen to be small.
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
TOL_FIRST = {"float32": 2e-5, "bfloat16": 1.6e-1}
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
    """(configuration, precision) -> model folder.  The 32-bit runs take routers with random weights and corrections that
    change the choice; the bfloat16 runs take models in which no choice of experts is a close call (``write_model``)."""
    out = {}
    for i, n in enumerate(vm.CONFIGS):
        for dtype in DT:
            out[n, dtype] = vm.write_model(str(tmp_path_factory.mktemp(f"vavadra{n}{dtype}")), vm.config(n), 40 + i, gain=GAIN[dtype],
                                           decisive_router=dtype == "bfloat16")
    return out


_PLAIN = {}


def plain(folder, ids, layers=False):
    if folder not in _PLAIN:
        _PLAIN[folder] = vm.load_plain(folder)
    key = (folder, tuple(ids), layers)
    if key not in _PLAIN:
        out = pv.forward(*_PLAIN[folder], list(ids), return_layers=layers)
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


def _paged(k, v, dt, P=16, seed=5):
    """k [n, G, kd], v [n, G, dv] of one sequence in pages that lie anywhere in a pool: (K, V, block table [1, pages])."""
    n, G, kd = k.shape
    dv = v.shape[2]
    pages = -(-n // P)
    pool = pages + 3
    where = torch.randperm(pool, generator=torch.Generator().manual_seed(seed))[:pages]
    K = torch.zeros(pool, G, P, kd, dtype=dt)
    V = torch.zeros(pool, G, dv, P, dtype=dt)
    for j in range(n):
        K[where[j // P], :, j % P] = k[j].to(dt)
        V[where[j // P], :, :, j % P] = v[j].to(dt)
    return K.to(DEV), V.to(DEV), where.to(torch.int32)[None].contiguous().to(DEV)


# ---- each mechanism's kernel alone ------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,chunk,nH,nKV,d,dv", [(70, 24, 4, 2, 8, 24), (200, 64, 2, 1, 32, 64), (130, 17, 3, 3, 12, 12), (97, 96, 8, 2, 64, 64),
                                                 (50, None, 2, 2, 10, 14), (300, 128, 4, 1, 48, 96)])
def test_differential_attention_sees_exactly_its_block(dtype, n, chunk, nH, nKV, d, dv):
    """Two maps over the same values, blocks counted from position 0.  A block's first rows are aimed at the key just outside
    the block and at the key just inside it, so that a block one token off changes such a row altogether."""
    dt = DT[dtype]
    lam, diff, eps, scale = 0.37, 0.3, 1e-5, 1.0 / d ** 0.5
    q, k, v = rnd(1, n, nH, 2, d).to(dt).double(), rnd(2, n, nKV, 2, d).to(dt).double(), rnd(3, n, nKV, dv).to(dt).double()
    for i in range(n):
        lo = 0 if chunk is None else i - i % chunk
        for h in range(nH):
            g = h // (nH // nKV)
            if i == lo and lo > 0:
                q[i, h, 0] = (6.0 * k[lo - 1, g, 0]).to(dt).double()             # map 1 of a block's first row: the last key of the block before
            elif i == lo + 1 and lo > 0:
                q[i, h, 1] = (6.0 * k[lo - 1, g, 1]).to(dt).double()             # map 2 of its second row: the same key
            elif i == lo + 2:
                q[i, h, 0] = (6.0 * k[lo, g, 0]).to(dt).double()                 # map 1 of its third row: the block's first key
    K, V, table = _paged(k.reshape(n, nKV, 2 * d), v, dt)
    rows = torch.arange(n, dtype=torch.int32, device=DEV)
    got = ops.attention_plain(q.reshape(n, nH, 2 * d).to(dt).to(DEV), K, V, torch.zeros(n, dtype=torch.int32, device=DEV), rows, table, None,
                              scale, chunk=chunk, differential=(lam, 1.0 - diff, eps)).cpu()
    mask = pv.chunk_mask(n, chunk)
    want = np.zeros((n, nH, dv))
    for h in range(nH):
        g = h // (nH // nKV)
        a = [pv.masked_softmax(N64(q[:, h, c]) @ N64(k[:, g, c]).T * scale, mask) @ N64(v[:, g]) for c in (0, 1)]
        want[:, h] = pv.rms_norm(a[0] - lam * a[1], None, eps) * (1.0 - diff)
    assert rel_err(got, T64(want.reshape(n, nH * dv))) < (2e-5 if dtype == "float32" else 2e-2)
    if chunk is not None:      # a block one token longer or shorter is another function
        for wrong in (chunk + 1, chunk - 1):
            other = ops.attention_plain(q.reshape(n, nH, 2 * d).to(dt).to(DEV), K, V, torch.zeros(n, dtype=torch.int32, device=DEV), rows,
                                        table, None, scale, chunk=wrong, differential=(lam, 1.0 - diff, eps)).cpu()
            assert rel_err(other, T64(want.reshape(n, nH * dv))) > 0.1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,window,nH,d,dv", [(90, 20, 4, 40, 32), (260, 96, 3, 144, 128), (40, None, 2, 24, 24), (150, 33, 5, 18, 14)])
def test_a_sink_per_head_joins_the_denominator(dtype, n, window, nH, d, dv):
    """One shared kv head (as attention through a latent has), a sliding window, and a score per head that takes part in the
    softmax's sum alone; queries aimed at the window's last key and at the first key outside it."""
    dt = DT[dtype]
    scale = 1.0 / d ** 0.5
    q, k, v = rnd(1, n, nH, d).to(dt).double(), rnd(2, n, 1, d).to(dt).double(), rnd(3, n, 1, dv).to(dt).double()
    sinks = torch.tensor([2.5, -1.0, 0.0, 4.0, -6.0][:nH], dtype=torch.float32)
    for i in range(n):
        lo = 0 if window is None else max(0, i - window + 1)
        for h in range(nH):
            if i % 3 == h % 3:
                q[i, h] = (5.0 * k[lo, 0] if (i + h) % 2 or lo == 0 else 5.0 * k[lo - 1, 0]).to(dt).double()
    K, V, table = _paged(k, v, dt)
    rows = torch.arange(n, dtype=torch.int32, device=DEV)
    zero = torch.zeros(n, dtype=torch.int32, device=DEV)
    got = ops.attention_plain(q.to(dt).to(DEV), K, V, zero, rows, table, window, scale, sinks=sinks.to(DEV)).cpu()
    mask = pv.window_mask(n, window)
    want = np.stack([pv.masked_softmax(N64(q[:, h]) @ N64(k[:, 0]).T * scale, mask, sink=float(sinks[h])) @ N64(v[:, 0]) for h in range(nH)], axis=1)
    assert rel_err(got, T64(want.reshape(n, nH * dv))) < (2e-5 if dtype == "float32" else 2e-2)
    without = ops.attention_plain(q.to(dt).to(DEV), K, V, zero, rows, table, window, scale).cpu()
    assert rel_err(without, T64(want.reshape(n, nH * dv))) > 0.05


def _delta_inputs(seed, T, H, G, d, dv, dt):
    u = rnd(seed, T, 2 * G * d + H * dv).to(dt)
    rows = torch.cat([rnd(seed + 1, T, 3), rnd(seed + 2, T, H * dv), rnd(seed + 3, T, 2 * H, scale=1.5)], dim=1).to(dt)   # 3 columns of something else first
    return u, rows, (3, 3 + H * dv, 3 + H * dv + H)


def _delta_plain(u, rows, cols, A_log, dt_bias, norm_w, eps, H, G, d, dv):
    u, rows = N64(u), N64(rows)
    T = u.shape[0]
    q, k = pv.unit(u[:, :G * d].reshape(T, G, d)) * d ** -0.5, pv.unit(u[:, G * d:2 * G * d].reshape(T, G, d))
    v = u[:, 2 * G * d:].reshape(T, H, dv)
    gate = pv.silu(rows[:, cols[0]:cols[0] + H * dv]).reshape(T, H, dv)
    beta = pv.sigmoid(rows[:, cols[1]:cols[1] + H])
    decay = np.exp(-np.exp(N64(A_log)) * pv.softplus(rows[:, cols[2]:cols[2] + H] + N64(dt_bias)))
    out = np.stack([pv.delta_recurrence(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h], decay[:, h]) for h in range(H)], axis=1)
    return (pv.rms_norm(out, N64(norm_w), eps) * gate).reshape(T, H * dv)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,d,dv", [(4, 2, 16, 24), (2, 2, 12, 12), (3, 1, 10, 14), (4, 4, 64, 64), (2, 1, 128, 128), (1, 1, 256, 64), (2, 2, 40, 512),
                                      (8, 8, 32, 96)])
def test_delta_rule_over_steps_with_state_in_slots(dtype, H, G, d, dv):
    """Three requests whose rows come in steps of unequal portions, their states in slots that lie anywhere behind a stretch
    of the row that belongs to somebody else, against each request's recurrence in one piece."""
    dt = DT[dtype]
    eps, lens = 1e-5, {"a": 45, "b": 9, "c": 23}
    A_log, dt_bias = (-3.0 + 3.5 * torch.rand(H, generator=torch.Generator().manual_seed(8))).float(), rnd(9, H).float()
    norm_w = (1.0 + 0.3 * rnd(10, dv)).to(dt)
    data = {r: _delta_inputs(20 + 10 * i, n, H, G, d, dv, dt) for i, (r, n) in enumerate(lens.items())}
    want = {r: _delta_plain(u, rows, cols, A_log, dt_bias, norm_w, eps, H, G, d, dv) for r, (u, rows, cols) in data.items()}
    offset = 37
    state = torch.zeros(6, offset + ops.delta_state_floats(H, d, dv), dtype=torch.float32, device=DEV)
    slot = {"a": 4, "b": 0, "c": 2}
    at, got = {r: 0 for r in lens}, {r: [] for r in lens}
    for step in [{"a": 20, "b": 1, "c": 2}, {"c": 16, "a": 1}, {"b": 8, "a": 9, "c": 1}, {"a": 15, "c": 4}]:
        us = torch.cat([data[r][0][at[r]:at[r] + m] for r, m in step.items()])
        rs = torch.cat([data[r][1][at[r]:at[r] + m] for r, m in step.items()])
        q_start, q_len = _step_arrays(list(step.values()))
        slots = torch.tensor([slot[r] for r in step], dtype=torch.int32)
        out = ops.delta_rule(us.to(DEV), rs.to(DEV), data["a"][2], A_log.to(DEV), dt_bias.to(DEV), norm_w.to(DEV), eps, H, G, d, dv, state,
                             offset, q_start.to(DEV), q_len.to(DEV), slots.to(DEV)).cpu()
        o = 0
        for r, m in step.items():
            got[r].append(out[o:o + m]); o += m; at[r] += m
    assert float(state[:, :offset].abs().max()) == 0 and float(state[[1, 3, 5]].abs().max()) == 0     # nobody else's floats were touched
    for r in lens:
        assert at[r] == lens[r]
        assert rel_err(torch.cat(got[r]), T64(want[r])) < (2e-5 if dtype == "float32" else 3e-2), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_is_still_in_the_state(dtype):
    """A head that hardly decays is written once along a key that no later token comes near, and asked for it 700 tokens
    later, decoded one by one at the end: the read-out is the value written then."""
    dt, H, G, d, dv, T = DT[dtype], 2, 1, 32, 16, 720
    u, rows, cols = _delta_inputs(3, T, H, G, d, dv, dt)
    u, rows = u.double(), rows.double()
    u[:, :2 * G * d][:, 0] = 0.0                       # channel 0 of q and of k belongs to the far key alone
    u[:, G * d] = 0.0
    u[0, G * d:2 * G * d] = 0.0
    u[0, G * d] = 3.0                                  # the key at token 0: channel 0
    u[T - 5:, :G * d] = 0.0
    u[T - 5:, 0] = 2.0                                 # the last five queries ask for channel 0
    rows[:, cols[1]:cols[1] + H] = 0.0
    rows[0, cols[1]:cols[1] + H] = 30.0                # beta 1 at the write
    u, rows = u.to(dt), rows.to(dt)
    A_log, dt_bias = torch.tensor([-14.0, 0.5]), torch.tensor([0.0, 0.0])    # head 0 keeps, head 1 forgets
    norm_w = torch.ones(dv, dtype=dt)
    want = _delta_plain(u, rows, cols, A_log, dt_bias, norm_w, 1e-6, H, G, d, dv)
    state = torch.zeros(2, ops.delta_state_floats(H, d, dv), dtype=torch.float32, device=DEV)
    got, p = [], 0
    for m in [300, 415, 1, 1, 1, 1, 1]:
        q_start, q_len = _step_arrays([m])
        got.append(ops.delta_rule(u[p:p + m].to(DEV), rows[p:p + m].to(DEV), cols, A_log.to(DEV), dt_bias.to(DEV), norm_w.to(DEV), 1e-6, H, G,
                                  d, dv, state, 0, q_start.to(DEV), q_len.to(DEV), torch.tensor([1], dtype=torch.int32, device=DEV)).cpu())
        p += m
    got = torch.cat(got)
    assert rel_err(got[T - 5:], T64(want[T - 5:])) < (2e-5 if dtype == "float32" else 3e-2)
    # what head 0 reads at the end points along the value written at token 0 (before the gate): undo the gate and compare directions
    gate = pv.silu(N64(rows)[T - 1, cols[0]:cols[0] + dv])
    read = N64(got)[T - 1, :dv] / gate
    v0 = N64(u)[0, 2 * G * d:2 * G * d + dv]
    assert float(read @ v0 / np.linalg.norm(read) / np.linalg.norm(v0)) > 0.999


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,E,I,top,K,ff", [(5, 6, 2, 2, 64, 24), (70, 12, 4, 2, 192, 64), (33, 3, 2, 5, 100, 22), (90, 8, 8, 3, 128, 32), (9, 4, 0, 1, 88, 40),
                                            (200, 30, 2, 6, 256, 128)])
def test_experts_with_identity_experts_a_correction_and_clamps(dtype, T, E, I, top, K, ff):
    """The router's softmax over experts and identity experts, the choice by score + correction, the weights by the score, the
    clamped activation, and rows handed back by identity experts: by the row kernels and, in bfloat16, by the grouped
    products on the matrix cores as well."""
    dt = DT[dtype]
    limit, scale = 0.8, 1.7
    p = "m"
    W = {f"{p}.router": rnd(1, E + I, K, scale=2.0 / K ** 0.5).to(dt).double(), f"{p}.correction": rnd(2, E + I, scale=0.2).float().double()}
    for e in range(E):
        W[f"{p}.e{e}.gate"], W[f"{p}.e{e}.up"] = rnd(10 + e, ff, K, scale=2.0 / K ** 0.5).to(dt).double(), rnd(50 + e, ff, K, scale=2.0 / K ** 0.5).to(dt).double()
        W[f"{p}.e{e}.down"] = rnd(90 + e, K, ff, scale=1.0 / ff ** 0.5).to(dt).double()
    h = rnd(3, T, K).to(dt)
    m = {"expert": {"ff": ff, "limit": limit}, "router": {"experts": E, "identity": I, "top": top, "scale": scale}}
    Wn = {k: N64(v) for k, v in W.items()}
    want_ids, want_w = pv.route(N64(h), Wn, p, m["router"])
    ids, weights = ops.moe_route(h.to(DEV), W[f"{p}.router"].to(dt).to(DEV), top, softmax=True, renormalize=False, scale=scale,
                                 choice_bias=W[f"{p}.correction"].float().to(DEV))
    if dtype == "float32":
        assert np.array_equal(ids.cpu().numpy(), want_ids) and rel_err(weights.cpu(), T64(want_w)) < 1e-5
        if T >= 33 and top < E + I:          # (the correction does change some row's choice: without it the ids differ somewhere)
            no_bias, _ = ops.moe_route(h.to(DEV), W[f"{p}.router"].to(dt).to(DEV), top, softmax=True, scale=scale)
            assert not np.array_equal(no_bias.cpu().numpy(), want_ids)
    # the experts' sums for the plain model's choices (so that a close call of the router's says nothing here)
    ids_t, w_t = torch.from_numpy(want_ids.astype(np.int32)).to(DEV), torch.from_numpy(want_w).float().to(DEV)
    want = np.zeros((T, K))
    for t in range(T):
        for e, w in zip(want_ids[t], want_w[t]):
            want[t] += w * (N64(h)[t] if e >= E else pv.clamped_expert(N64(h)[t:t + 1], Wn, f"{p}.e{e}", limit)[0])
    stack = lambda k: torch.stack([W[f"{p}.e{e}.{k}"].to(dt) for e in range(E)]).contiguous().to(DEV)
    gate, up, down = stack("gate"), stack("up"), stack("down")
    got = ops.moe_experts(h.to(DEV), gate, up, down, ids_t, w_t, ops.ACT_CLAMPED_SWISH, limit, I).cpu()
    assert rel_err(got, T64(want)) < (2e-5 if dtype == "float32" else 2e-2)
    assert I == 0 or (want_ids >= E).any()
    if dtype == "bfloat16" and ops.grouped_takes(dt, K, ff):
        parts = ops.moe_experts_grouped(h.to(DEV), ops.pair_gate_up(gate, up), down, ids_t, w_t, ops.ACT_CLAMPED_SWISH, limit, I)
        assert rel_err(parts.sum(torch.float32).cpu(), T64(want)) < 2e-2
        paired = ops.moe_experts(h.to(DEV), ops.pair_gate_up(gate, up), None, down, ids_t, w_t, ops.ACT_CLAMPED_SWISH, limit, I).cpu()
        assert rel_err(paired, T64(want)) < 2e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,I,limit", [(3, 40, 1.0), (70, 128, 2.0), (9, 22, 0.5)])
def test_clamped_activation_beyond_both_limits(dtype, T, I, limit):
    dt = DT[dtype]
    gu = rnd(1, T, 2 * I, scale=2.0).to(dt)            # many values beyond the limit on either side
    g, u = N64(gu)[:, 0::2], N64(gu)[:, 1::2]
    gc = np.minimum(g, limit)
    want = gc * pv.sigmoid(1.702 * gc) * (np.clip(u, -limit, limit) + 1.0)
    got = ops.swiglu(gu.to(DEV), interleaved=True, act=ops.ACT_CLAMPED_SWISH, limit=limit).cpu()
    assert rel_err(got, T64(want)) < (1e-6 if dtype == "float32" else 1e-2)
    assert (np.abs(u) > limit).any() and (g > limit).any() and (g < -limit).any()      # (negative gates are not clamped)


def test_a_pass_input_is_added_to_the_stream_in_place():
    x, rows = rnd(1, 37, 100).float(), rnd(2, 37, 100).float()
    for dt in (torch.float32, torch.bfloat16):
        vec = rnd(3, 100).to(dt)
        for r, v in ((rows, vec), (None, vec), (rows, None)):
            got = ops.stream_add(x.clone().to(DEV), None if r is None else r.to(DEV), None if v is None else v.to(DEV)).cpu()
            want = x.double() + (0 if r is None else r.double()) + (0 if v is None else v.double())
            assert rel_err(got, want) < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_maps_as_heads_of_their_own_and_joined_again(dtype):
    dt, T, H, d, dv = DT[dtype], 37, 3, 16, 32
    q = rnd(1, T, H, 2 * d).to(dt)
    wide = ops.diff_expand(q.to(DEV)).cpu()
    assert wide.shape == (T, 2 * H, 2 * d)
    assert torch.equal(wide[:, 0::2, :d], q[:, :, :d]) and torch.equal(wide[:, 1::2, d:], q[:, :, d:])
    assert float(wide[:, 0::2, d:].abs().max()) == 0 and float(wide[:, 1::2, :d].abs().max()) == 0
    a = rnd(2, T, 2 * H * dv).to(dt)
    lam, scale, eps = 0.63, 0.7, 1e-5
    pairs = N64(a).reshape(T, H, 2, dv)
    want = pv.rms_norm(pairs[:, :, 0] - lam * pairs[:, :, 1], None, eps) * scale
    got = ops.diff_combine(a.to(DEV), H, dv, lam, scale, eps).cpu()
    assert rel_err(got, T64(want.reshape(T, H * dv))) < (1e-6 if dtype == "float32" else 1e-2)


# ---- the model through the engine -----------------------------------------------------------------
@pytest.mark.parametrize("chunk", [17, 48, 100, 64, None])
def test_blocks_and_two_maps_on_the_matrix_cores(chunk, tmp_path):
    """Differential attention whose values are as wide as both maps' keys together runs on the matrix-core kernels in bfloat16:
    blocks whose edges lie inside the kernels' tiles of keys and of rows, in a prompt, in portions and token by token."""
    cfg = vm.model(200, 64, 1e-5, [vm.layer(vm.differential(4, 2, 32, 64, 0.2, 0.4, chunk=chunk), None),
                                   vm.layer(vm.differential(2, 2, 8, 16, 0.4, 0.7, chunk=chunk), vm.moe(4, 1, 2, 16, 2.0))], emb_scale=2.0)
    folder = vm.write_model(str(tmp_path / "m"), cfg, 3, gain=1.5, decisive_router=True)
    runner = load_runner(folder, torch.bfloat16, num_pages=40, max_requests=3)
    ids = ids_of(5, 330, 200)
    want = plain(folder, ids)
    assert off(run_whole(runner, "w", ids), want, "bfloat16") < 1
    runner.add_request("c")
    rows, p = [], 0
    for m in [100, 1, 1, 63, 2, 17, 1, 1, 1, 1, 130, 2, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1]:
        rows.append(runner.step([StepEntry("c", ids[p:p + m], list(range(m)))]).cpu())
        p += m
    assert p == len(ids) and off(torch.cat(rows), want, "bfloat16") < 1
    runner.manager.check()



@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(vm.CONFIGS))
def test_whole_prompts(name, dtype, folders):
    folder, vocab = folders[name, dtype], vm.CONFIGS[name]["vocab"]
    runner = load_runner(folder, DT[dtype], num_pages=32, max_requests=2)
    for seed, n in ((1, 1), (2, 2), (3, 37), (4, 200)):
        ids = ids_of(seed, n, vocab)
        assert off(run_whole(runner, "w", ids), plain(folder, ids), dtype) < 1, (name, n)
    runner.manager.check()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_stream_after_every_layer(name, folders):
    folder = folders[name, "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    ids = ids_of(3, 50, vm.CONFIGS[name]["vocab"])
    _, streams = plain(folder, ids, layers=True)
    runner.add_request("p")
    runner.manager.reserve("p", len(ids))
    ctx = StepContext([StepEntry("p", ids, [0])], runner.manager, torch.float32, runner.device)
    model = runner.model
    assert len(model.plan.schedule) == streams.shape[0]
    x, pending = model.embedding.forward(ctx), None
    embedded = x.clone()
    for i, e in enumerate(model.plan.schedule):
        if e.before is not None:
            model.injections[e.before].forward(x, ctx, embedded)
        x, pending = model.blocks[e.layer].forward(x, pending, ctx, runner.storage.binding(i))
        after = x + (pending.sum(torch.float32) if hasattr(pending, "parts") else pending.float())
        assert rel_err(after.cpu(), streams[i]) < 1e-5, i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["recurrent_only", "no_masks", "taps_from_the_tensors"])
def test_models_without_pages_without_masks_and_with_open_sizes(kind, dtype, tmp_path):
    """A model of recurrences alone keeps no pages at all; attention without a block size or a window keeps everything; a
    config that leaves the taps to the tensors' shapes."""
    layers = {
        "recurrent_only": [vm.layer(vm.delta(2, 1, 16, 16, 3), vm.moe(4, 1, 2, 24, 1.0)), vm.layer(vm.delta(1, 1, 24, 40, 4), None)],
        "no_masks": [vm.layer(vm.latent(4, 16, 8, 16, 24, 0.3, 10000.0), vm.moe(4, 2, 2, 24, 2.0, shared=16)),
                     vm.layer(vm.differential(2, 2, 16, 8, 0.4, 0.6), None)],
        "taps_from_the_tensors": [vm.layer(vm.latent(4, 32, 32, 64, 64, 0.2, 5e5, dims=16, window=70), vm.moe(8, 0, 8, 16, 2.0)),
                                  vm.layer(vm.delta(2, 2, 32, 32, 5), vm.moe(6, 6, 3, 16, 2.0, scale=3.0))],
    }[kind]
    cfg = vm.model(150, 64, 1e-5, layers, emb_scale=2.0, loop=(0, 2, 2) if kind == "recurrent_only" else None)
    folder = vm.write_model(str(tmp_path / "m"), cfg, 9, gain=GAIN[dtype], decisive_router=dtype == "bfloat16",
                            keep_taps=kind != "taps_from_the_tensors")
    runner = load_runner(folder, DT[dtype], num_pages=20, max_requests=3)
    assert len(runner.manager.groups) == {"recurrent_only": 0, "no_masks": 1, "taps_from_the_tensors": 1}[kind]
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
    """Position 0 sees itself alone, its sink, a zero state and zeros before the convolution: its logits are a function of
    the token."""
    folder = folders["D", "float32"]
    runner = load_runner(folder, torch.float32, num_pages=8)
    for tok in (0, 77, 98):
        a, b = run_whole(runner, "x", [tok]), run_whole(runner, "y", [tok, 5, 9, 2])
        assert rel_err(a, plain(folder, [tok])) < TOL["float32"] and torch.equal(a[0], b[0])
        assert rel_err(b, plain(folder, [tok, 5, 9, 2])) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(vm.CONFIGS))
def test_prefill_against_decoding_and_portions(name, dtype, folders):
    folder, vocab = folders[name, dtype], vm.CONFIGS[name]["vocab"]
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
    if dtype == "float32":      # in 32-bit a row's arithmetic does not depend on the cutting, beyond rounding
        assert rel_err(single, whole) < 2e-6 and rel_err(torch.cat(rows), whole) < 2e-6
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_unequal_requests_in_one_batch_against_each_alone(name, dtype, folders):
    folder, vocab = folders[name, dtype], vm.CONFIGS[name]["vocab"]
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
    assert [g.window for g in runner.manager.groups] == [17, 20, 24, 33]      # blocks keep a window of their size
    held = [sum(1 for p in runner.manager.block_table("d", g) if p >= 0) for g in range(4)]
    assert all(n <= w // 16 + 2 for n, w in zip(held, (17, 20, 24, 33)))
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
@pytest.mark.parametrize("name", list(vm.CONFIGS))
def test_replay_of_traces_with_pages_and_slots_used_again(name, dtype, folders, tmp_path):
    """Through bin/trace_run as a user would: whole, prefill then decode, portions, and mixed steps of up to four live
    requests, one process, a pool so small that pages and slots are used again."""
    folder, vocab = folders[name, dtype], vm.CONFIGS[name]["vocab"]
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
    """A configuration drawn from sizes of every kind: heads of many and few channels, grouped and ungrouped, values wider
    and narrower than keys, blocks and windows around a page's size or absent, recurrences of few and many channels and
    taps, identity experts or none, layers in any order with and without feed-forward, loops anywhere."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 72, 96, 160])
    layers = []
    for _ in range(rng.choice([1, 2, 3, 4])):
        kind = rng.choice(["attention", "delta", "latent"])
        if kind == "delta":
            kv = rng.choice([1, 2, 3])
            mixer = vm.delta(kv * rng.choice([1, 2]), kv, rng.choice([8, 10, 16, 32, 48, 64, 128]), rng.choice([8, 14, 16, 32, 64, 128]),
                             rng.choice([1, 2, 3, 4, 6]))
        elif kind == "attention":
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 12, 16, 32, 48, 64, 96])
            mixer = vm.differential(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([dim, 8, 10, 16, 32, 64]), rng.choice([1.0, 2.0]) / dim ** 0.5,
                                    rng.choice([0.2, 0.5, 0.8]), rng.choice([None, 1, 5, 16, 17, 64, 100]))
        else:
            rot = rng.choice([2, 4, 8, 16, 32])
            dim = rng.choice([8, 12, 16, 32, 64])
            mixer = vm.latent(rng.choice([1, 2, 3, 4, 8]), dim, rot, rng.choice([dim, 8, 10, 16, 32, 64]), rng.choice([8, 20, 32, 48, 96, 112]),
                              rng.choice([1.0, 2.0]) / (dim + rot) ** 0.5, rng.choice([100.0, 10000.0, 1e6]), rng.choice([rot, 2]),
                              rng.choice([None, 1, 5, 16, 17, 64, 100]))
        mlp = rng.choice([None, vm.moe(4, 2, 2, 24, 2.0, scale=2.0), vm.moe(8, 0, 3, 16, 1.0, shared=24, shared_limit=3.0), vm.moe(3, 1, 1, 40, 0.5, shared=8),
                          vm.moe(2, 2, 4, 8, 2.0, scale=0.5), vm.moe(5, 3, 2, 32, 7.0)])
        layers.append(vm.layer(mixer, mlp))
    n = len(layers)
    loop = None
    if rng.random() < 0.6:
        start = rng.randrange(n)
        loop = (start, rng.randrange(start + 1, n + 1), rng.choice([1, 2, 3]))
    return vm.model(rng.choice([61, 128, 500]), width, rng.choice([1e-5, 1e-6, 1e-3]), layers, emb_scale=rng.choice([1.0, 0.5, 3.0]),
                    logit_scale=rng.choice([1.0, 0.5, 2.0]), loop=loop)


@pytest.mark.parametrize("seed", range(14))
def test_drawn_configurations(seed, tmp_path):
    """Whole prompts, portions and decoding of drawn configurations against the plain implementation, both precisions."""
    cfg = _drawn_config(seed)
    for dtype in ("float32", "bfloat16"):
        folder = vm.write_model(str(tmp_path / dtype), cfg, 80 + seed, gain=GAIN[dtype], decisive_router=dtype == "bfloat16")
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
    folder, vocab = folders[name, "float32"], vm.CONFIGS[name]["vocab"]
    cfg, W = vm.load_plain(folder)
    prompts = [ids_of(70 + i, n, vocab) for i, n in enumerate([5, 40, 1, 77, 19, 130])]
    want = [pv.greedy_generate(cfg, W, p, 10) for p in prompts]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32, prefill_tokens_alone=48)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert [o.token_ids for o in outs] == want
    assert engine.runner.graph_replays > 0                       # decode steps ran as replayed graphs
    folder = folders[name, "bfloat16"]
    cfg, W = vm.load_plain(folder)
    engine = Engine.load(folder, dtype="bfloat16", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for p, o in zip(prompts, outs):        # bfloat16 may pick another token where two logits nearly tie
        full = pv.forward(cfg, W, p + o.token_ids)
        for i, tok in enumerate(o.token_ids):
            row = full[len(p) - 1 + i]
            assert row[tok] >= row.max() - 0.08 * np.abs(row).max(), (name, i)


def test_completion_from_the_command_line(folders, capsys):
    from inferflux_amd import cli
    folder = folders["B", "float32"]
    cfg, W = vm.load_plain(folder)
    prompt = ids_of(90, 21, 131)
    assert cli.main(["completion", "--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "7", "--temperature", "0",
                     "--ignore-eos", "--dtype", "float32", "--kv-pages", "32", "--max-parallel-sequences", "2"]) == 0
    said = capsys.readouterr().out
    want = pv.greedy_generate(cfg, W, prompt, 7)
    assert str(want)[1:-1].replace(" ", "") in said.replace(" ", ""), (want, said)
