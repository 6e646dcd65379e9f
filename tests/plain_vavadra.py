"""The Vavadra decoder written out plainly, in float64 on the CPU: one function per mechanism, no cache, no batching,
nothing shared with the engine.  What the engine's kernels are compared with.

A model is (config, tensors): ``config`` the parsed config.json (a dict), ``tensors`` a dict of float64 arrays by the
names the model file uses.  Everything works on one whole sequence [T, ...].
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w None: no weight)."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


# ---- masks ------------------------------------------------------------------------------------------------------------
def chunk_mask(T, size):
    """[T, T] True where query i sees key j: j <= i and both in the same block of ``size`` positions counted from 0 (None:
    every j <= i)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) if size is None else (j <= i) & (i // size == j // size)


def window_mask(T, size):
    """[T, T] True where query i sees key j: 0 <= i - j < size (None: every j <= i)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) if size is None else (j <= i) & (i - j < size)


def masked_softmax(s, mask, sink=None):
    """Softmax of each row of s [T, T] over the keys the mask allows; ``sink``: one more term exp(sink) in the denominator."""
    s = np.where(mask, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.exp(s - m)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - m)
    return e / den


# ---- differential attention -------------------------------------------------------------------------------------------
def _size(m):
    return (m.get("mask") or {}).get("size")


def differential_attention(h, W, p, m, eps):
    """Two softmax maps per head over the same values, the second subtracted lambda times; chunked mask; no positions."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = (h @ W[p + ".q"].T + W[p + ".q.b"]).reshape(T, H, 2, d)
    k = (h @ W[p + ".k"].T + W[p + ".k.b"]).reshape(T, G, 2, d)
    v = (h @ W[p + ".v"].T + W[p + ".v.b"]).reshape(T, G, dv)
    lam = math.exp(float(np.sum(W[p + ".lq1"] * W[p + ".lk1"]))) - math.exp(float(np.sum(W[p + ".lq2"] * W[p + ".lk2"]))) + m["diff"]
    mask = chunk_mask(T, _size(m))
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // (H // G)
        a = [masked_softmax((q[:, hd, c] @ k[:, g, c].T) * m["scale"], mask) @ v[:, g] for c in (0, 1)]
        o = a[0] - lam * a[1]
        out[:, hd] = rms_norm(o, None, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ W[p + ".o"].T


# ---- gated delta rule ---------------------------------------------------------------------------------------------------
def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - (taps - 1) + j), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x])
    return sum(padded[j:j + T] * w[:, j] for j in range(taps))


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_recurrence(q, k, v, beta, decay):
    """One head: q, k [T, d], v [T, dv], beta, decay [T].  S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, d = q.shape
    S, out = np.zeros((d, v.shape[1])), np.zeros_like(v)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def gated_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = silu(causal_conv(h @ W[p + ".q"].T, W[p + ".q.conv"])).reshape(T, G, d)
    k = silu(causal_conv(h @ W[p + ".k"].T, W[p + ".k.conv"])).reshape(T, G, d)
    v = silu(causal_conv(h @ W[p + ".v"].T, W[p + ".v.conv"])).reshape(T, H, dv)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = sigmoid(h @ W[p + ".b"].T)                                                         # [T, H]
    decay = np.exp(-np.exp(W[p + ".A_log"]) * softplus(h @ W[p + ".a"].T + W[p + ".dt_bias"]))   # [T, H]
    gate = silu(h @ W[p + ".g"].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // (H // G)
        out[:, hd] = delta_recurrence(q[:, g], k[:, g], v[:, hd], beta[:, hd], decay[:, hd])
    out = rms_norm(out, W[p + ".norm"], eps) * gate
    return out.reshape(T, H * dv) @ W[p + ".o"].T


# ---- attention through a latent -------------------------------------------------------------------------------------------
def rotate_pairs(x, positions, dims, base):
    """x [T, ..., D]: of the first ``dims`` dimensions, (2i, 2i + 1) turned by position * base^(-2i / dims)."""
    f = base ** (-2.0 * np.arange(dims // 2) / dims)
    a = positions.astype(np.float64)[:, None] * f[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = np.cos(a).reshape(shape), np.sin(a).reshape(shape)
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, W, p, m, eps, positions):
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m.get("vdim", m["dim"]), m["kv_rank"]
    dims = m["rot"].get("dims", r)
    q = (h @ W[p + ".q"].T).reshape(T, H, d + r)
    down = h @ W[p + ".dkv"].T
    c = rms_norm(down[:, :rank], W[p + ".dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, rank:], positions, dims, m["rot"]["base"])      # [T, r], one for all heads
    q_rot = rotate_pairs(q[:, :, d:], positions, dims, m["rot"]["base"])
    k_plain = (c @ W[p + ".uk"].T).reshape(T, H, d)
    v = (c @ W[p + ".uv"].T).reshape(T, H, dv)
    mask = window_mask(T, _size(m))
    out = np.zeros((T, H, dv))
    for hd in range(H):
        s = (q[:, hd, :d] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * m["scale"]
        out[:, hd] = masked_softmax(s, mask, sink=float(W[p + ".sink"][hd])) @ v[:, hd]
    return out.reshape(T, H * dv) @ W[p + ".o"].T


# ---- feed-forward ---------------------------------------------------------------------------------------------------------
def clamped_expert(h, W, p, limit):
    g = np.minimum(h @ W[p + ".gate"].T, limit)
    u = np.clip(h @ W[p + ".up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + ".down"].T


def route(h, W, p, r):
    """(ids [T, top], weights [T, top]): softmax over experts + identity; the choice adds the correction, the weights do not."""
    z = h @ W[p + ".router"].T
    s = np.exp(z - z.max(axis=-1, keepdims=True))
    s = s / s.sum(axis=-1, keepdims=True)
    choice = s + W[p + ".correction"]
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :r["top"]]
    return ids, np.take_along_axis(s, ids, axis=-1) * r.get("scale", 1.0)


def moe(h, W, p, m):
    r = m["router"]
    n_real = r["experts"]
    ids, weights = route(h, W, p, r)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t], weights[t]):
            y = h[t] if e >= n_real else clamped_expert(h[t:t + 1], W, f"{p}.e{e}", m["expert"]["limit"])[0]
            out[t] += w * y
    if m.get("shared"):
        out = out + clamped_expert(h, W, p + ".shared", m["shared"]["limit"])
    return out


# ---- the model ------------------------------------------------------------------------------------------------------------
def run_order(config):
    """[(layer, pass or None)]: the looped span ``times`` times in a row; pass is set on a pass's first layer."""
    n, lp = len(config["layers"]), config.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        out += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return out + [(i, None) for i in range(lp["stop"], n)]


def mixer(h, W, i, L, eps, positions):
    p = f"l{i}.mix"
    if L["type"] == "attention":
        return differential_attention(h, W, p, L["mixer"], eps)
    if L["type"] == "delta":
        return gated_delta(h, W, p, L["mixer"], eps)
    return latent_attention(h, W, p, L["mixer"], eps, positions)


def forward(config, W, tokens, return_layers=False):
    """float64 logits [T, vocab] of one sequence (and the stream after every layer run)."""
    tokens = np.asarray(tokens)
    eps = config["norm"]["eps"]
    positions = np.arange(tokens.shape[0])
    x0 = W["embed"][tokens] * config.get("embedding", {}).get("scale", 1.0)
    x, after = x0.copy(), []
    for i, t in run_order(config):
        L = config["layers"][i]
        if t is not None:
            if t > 0:
                x = x + x0
            x = x + W["loop.step"][t]
        x = x + mixer(rms_norm(x, W[f"l{i}.norm1"], eps), W, i, L, eps, positions)
        if L.get("mlp"):
            x = x + moe(rms_norm(x, W[f"l{i}.norm2"], eps), W, f"l{i}.mlp", L["mlp"])
        after.append(x.copy())
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].T * config.get("logit_scale", 1.0)
    return (logits, np.stack(after)) if return_layers else logits


def greedy_generate(config, W, prompt, n):
    """The n tokens that follow ``prompt`` when the most likely token is taken every time (the lowest id among equals)."""
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(np.argmax(forward(config, W, ids)[-1])))
    return ids[len(prompt):]
