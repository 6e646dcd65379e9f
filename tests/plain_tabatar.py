"""The Tabatar decoder written out plainly, in float64 on the CPU: one function per mechanism, no cache, no batching,
nothing shared with the engine.  What the engine's kernels are compared with.

A model is (config, tensors): ``config`` the parsed config.json (a dict), ``tensors`` a dict of float64 arrays by the
names the model file uses.  Everything works on one whole sequence [T, ...].
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def banded_frequencies(dims, base, scaling):
    """Frequency of each of the dims / 2 pairs.  ``scaling`` {factor, low, high, original}: a pair whose wavelength is
    shorter than original / high keeps its frequency, one longer than original / low turns ``factor`` times slower, and
    between the two the frequency is blended by where original / wavelength lies between low and high."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return np.array(out, dtype=np.float64)


def rotate(x, positions, dims, base, scaling):
    """x [T, heads, d]: the first ``dims`` dimensions of every head turned, pair (i, i + dims/2) by position * f_i."""
    f = banded_frequencies(dims, base, scaling)
    a = positions.astype(np.float64)[:, None] * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    out = x.copy()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def window_attention(q, k, v, scale, size):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; position i sees j with 0 <= i - j < size (None: all j <= i)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if size is None else max(0, i - size + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ v[lo:i + 1, g]
    return out


def attention_mixer(h, W, p, m, eps):
    """The attention mixer with tensor prefix ``p`` (ending in '.') and sizes ``m`` on input h [T, width]."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    G, dv = m.get("kv_heads", H), m.get("vdim", d)
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    k = (h @ W[p + "k"].T).reshape(T, G, d)
    v = (h @ W[p + "v"].T).reshape(T, G, dv)
    q = rms_norm(q, W[p + "q.norm"], eps)
    k = rms_norm(k, W[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        pos = np.arange(T)
        dims = rot.get("dims", d)
        q = rotate(q, pos, dims, rot["base"], rot.get("scaling"))
        k = rotate(k, pos, dims, rot["base"], rot.get("scaling"))
    o = window_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size"))
    o = o.reshape(T, H * dv) * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def gla_decay(h, W, p, tau):
    """alpha [T, heads * dim]: sigmoid(W_a2 (W_a1 h) + b) ^ (1 / tau)."""
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    return sigmoid(z) ** (1.0 / tau)


def gla_recurrence(q, k, v, alpha, S0=None):
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k, alpha [T, H, d]; v [T, H, dv].
    Returns (o [T, H, dv], the last S [H, d, dv])."""
    T, H, d = q.shape
    dv = v.shape[2]
    S = np.zeros((H, d, dv)) if S0 is None else S0.copy()
    o = np.zeros((T, H, dv))
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    return o, S


def gla_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    dv = m.get("vdim", d)
    q = (h @ W[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, dv)
    alpha = gla_decay(h, W, p, float(m["tau"])).reshape(T, H, d)
    o, _ = gla_recurrence(q, k, v, alpha)
    o = rms_norm(o, W[p + "norm"], eps).reshape(T, H * dv)
    return (o * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def dense_ff(h, W, p):
    return gelu_tanh(h @ W[p + "up"].T) @ W[p + "down"].T


def gated_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, top):
    """(chosen experts [T, top], their weights [T, top]): the largest logits, softmax over those alone."""
    z = h @ W[p + "router"].T + W[p + "router.b"]
    ids = np.argsort(-z, axis=1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, ids, axis=1)
    e = np.exp(zc - zc.max(axis=1, keepdims=True))
    return ids, e / e.sum(axis=1, keepdims=True)


def moe_ff(h, W, p, m):
    ids, w = route(h, W, p, m["router"]["top"])
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, we in zip(ids[t], w[t]):
            out[t] += we * gated_expert(h[t:t + 1], W, f"{p}e{e}.")[0]
    if m.get("shared"):
        out = out + sigmoid(h @ W[p + "shared.sg"].T) * gated_expert(h, W, p + "shared.")
    return out


def feed_forward(h, W, p, m):
    return dense_ff(h, W, p) if m["kind"] == "dense" else moe_ff(h, W, p, m)


def hyper_step(xs, W, p, sublayer):
    """Streams xs [S, T, width] through one sub-block: read sum_s in[s] x_s, write x_t <- sum_s mix[s, t] x_s + out[t] y."""
    u = np.einsum("s,stw->tw", W[p + "in"], xs)
    y = sublayer(u)
    return np.einsum("st,sjw->tjw", W[p + "mix"], xs) + W[p + "out"][:, None, None] * y[None]


def layer_order(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(config, W, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the stream after every layer run, streams summed)."""
    eps = config["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)] * (config.get("embedding") or {}).get("scale", 1.0)
    streams = config.get("streams")
    xs = np.stack([x] * streams) if streams else None
    after = []
    for i in layer_order(config):
        L, p = config["layers"][i], f"l{i}."
        mixer = attention_mixer if L["type"] == "attention" else gla_mixer
        sub1 = lambda u: mixer(rms_norm(u, W[p + "norm1"], eps), W, p + "mix.", L["mixer"], eps)
        sub2 = lambda u: feed_forward(rms_norm(u, W[p + "norm2"], eps), W, p + "mlp.", L["mlp"])
        if streams:
            xs = hyper_step(xs, W, p + "hc1.", sub1)
            if L.get("mlp"):
                xs = hyper_step(xs, W, p + "hc2.", sub2)
            after.append(xs.sum(axis=0))
        else:
            x = x + sub1(x)
            if L.get("mlp"):
                x = x + sub2(x)
            after.append(x)
    x = xs.sum(axis=0) if streams else x
    logits = rms_norm(x, W["final.norm"], eps) @ W["head"].T * config.get("logit_scale", 1.0)
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * np.tanh(logits / cap)
    return (logits, np.stack(after)) if return_layers else logits


def greedy_generate(config, W, prompt, n):
    """n tokens, each the largest logit after everything before it (the whole sequence anew every time)."""
    ids, out = list(prompt), []
    for _ in range(n):
        tok = int(np.argmax(forward(config, W, ids)[-1]))
        ids.append(tok)
        out.append(tok)
    return out
