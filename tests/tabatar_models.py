"""Small Tabatar configurations for the tests and the folders they are written to: random weights made sharp, so that a
misplaced key, a window one token off, a lost state, a forgotten bias or a stream mixed the wrong way round moves the
logits by far more than rounding."""
import copy
import json
import os

import torch


def attention(heads, kv_heads, dim, vdim, scale, base, dims, window=None, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m}


def gla(heads, dim, vdim, tau, rank):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=0):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


def model(vocab, width, eps, layers, emb_scale=1.0, streams=None, logit_scale=1.0, softcap=None, loop=None):
    out = {"architecture": "Tabatar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb_scale},
           "logit_scale": logit_scale, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    if softcap is not None:
        out["logit_softcap"] = softcap
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


CONFIGS = {
    # layers that differ in everything: recurrences of two shapes, grouped heads with values wider than keys, windows of 20
    # and 33 (two cache groups), scaled and plain frequencies, both feed-forwards, a layer without one, three streams, and
    # two layers that run twice
    "A": model(300, 64, 1e-5, [
        layer(gla(2, 16, 24, 8.0, 6), dense(96)),
        layer(attention(4, 2, 16, 24, 0.6, 10000.0, 8, window=20, scaling=(4.0, 1.0, 4.0, 64)), moe(8, 2, 24, shared=40)),
        layer(gla(3, 8, 16, 3.0, 4), moe(6, 3, 32)),
        layer(attention(4, 2, 16, 24, 0.55, 500.0, 16, window=33), None),
        layer(gla(1, 32, 8, 20.0, 5), dense(72)),
    ], emb_scale=2.0, streams=3, logit_scale=1.5, softcap=12.0, loop=(1, 3, 2)),
    # what one model of the design may happen to make equal or 1, made so here and otherwise elsewhere: a single stream with
    # its connections, as many kv heads as heads, values as wide as keys, a rotation over the whole head, no window, tau 1,
    # one expert chosen, no shared expert, no loop, logits neither scaled nor capped
    "B": model(131, 88, 1e-6, [
        layer(attention(3, 3, 12, 12, 0.7, 2000.0, 12), moe(4, 1, 40)),
        layer(gla(2, 12, 12, 1.0, 7), dense(56)),
        layer(attention(2, 1, 20, 20, 0.5, 100.0, 20, window=7), dense(40)),
    ], streams=1),
    # no streams at all (the ordinary residual), sizes the matrix-core kernels take, a layer that runs three times
    "C": model(512, 128, 1e-5, [
        layer(attention(4, 2, 64, 64, 0.16, 10000.0, 32, window=48, scaling=(8.0, 1.0, 4.0, 256)), dense(192)),
        layer(gla(4, 64, 64, 16.0, 16), moe(16, 4, 64, shared=128)),
        layer(attention(8, 2, 32, 32, 0.3, 10000.0, 16, window=48), moe(16, 4, 64, shared=128)),
    ], emb_scale=0.5, logit_scale=0.7, softcap=30.0, loop=(1, 2, 3)),
    # nothing a multiple of 8; every expert chosen; five streams; the whole model in the loop
    "D": model(99, 100, 1e-5, [
        layer(gla(3, 10, 14, 5.0, 3), moe(5, 5, 22, shared=18)),
        layer(attention(3, 1, 10, 14, 0.9, 3000.0, 6, window=9), dense(50)),
    ], emb_scale=1.5, streams=5, logit_scale=2.0, softcap=8.0, loop=(0, 2, 2)),
    # a size at which the products take their other kernels (weights in tiles, K in slices, the library for prompts), heads of
    # 128 channels in the recurrence and of 48 and 96 in attention, many experts
    "E": model(1000, 512, 1e-5, [
        layer(gla(4, 128, 128, 16.0, 32), moe(32, 6, 256, shared=512)),
        layer(attention(16, 2, 48, 96, 0.2, 50000.0, 48, window=56, scaling=(4.0, 2.0, 16.0, 512)), dense(1536)),
        layer(gla(8, 32, 96, 4.0, 24), dense(1024)),
        layer(attention(8, 2, 96, 96, 0.12, 50000.0, 32, window=128), moe(32, 6, 256, shared=512)),
    ], emb_scale=4.0, streams=2, logit_scale=1.0, softcap=20.0),
}


def config(name):
    return copy.deepcopy(CONFIGS[name])


def router_values(n):
    """n distinct router logits between -2 and 2.6, unevenly spaced, no two closer than half the mean spacing."""
    import math
    step = 4.6 / max(n - 1, 1)
    return [-2.0 + step * k + 0.2 * step * math.sin(1.7 * k + 0.3) for k in range(n)]


def write_model(folder, cfg, seed, gain=1.0, keep_rank=False, decisive_router=False):
    """config.json and model.safetensors with seeded weights, bfloat16-representable, shaped so that faults show: norm
    weights away from 1, query/key projections with a gain (peaked attention), decays over the range a trained recurrence
    has (from forgetting within a few tokens to remembering hundreds), router and gate biases that matter, stream
    connections that are neither the identity nor symmetric.  Without ``keep_rank`` the written config.json leaves the
    recurrences' decay rank to the tensors' shapes.

    With ``decisive_router`` no choice of experts is a close call, so that an engine that rounds its activations to
    bfloat16 makes the choices of the exact model (a choice that rounding flips changes a row's logits altogether and says
    nothing about the kernels): expert e's router row reads channel e of its input alone, a token's embedding holds a
    permutation of ``router_values`` on those channels, nothing writes into them (the rows of every matrix that writes into
    the stream are zero there), the norms before the experts have weight 1 on them and the routers have no bias, so a
    router's logits are a token's values times one positive number.  (Routers with random weights and biases run in 32-bit.)"""
    from safetensors.torch import save_file
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.model import Model
    g = torch.Generator().manual_seed(seed)
    specs = Model.param_specs_for(config_from_dict(cfg))
    tensors = {}
    for name, spec in specs.items():
        shape = tuple(spec.shape)
        if name.endswith(("norm", "norm1", "norm2")):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith((".hc1.in", ".hc2.in")):
            t = (0.5 + torch.rand(shape, generator=g)) / shape[0]
        elif name.endswith((".hc1.out", ".hc2.out")):
            t = 0.4 + 0.8 * torch.rand(shape, generator=g)
        elif name.endswith((".hc1.mix", ".hc2.mix")):
            t = 0.6 * torch.eye(shape[0]) + 0.8 * torch.rand(shape, generator=g) / shape[0]
        elif name.endswith(".a2.b"):
            t = -1.0 + 7.0 * torch.rand(shape, generator=g)
        elif name.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.5
        else:
            t = torch.randn(shape, generator=g) / (shape[-1] ** 0.5)
            if name.endswith((".mix.q", ".mix.k")):
                t = t * gain
            elif name.endswith((".mix.a2", ".router", ".shared.sg")):
                t = t * 2.0
            elif name == "embed":
                t = t * shape[-1] ** 0.5
        tensors[name] = t.to(torch.bfloat16).contiguous()
    n = max([L["mlp"]["router"]["experts"] for L in cfg["layers"] if L["mlp"] is not None and L["mlp"]["kind"] == "moe"], default=0)
    if decisive_router and n:
        values = torch.tensor(router_values(n))
        for tok in range(cfg["vocab"]):
            tensors["embed"][tok, :n] = values[torch.randperm(n, generator=g)].to(torch.bfloat16)
        for name, t in tensors.items():
            if name.endswith((".o", ".down")):
                t[:n] = 0
            elif name.endswith(".norm2"):
                t[:n] = 1
            elif name.endswith(".router"):
                t.zero_()
                t[:, :t.shape[0]] = torch.eye(t.shape[0]).to(t.dtype)
            elif name.endswith(".router.b"):
                t.zero_()
    os.makedirs(folder, exist_ok=True)
    written = copy.deepcopy(cfg)
    if not keep_rank:
        for L in written["layers"]:
            L["mixer"].pop("rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(written, f)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    return folder


def load_plain(folder):
    """(config, tensors as float64 arrays) for the plain implementation."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
