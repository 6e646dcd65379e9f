"""Small Vavadra configurations for the tests and the folders they are written to: random weights made sharp, so that a
misplaced key, a block or a window one token off, a lost state, a forgotten sink or bias, or a pass that was not given its
input moves the logits by far more than rounding."""
import copy
import json
import math
import os

import torch


def differential(heads, kv_heads, dim, vdim, scale, diff, chunk=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if chunk:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, dims=None, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def moe(experts, identity, top, ff, limit, scale=1.0, shared=0, shared_limit=None):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "identity": identity, "top": top, "scale": scale}}
    if shared:
        m["shared"] = {"ff": shared, "limit": limit if shared_limit is None else shared_limit}
    return m


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


def model(vocab, width, eps, layers, emb_scale=1.0, logit_scale=1.0, loop=None):
    out = {"architecture": "Vavadra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb_scale},
           "logit_scale": logit_scale, "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


CONFIGS = {
    # layers that differ in everything: two latent layers with windows of 20 and 33 (two cache groups) of which one turns only
    # some of its rotated dimensions, blocks of 24, grouped heads, values wider than keys, a recurrence whose query/key heads
    # are fewer than its value heads, identity experts, a layer without feed-forward, two layers that run twice
    "A": model(300, 64, 1e-5, [
        layer(latent(4, 16, 8, 24, 32, 0.3, 10000.0, window=20), moe(6, 2, 2, 24, 2.0, scale=2.0, shared=40, shared_limit=1.0)),
        layer(differential(4, 2, 8, 24, 0.5, 0.4, chunk=24), moe(5, 3, 3, 32, 1.5, scale=1.5)),
        layer(delta(4, 2, 16, 24, 4), None),
        layer(latent(2, 24, 12, 16, 40, 0.25, 500.0, dims=8, window=33), moe(6, 2, 2, 24, 2.0, scale=2.0, shared=40, shared_limit=1.0)),
        layer(differential(3, 1, 16, 8, 0.35, 0.7, chunk=17), moe(4, 1, 1, 40, 3.0)),
    ], emb_scale=3.0, logit_scale=1.5, loop=(1, 3, 2)),
    # what one model of the design may happen to make equal or 1, made so here and otherwise elsewhere: as many kv heads as
    # heads, values as wide as keys, no identity experts, one expert chosen, no shared expert, no loop, no masks, logits and
    # embedding unscaled, two taps
    "B": model(131, 88, 1e-6, [
        layer(differential(3, 3, 12, 12, 0.4, 0.2), moe(4, 0, 1, 40, 2.0)),
        layer(delta(2, 2, 12, 12, 2), moe(3, 0, 2, 24, 1.0)),
        layer(latent(1, 20, 20, 20, 24, 0.3, 100.0), moe(4, 0, 1, 40, 2.0)),
    ]),
    # sizes the matrix-core kernels take, a layer that runs three times, the loop from the first layer
    "C": model(512, 128, 1e-5, [
        layer(delta(4, 4, 64, 64, 4), moe(14, 2, 4, 64, 2.0, scale=2.0, shared=128)),
        layer(latent(4, 64, 16, 64, 112, 0.11, 10000.0, window=48), moe(14, 2, 4, 64, 2.0, scale=2.0, shared=128)),
        layer(differential(8, 2, 32, 64, 0.18, 0.5, chunk=48), moe(8, 8, 2, 64, 2.0, shared=64)),
    ], emb_scale=6.0, logit_scale=2.0, loop=(0, 1, 3)),
    # nothing a multiple of 8; every expert and identity expert chosen; the whole model in the loop; one tap
    "D": model(99, 100, 1e-5, [
        layer(delta(3, 1, 10, 14, 1), moe(3, 2, 5, 22, 0.7, scale=0.5, shared=18, shared_limit=2.5)),
        layer(differential(3, 1, 10, 14, 0.6, 0.3, chunk=9), None),
        layer(latent(3, 10, 6, 14, 18, 0.5, 3000.0, dims=2, window=9), moe(5, 1, 2, 22, 1.2)),
    ], emb_scale=1.5, logit_scale=2.0, loop=(0, 3, 2)),
    # a size at which the products take their other kernels (weights in tiles, K in slices, the library for prompts), heads of
    # 128 channels in the recurrence, many experts
    "E": model(1000, 512, 1e-5, [
        layer(delta(4, 2, 128, 128, 4), moe(30, 2, 6, 256, 2.0, scale=2.0, shared=512, shared_limit=1.0)),
        layer(differential(8, 2, 48, 96, 0.15, 0.5, chunk=56), moe(30, 2, 6, 256, 2.0, scale=2.0, shared=512, shared_limit=1.0)),
        layer(latent(8, 64, 32, 96, 160, 0.1, 50000.0, dims=32, window=128), None),
        layer(delta(8, 8, 32, 96, 3), moe(12, 4, 2, 128, 4.0)),
    ], emb_scale=4.0, loop=(1, 3, 2)),
}


def config(name):
    return copy.deepcopy(CONFIGS[name])


def router_values(n):
    """n distinct router logits between -2 and 2.6, unevenly spaced, no two closer than half the mean spacing."""
    step = 4.6 / max(n - 1, 1)
    return [-2.0 + step * k + 0.2 * step * math.sin(1.7 * k + 0.3) for k in range(n)]


def write_model(folder, cfg, seed, gain=1.0, keep_taps=True, decisive_router=False):
    """config.json and model.safetensors with seeded weights, bfloat16-representable, shaped so that faults show: norm
    weights away from 1, query/key projections with a gain (peaked attention), sinks of both signs, lambdas away from their
    constant, decays from forgetting within a few tokens to remembering hundreds, corrections that change the choice, pass
    inputs as large as the stream.  Without ``keep_taps`` the written config.json leaves the taps to the tensors' shapes.

    With ``decisive_router`` no choice of experts is a close call, so that an engine that rounds its activations to
    bfloat16 makes the choices of the exact model: output e of a router reads channel e of its input alone, a token's
    embedding holds a permutation of ``router_values`` on those channels, nothing but identity experts and the embedding fed
    in again writes into them (which scale them all alike), the norms before the experts have weight 1 on them, and the
    corrections are small beside the gaps between the highest scores."""
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
        elif name.endswith(".sink"):
            t = 1.5 * torch.randn(shape, generator=g)
        elif name.endswith((".lq1", ".lk1", ".lq2", ".lk2")):
            t = 0.35 * torch.randn(shape, generator=g)
        elif name.endswith(".A_log"):
            t = -3.5 + 4.0 * torch.rand(shape, generator=g)
        elif name.endswith(".dt_bias"):
            t = -2.0 + 3.0 * torch.rand(shape, generator=g)
        elif name.endswith(".conv"):
            t = 0.6 * torch.randn(shape, generator=g)
        elif name.endswith(".correction"):
            t = (0.01 if decisive_router else 0.15) * torch.randn(shape, generator=g)
        elif name == "loop.step":
            t = torch.randn(shape, generator=g)
        elif name.endswith(".b") and len(shape) == 1:
            t = torch.randn(shape, generator=g) * 0.5
        else:
            t = torch.randn(shape, generator=g) / (shape[-1] ** 0.5)
            if name.endswith((".mix.q", ".mix.k")):
                t = t * gain
            elif name.endswith((".mix.a", ".mix.b", ".router")):
                t = t * 2.0
            elif name == "embed":
                t = t * shape[-1] ** 0.5 / 3.0
        tensors[name] = t.to(torch.bfloat16).contiguous()
    n = max([L["mlp"]["router"]["experts"] + L["mlp"]["router"].get("identity", 0) for L in cfg["layers"] if L["mlp"] is not None],
            default=0)
    if decisive_router and n:
        values = torch.tensor(router_values(n)) / 3.0
        for tok in range(cfg["vocab"]):
            tensors["embed"][tok, :n] = values[torch.randperm(n, generator=g)].to(torch.bfloat16)
        for name, t in tensors.items():
            if name.endswith((".o", ".down")):
                t[:n] = 0
            elif name.endswith(".norm2"):
                t[:n] = 1
            elif name == "loop.step":
                t[:, :n] = 0
            elif name.endswith(".router"):
                t.zero_()
                t[:, :t.shape[0]] = 3.0 * torch.eye(t.shape[0]).to(t.dtype)
    os.makedirs(folder, exist_ok=True)
    written = copy.deepcopy(cfg)
    if not keep_taps:
        for L in written["layers"]:
            L["mixer"].pop("conv", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(written, f)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    return folder


def load_plain(folder):
    """(config, tensors as float64 arrays) for the plain implementation.  A config that leaves the taps out gets them from
    the tensors, as the engine's does."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
