"""The Vavadra decoder as a plan of parts.

A token's row of ``embed`` times a scale starts the residual stream.  Every layer is pre-norm, x <- x + mixer(norm1(x)) and,
where it has a feed-forward, x <- x + ff(norm2(x)), with RMS norms.  After the last layer the model's norm (``final.norm``)
and the embedding table itself as the output matrix follow; the logits are scaled.  A layer's mixer is one of

  attention          differential attention without positions: two softmax maps per head over the same values, the second
                     subtracted lambda times, the difference divided by its root mean square per head; biases on q, k
                     and v; a query sees the keys of its own block of ``mask.size`` positions
  delta              the gated delta rule: a matrix state per head, decayed per token and corrected along the token's
                     key; short causal convolutions on q, k and v; the output normed per head and gated
  latent_attention   attention through a key/value latent with one shared rotated key part (pairs of neighbouring
                     dimensions turn), a sliding window, and a learned sink score per head in the softmax's denominator

and its feed-forward a mixture of experts whose router takes a softmax over experts and identity experts (which hand the
row back as it is), chooses by score + correction, weighs by the score itself times a factor, and whose experts and shared
expert clamp gate and up before g sigmoid(1.702 g) (u + 1).  A span of layers may run several times in a row (``loop``):
the schedule names those layers once per pass, which gives each pass its own cache and state, and the first layer of each
pass is preceded by that pass's input (from the second pass on the embedding's output again, and always the pass's row of
``loop.step``).

Tensor names: ``embed``, ``loop.step``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``; a bias is
its matrix's name with ``.b``, a convolution's weight its projection's name with ``.conv``.
"""
from __future__ import annotations

from ..config.base import ConfigError
from ..config.registry import register_architecture
from ..config.vavadra import VavadraConfig
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry


def _differential(p: str, m, cfg: VavadraConfig) -> PartSpec:
    names = {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o", "q_bias": f"{p}.q.b", "k_bias": f"{p}.k.b",
             "v_bias": f"{p}.v.b", "lq1": f"{p}.lq1", "lk1": f"{p}.lk1", "lq2": f"{p}.lq2", "lk2": f"{p}.lk2"}
    return PartSpec("paged_attention", {
        "name": p, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim, "bias": True,
        "scale": m.scale, "chunk": m.chunk, "differential": {"diff": m.diff, "eps": cfg.norm_eps},
        "position": PartSpec("none", {}), "tensors": names})


def _delta(p: str, i: int, m, cfg: VavadraConfig) -> PartSpec:
    if m.conv is None:
        raise ConfigError(f"config.json: 'layers[{i}].mixer.conv' is left to the model file's tensors: load the config from a "
                          "model folder, or name the taps")
    names = {k: f"{p}.{k}" for k in ("q", "k", "v", "g", "b", "a", "o", "A_log", "dt_bias", "norm")}
    names.update({f"{k}_conv": f"{p}.{k}.conv" for k in "qkv"})
    return PartSpec("gated_delta", {"name": p, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim,
                                    "v_head_dim": m.vdim, "conv": m.conv, "norm_eps": cfg.norm_eps, "tensors": names})


def _latent(p: str, m, cfg: VavadraConfig) -> PartSpec:
    position = PartSpec("rotary", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dims, "theta": m.rot_base, "style": "split_half"})
    return PartSpec("latent_attention", {
        "name": p, "n_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "v_dim": m.vdim, "q_rank": None, "kv_rank": m.kv_rank,
        "scale": m.scale, "eps": cfg.norm_eps, "window": m.window, "sinks": True, "pairing": "interleaved", "position": position})


def _mlp(p: str, m) -> PartSpec:
    return PartSpec("moe", {"name": p, "n_experts": m.experts, "n_identity": m.identity, "top": m.top, "ff": m.ff,
                            "scoring": "softmax", "renormalize": False, "route_scale": m.route_scale, "choice_bias": True,
                            "activation": "clamped_swish", "limit": m.limit, "shared_ff": m.shared_ff,
                            "shared_limit": m.shared_limit})


def vavadra_plan(cfg: VavadraConfig) -> ModelPlan:
    layers = []
    norm = lambda name: PartSpec("rmsnorm", {"name": name, "tensor": name, "eps": cfg.norm_eps})
    for i, L in enumerate(cfg.layers):
        p = f"l{i}"
        if L.type == "attention":
            mixer = _differential(f"{p}.mix", L.mixer, cfg)
        elif L.type == "delta":
            mixer = _delta(f"{p}.mix", i, L.mixer, cfg)
        else:
            mixer = _latent(f"{p}.mix", L.mixer, cfg)
        ffn = norm_post = None
        if L.mlp is not None:
            ffn, norm_post = _mlp(f"{p}.mlp", L.mlp), norm(f"{p}.norm2")
        layers.append(LayerSpec(prefix=p, block=PartSpec("prenorm", {}), norm_in=norm(f"{p}.norm1"), mixer=mixer,
                                norm_post=norm_post, ffn=ffn))
    times = cfg.loop.times if cfg.loop is not None else 0
    injections = tuple(PartSpec("pass_input", {"index": t, "times": times, "tensor": "loop.step", "add_embedding": t > 0})
                       for t in range(times))
    return ModelPlan(
        vocab_size=cfg.vocab, hidden_size=cfg.width, max_position=cfg.max_positions,
        embedding=PartSpec("token_embedding", {"name": "embed", "tensor": "embed", "vocab_size": cfg.vocab,
                                               "scale": cfg.embedding_scale}),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i, before=t) for i, t in cfg.run_order()),
        final_norm=norm("final.norm"),
        lm_head=PartSpec("linear_head", {"name": "head", "tied_to": "embed", "vocab_size": cfg.vocab, "scale": cfg.logit_scale}),
        injections=injections,
    )


register_architecture(VavadraConfig, vavadra_plan)
