"""The Tabatar decoder as a plan of parts.

A token's row of ``embed`` times a scale starts ``streams`` equal residual streams.  Every layer reads them through
learned weights, norms what it read (RMS norms), runs its mixer and writes the result back into all streams through a
mixing matrix and output weights (the "hyper" arrangement); where it has a feed-forward the same happens again around
it.  After the last layer the streams are added up, and the model's norm (``final.norm``) and the output matrix ``head``
follow; the logits are scaled and squashed by c * tanh(logit / c).  A config without ``streams`` gives the ordinary
pre-norm arrangement over one stream.  A layer's mixer is either

  attention   grouped-query attention without biases, an RMS norm with a weight on every q and k head before the
              rotation, a rotation of the first dimensions of every head with frequencies scaled in bands of
              wavelength, a sliding window, an ordinary softmax, and a sigmoid gate on every element of the
              concatenated heads; or
  gla         gated linear attention: a matrix-valued recurrence per head with a decay per key channel, a norm per
              head on its output and a silu gate,

and its feed-forward is either a plain one with the tanh form of gelu or a mixture of experts (gated with silu; a
biased router whose chosen logits go through a softmax of their own; a shared expert behind a sigmoid gate of one
number per token).  A span of layers may run several times in a row (``loop``): the schedule names those layers once
per pass, which gives each pass its own cache and state.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.hc1.*``, ``l<i>.hc2.*``,
``final.norm``, ``head``; a bias is its matrix's name with ``.b``.
"""
from __future__ import annotations

from ..config.base import ConfigError
from ..config.registry import register_architecture
from ..config.tabatar import TabatarConfig
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, ScheduleEntry


def _attention(p: str, m, cfg: TabatarConfig) -> PartSpec:
    names = {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o", "gate": f"{p}.g", "q_norm": f"{p}.q.norm",
             "k_norm": f"{p}.k.norm"}
    position = PartSpec("rotary", {"head_dim": m.dim, "rotary_dim": m.rot_dims, "theta": m.rot_base, "style": "split_half",
                                   "scaling": m.rot_scaling.to_dict() if m.rot_scaling is not None else None})
    return PartSpec("paged_attention", {
        "name": p, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim, "bias": False,
        "scale": m.scale, "window": m.window, "qk_norm_eps": cfg.norm_eps, "output_gate": "elementwise",
        "position": position, "tensors": names})


def _gla(p: str, i: int, m, cfg: TabatarConfig) -> PartSpec:
    if m.rank is None:
        raise ConfigError(f"config.json: 'layers[{i}].mixer.rank' is left to the model file's tensors: load the config from a "
                          "model folder, or name the rank")
    names = {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "g": f"{p}.g", "o": f"{p}.o", "a1": f"{p}.a1", "a2": f"{p}.a2",
             "a2_bias": f"{p}.a2.b", "norm": f"{p}.norm"}
    return PartSpec("gated_linear_attention", {"name": p, "n_heads": m.heads, "head_dim": m.dim, "v_head_dim": m.vdim,
                                               "decay_rank": m.rank, "tau": m.tau, "norm_eps": cfg.norm_eps, "tensors": names})


def _mlp(p: str, m) -> PartSpec:
    if m.kind == "dense":
        return PartSpec("dense_ffn", {"name": p, "intermediate_size": m.ff, "activation": "gelu_tanh",
                                      "tensors": {"up": f"{p}.up", "down": f"{p}.down"}})
    return PartSpec("moe", {"name": p, "n_experts": m.experts, "top": m.top, "ff": m.ff, "scoring": "softmax",
                            "renormalize": True, "router_bias": True, "shared_ff": m.shared_ff, "shared_gate": bool(m.shared_ff)})


def tabatar_plan(cfg: TabatarConfig) -> ModelPlan:
    layers = []
    norm = lambda name: PartSpec("rmsnorm", {"name": name, "tensor": name, "eps": cfg.norm_eps})
    block = PartSpec("prenorm", {}) if cfg.streams is None else PartSpec("hyper", {"streams": cfg.streams})
    for i, L in enumerate(cfg.layers):
        p = f"l{i}"
        mixer = _attention(f"{p}.mix", L.mixer, cfg) if L.type == "attention" else _gla(f"{p}.mix", i, L.mixer, cfg)
        ffn = norm_post = None
        if L.mlp is not None:
            ffn, norm_post = _mlp(f"{p}.mlp", L.mlp), norm(f"{p}.norm2")
        layers.append(LayerSpec(prefix=p, block=block, norm_in=norm(f"{p}.norm1"), mixer=mixer, norm_post=norm_post, ffn=ffn))
    return ModelPlan(
        vocab_size=cfg.vocab, hidden_size=cfg.width, max_position=cfg.max_positions,
        embedding=PartSpec("token_embedding", {"name": "embed", "tensor": "embed", "vocab_size": cfg.vocab,
                                               "scale": cfg.embedding_scale}),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in cfg.run_order()),
        final_norm=norm("final.norm"),
        lm_head=PartSpec("linear_head", {"name": "head", "tensor": "head", "vocab_size": cfg.vocab,
                                         "scale": cfg.logit_scale, "softcap": cfg.logit_softcap}),
    )


register_architecture(TabatarConfig, tabatar_plan)
