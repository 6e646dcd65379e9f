"""Gated linear attention: a recurrence per head whose state is a matrix S [d, dv] and whose decay is a vector per token.

With ``n_heads`` heads, keys and queries of ``head_dim`` channels, values of ``v_head_dim`` and a decay projected through
``decay_rank`` numbers, for a request's tokens t = 0, 1, ...:

    q = W_q h * head_dim^(-1/2),  k = W_k h,  v = W_v h,  g = W_g h
    z = W_a2 (W_a1 h) + b_a2                               (n_heads x head_dim)
    alpha = sigmoid(z) ^ (1 / tau)                         per key channel, in float
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  S_(-1) = 0   per head, in float
    o_t = S_t^T q_t
    out = W_o ( rmsnorm_head(o_t) * w_norm * silu(g) )     the norm over each head's v_head_dim, one weight for all heads

What a request carries from step to step is its S: one float32 row of the engine's per-request state (``StateSpec``), laid
out as the kernel of ``csrc/gla.hip`` wants it, zeroed when the request starts.  Nothing is kept per token, so the layer
owns no cache pages.  q, k, v, g and the decay's first product come from one fused projection in the activation type; the
decay's second product gives float32, and decays, S, o, the norm and the gate are float whatever the activation type.

Tensors (``tensors`` maps the roles "q", "k", "v", "g", "o", "a1", "a2", "a2_bias", "norm" to full names; by default
``<name>.q_proj.weight`` and so on, ``<name>.a2_proj.bias``, ``<name>.norm.weight``).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, MixerBinding, register_part
from .ffn import concat_weights
from .plan import ParamSpec, StateSpec


SCAN_CHUNK = 32             # rows of a chunk where long portions are cut into chunks that run side by side
SCAN_CHUNK_MIN_ROWS = 128   # ... which happens in steps that bring some request this many rows or more


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    graph_safe = True          # the kernel reads the step's layout from the context's device arrays
    adds_to_stream = True

    def __init__(self, name: str, hidden_size: int, n_heads: int, head_dim: int, v_head_dim: int, decay_rank: int, tau: float,
                 norm_eps: float, init_std: float = 0.02, tensors: Optional[Mapping[str, str]] = None):
        self.name, self.hidden_size = name, int(hidden_size)
        self.n_heads, self.head_dim, self.v_head_dim = int(n_heads), int(head_dim), int(v_head_dim)
        self.decay_rank, self.tau, self.norm_eps = int(decay_rank), float(tau), float(norm_eps)
        if min(self.n_heads, self.head_dim, self.v_head_dim, self.decay_rank) <= 0 or self.tau <= 0:
            raise ValueError(f"{name}: heads, head_dim, v_head_dim, decay_rank and tau must be positive")
        ops.gla_layout(self.head_dim, self.v_head_dim)          # (refuses head sizes the kernel has no layout for)
        self.init_std = init_std
        self.names = {k: f"{name}.{k}_proj.weight" for k in ("q", "k", "v", "g", "o", "a1", "a2")}
        self.names.update({"a2_bias": f"{name}.a2_proj.bias", "norm": f"{name}.norm.weight"})
        self.names.update(tensors or {})
        self.w_in = self.w_a2 = self.w_o = self.a2_bias = self.norm_w = None

    def state_spec(self) -> StateSpec:
        return StateSpec((ops.gla_state_floats(self.n_heads, self.head_dim, self.v_head_dim),), "float32")

    def param_specs(self) -> Dict[str, ParamSpec]:
        nm, H, s = self.names, self.hidden_size, ("normal", self.init_std)
        HD, HV, r = self.n_heads * self.head_dim, self.n_heads * self.v_head_dim, self.decay_rank
        return {
            nm["q"]: ParamSpec((HD, H), s), nm["k"]: ParamSpec((HD, H), s), nm["v"]: ParamSpec((HV, H), s),
            nm["g"]: ParamSpec((HV, H), s), nm["o"]: ParamSpec((H, HV), s), nm["a1"]: ParamSpec((r, H), s),
            nm["a2"]: ParamSpec((HD, r), ("normal", 0.5)), nm["a2_bias"]: ParamSpec((HD,), ("uniform", 0.0, 6.0)),
            nm["norm"]: ParamSpec((self.v_head_dim,), ("ones",)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        nm = self.names
        self.w_in = ops.prepare_linear(concat_weights([tensors[nm[p]] for p in ("q", "k", "v", "g", "a1")]))
        self.w_a2 = ops.prepare_linear(tensors[nm["a2"]])
        self.w_o = ops.prepare_linear(tensors[nm["o"]])
        self.a2_bias = tensors[nm["a2_bias"]].float().contiguous()      # float whatever the file holds
        self.norm_w = tensors[nm["norm"]]

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_in)

    def forward(self, h, ctx, binding: MixerBinding, sink=None):
        state, t = binding.state, ctx.timer
        if state is None:
            raise ValueError(f"{self.name}: the mixer was given no per-request state")
        HD, HV, r = self.n_heads * self.head_dim, self.n_heads * self.v_head_dim, self.decay_rank
        rows = ops.linear(h, self.w_in)                                 # [T, q | k | v | g | a1]
        a1 = rows[:, 2 * HD + 2 * HV:].contiguous() if rows.shape[0] else rows.new_empty((0, r))
        z = ops.linear(a1, self.w_a2, out_dtype=torch.float32)         # the decays' logits are never rounded
        if t is not None:
            t.mark("mixer.project")
        # A prompt's portion walked token by token leaves most of the chip idle: in bfloat16 long portions are cut into
        # chunks that run side by side.  In 32-bit the walk stays in one piece, so that a token's sums do not depend on
        # where its request was cut.  (Steps of single tokens never take the chunks: a captured layout keeps its launches.)
        chunks = None
        if rows.dtype == torch.bfloat16 and ctx.n_tokens > ctx.n_requests and int(ctx.h_q_len.max()) >= SCAN_CHUNK_MIN_ROWS:
            chunks = ctx.derived(("scan_chunks", SCAN_CHUNK), lambda: ops.scan_chunks(ctx.h_q_start, ctx.h_q_len, SCAN_CHUNK, ctx.device))
        y = ops.gla_scan(rows, (0, HD, 2 * HD, 2 * HD + HV), z, self.a2_bias, self.tau, self.head_dim ** -0.5, self.norm_w,
                         self.norm_eps, self.n_heads, self.head_dim, self.v_head_dim, state, 0, ctx.q_start, ctx.q_len,
                         ctx.state_slots, chunks)
        if t is not None:
            t.mark("mixer.scan")
        if sink is not None and ops.adds_into_stream(y.shape[0], self.w_o, sink.norm_weight):
            return ops.linear_into_stream(y, self.w_o, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(y, self.w_o, keep_slices=sink is not None)
