"""The gated delta rule: a recurrence per head whose state is a matrix S [d, dv], decayed by one number per token and
corrected towards the token's value along the token's key.

With ``n_heads`` value heads of ``v_head_dim``, ``n_kv_heads`` query/key heads of ``head_dim`` (value head h reads
query/key head h // (n_heads / n_kv_heads)) and a short causal convolution of ``conv`` taps, for a request's tokens
t = 0, 1, ...:

    q, k, v = silu(conv_q(W_q h)), silu(conv_k(W_k h)), silu(conv_v(W_v h))    per channel, zeros before the start,
                                                                               the last tap is the current token's
    q = unit(q) * head_dim^(-1/2),  k = unit(k),  unit(x) = x / sqrt(sum(x^2) + 1e-6) per head
    beta = sigmoid(W_b h),  g = exp(-exp(A_log) * softplus(W_a h + dt_bias))   one of each per value head
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q               (the read-out sees the token's own write)
    out = W_o ( o / sqrt(mean(o^2) + eps) * w_norm * silu(W_g h) )             the norm over each head's v_head_dim

What a request carries from step to step is the convolution's last conv - 1 inputs and its S: one float32 row of the
engine's per-request state (``StateSpec``), the convolution's part first, laid out as the kernels of ``csrc/ssm.hip`` and
``csrc/delta.hip`` want them, zeroed when the request starts.  Nothing is kept per token, so the layer owns no cache
pages.  All seven projections are one product in the activation type; unit norms, beta, the decay, S, the output's norm
and the gate are float whatever the activation type.

Tensors (``tensors`` maps the roles "q", "k", "v", "g", "b", "a", "o", "q_conv", "k_conv", "v_conv", "A_log", "dt_bias",
"norm" to full names; by default ``<name>.q_proj.weight`` and so on, ``<name>.q_conv.weight`` [channels, conv],
``<name>.A_log``, ``<name>.dt_bias``, ``<name>.norm.weight``).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, MixerBinding, register_part
from .ffn import concat_weights
from .plan import ParamSpec, StateSpec


@register_part("mixer", "gated_delta")
class GatedDeltaRule(Mixer):
    graph_safe = True          # every kernel reads the step's layout from the context's device arrays
    adds_to_stream = True

    def __init__(self, name: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int, conv: int,
                 norm_eps: float, init_std: float = 0.02, tensors: Optional[Mapping[str, str]] = None):
        self.name, self.hidden_size = name, int(hidden_size)
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.head_dim, self.v_head_dim, self.taps, self.norm_eps = int(head_dim), int(v_head_dim), int(conv), float(norm_eps)
        if min(self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.taps) <= 0 or self.n_heads % self.n_kv_heads:
            raise ValueError(f"{name}: heads, kv heads (a divisor of heads), head_dim, v_head_dim and conv must be positive")
        if self.taps > 16:
            raise ValueError(f"{name}: at most 16 taps (got {self.taps})")
        ops.delta_layout(self.head_dim, self.v_head_dim)          # (refuses head sizes the kernel has no layout for)
        self.init_std = init_std
        self.names = {k: f"{name}.{k}_proj.weight" for k in ("q", "k", "v", "g", "b", "a", "o")}
        self.names.update({f"{k}_conv": f"{name}.{k}_conv.weight" for k in "qkv"})
        self.names.update({"A_log": f"{name}.A_log", "dt_bias": f"{name}.dt_bias", "norm": f"{name}.norm.weight"})
        self.names.update(tensors or {})
        self.qk_width = self.n_kv_heads * self.head_dim
        self.v_width = self.n_heads * self.v_head_dim
        self.channels = 2 * self.qk_width + self.v_width                  # what the convolution runs over: q | k | v
        self.conv_floats = self.channels * (self.taps - 1)               # the convolution's part of a state row comes first
        self.w_in = self.w_o = self.conv_w = self.A_log = self.dt_bias = self.norm_w = None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.conv_floats + ops.delta_state_floats(self.n_heads, self.head_dim, self.v_head_dim),), "float32")

    def param_specs(self) -> Dict[str, ParamSpec]:
        nm, H, s = self.names, self.hidden_size, ("normal", self.init_std)
        QK, V, nh = self.qk_width, self.v_width, self.n_heads
        return {
            nm["q"]: ParamSpec((QK, H), s), nm["k"]: ParamSpec((QK, H), s), nm["v"]: ParamSpec((V, H), s),
            nm["g"]: ParamSpec((V, H), s), nm["b"]: ParamSpec((nh, H), s), nm["a"]: ParamSpec((nh, H), s),
            nm["o"]: ParamSpec((H, V), s),
            nm["q_conv"]: ParamSpec((QK, self.taps), ("normal", 0.3)), nm["k_conv"]: ParamSpec((QK, self.taps), ("normal", 0.3)),
            nm["v_conv"]: ParamSpec((V, self.taps), ("normal", 0.3)),
            nm["A_log"]: ParamSpec((nh,), ("uniform", -3.0, 0.5)), nm["dt_bias"]: ParamSpec((nh,), ("uniform", -2.0, 1.0)),
            nm["norm"]: ParamSpec((self.v_head_dim,), ("ones",)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        nm = self.names
        # one product: q | k | v (the convolution's channels, in this order) | gate | beta | decay
        self.w_in = ops.prepare_linear(concat_weights([tensors[nm[p]] for p in ("q", "k", "v", "g", "b", "a")]))
        self.w_o = ops.prepare_linear(tensors[nm["o"]])
        self.conv_w = concat_weights([tensors[nm[p + "_conv"]] for p in "qkv"])
        self.A_log = tensors[nm["A_log"]].float().contiguous()          # float whatever the file holds
        self.dt_bias = tensors[nm["dt_bias"]].float().contiguous()
        self.norm_w = tensors[nm["norm"]]

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_in)

    def forward(self, h, ctx, binding: MixerBinding, sink=None):
        state, t = binding.state, ctx.timer
        if state is None:
            raise ValueError(f"{self.name}: the mixer was given no per-request state")
        C, V, nh = self.channels, self.v_width, self.n_heads
        rows = ops.linear(h, self.w_in)                                 # [T, q | k | v | g | b | a]
        u = ops.causal_conv_silu(rows, C, self.conv_w, None, state, ctx.row_req, ctx.q_start, ctx.q_len, ctx.state_slots)
        if t is not None:
            t.mark("mixer.conv")
        y = ops.delta_rule(u, rows, (C, C + V, C + V + nh), self.A_log, self.dt_bias, self.norm_w, self.norm_eps, nh,
                           self.n_kv_heads, self.head_dim, self.v_head_dim, state, self.conv_floats, ctx.q_start, ctx.q_len,
                           ctx.state_slots, single_tokens=ctx.n_tokens == ctx.n_requests)
        if t is not None:
            t.mark("mixer.scan")
        if sink is not None and ops.adds_into_stream(y.shape[0], self.w_o, sink.norm_weight):
            return ops.linear_into_stream(y, self.w_o, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(y, self.w_o, keep_slices=sink is not None)
