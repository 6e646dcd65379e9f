"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases; act is silu ("SwiGLU", the default) or the tanh form
of gelu, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).  "clamped_swish" with its ``limit`` L is another form of the
inner part: g = min(gate(x), L), u = clamp(up(x), -L, L), down( g sigmoid(1.702 g) (u + 1) ).

g = h Wg^T, u = h Wu^T, a = g / (1 + exp(-g)) * u in float, delta = a Wd^T
(runtime/backends/cuda/native/transformer_forward.cu:2383-2419, 2487-2494, 2528-2547;
cuda_kernels.cu:139-151).  The reference runs gate and up as two products; here the two
matrices are merged at load time into one [2I, H] matrix whose rows alternate gate_i, up_i, so
that one product yields both and the kernel that holds a gate value also holds its up value
(the activation is then the product's epilogue).  This changes nothing in the arithmetic of
any output element.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import FeedForward, register_part
from .plan import ParamSpec


def concat_weights(parts):
    """Stack matrices along the output axis; mixed storage types are widened to float32."""
    if len({p.dtype for p in parts}) > 1:
        parts = [p.float() for p in parts]
    return torch.cat(list(parts), dim=0).contiguous()


ACTIVATIONS = {"silu": ops.ACT_SILU, "gelu_tanh": ops.ACT_GELU_TANH}
GATED_ACTIVATIONS = {**ACTIVATIONS, "clamped_swish": ops.ACT_CLAMPED_SWISH}      # (the last one takes a limit)


@register_part("ffn", "gated_ffn")
@register_part("ffn", "swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, intermediate_size: int, init_std: float = 0.02,
                 activation: str = "silu", tensors: Optional[Mapping[str, str]] = None, limit: Optional[float] = None):
        """``activation``: "silu", "gelu_tanh" or "clamped_swish" (with its ``limit``).  ``tensors``: the full names of
        "gate", "up" and "down" in the model file where they are not ``<name>.gate_proj.weight`` and so on."""
        self.name, self.hidden_size, self.intermediate_size = name, int(hidden_size), int(intermediate_size)
        self.init_std = init_std
        if activation not in GATED_ACTIVATIONS:
            raise ValueError(f"{name}: activation '{activation}' unknown (one of {sorted(GATED_ACTIVATIONS)})")
        self.activation, self.act = activation, GATED_ACTIVATIONS[activation]
        self.limit = float(limit) if limit is not None else 0.0
        if (self.act == ops.ACT_CLAMPED_SWISH) != (self.limit > 0):
            raise ValueError(f"{name}: the activation '{activation}' and a limit of {limit} do not go together")
        self.names = {k: f"{name}.{k}_proj.weight" for k in ("gate", "up", "down")}
        self.names.update(tensors or {})
        self.w_gate_up = None
        self.w_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, I, s = self.hidden_size, self.intermediate_size, ("normal", self.init_std)
        return {
            self.names["gate"]: ParamSpec((I, H), s),
            self.names["up"]: ParamSpec((I, H), s),
            self.names["down"]: ParamSpec((H, I), s),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = ops.prepare_linear(
            torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous())
        self.w_down = ops.prepare_linear(tensors[self.names["down"]])

    adds_to_stream = True

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_gate_up)

    def forward(self, h, ctx, sink=None):
        a = ops.linear_swiglu(h, self.w_gate_up, self.act, self.limit)
        if ctx.timer is not None:
            ctx.timer.mark("ffn.gate_up")
        if sink is not None and ops.adds_into_stream(a.shape[0], self.w_down, sink.norm_weight):
            return ops.linear_into_stream(a, self.w_down, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(a, self.w_down, keep_slices=sink is not None)   # an RMS norm's kernel adds partial sums itself


@register_part("ffn", "dense_ffn")
class DenseFFN(FeedForward):
    """A feed-forward without a gate: down( act(up(x)) ), no biases; act is "gelu_tanh" (the default) or "silu", formed in
    float.  ``tensors``: the full names of "up" and "down" where they are not ``<name>.up_proj.weight`` and so on."""
    graph_safe = True
    adds_to_stream = True

    def __init__(self, name: str, hidden_size: int, intermediate_size: int, init_std: float = 0.02,
                 activation: str = "gelu_tanh", tensors: Optional[Mapping[str, str]] = None):
        self.name, self.hidden_size, self.intermediate_size = name, int(hidden_size), int(intermediate_size)
        self.init_std = init_std
        if activation not in ACTIVATIONS:
            raise ValueError(f"{name}: activation '{activation}' unknown (one of {sorted(ACTIVATIONS)})")
        self.activation, self.act = activation, ACTIVATIONS[activation]
        self.names = {k: f"{name}.{k}_proj.weight" for k in ("up", "down")}
        self.names.update(tensors or {})
        self.w_up = self.w_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, I, s = self.hidden_size, self.intermediate_size, ("normal", self.init_std)
        return {self.names["up"]: ParamSpec((I, H), s), self.names["down"]: ParamSpec((H, I), s)}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_up = ops.prepare_linear(tensors[self.names["up"]])
        self.w_down = ops.prepare_linear(tensors[self.names["down"]])

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_up)

    def forward(self, h, ctx, sink=None):
        a = ops.linear_act(h, self.w_up, self.act)
        if ctx.timer is not None:
            ctx.timer.mark("ffn.up")
        if sink is not None and ops.adds_into_stream(a.shape[0], self.w_down, sink.norm_weight):
            return ops.linear_into_stream(a, self.w_down, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(a, self.w_down, keep_slices=sink is not None)
