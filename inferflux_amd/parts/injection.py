"""What is fed into the residual stream between layers, apart from the layers' own outputs.

"pass_input" is the input of one pass of a span of layers that runs several times with the same weights: before the
pass's first layer the stream x becomes

    x + e (only with ``add_embedding``: e is the embedding's output, x as it was before the first layer) + step[index]

with ``step`` a tensor [times, H] that gives every pass a learned vector of its own.  A plan has one such part for every pass
(they share the tensor) and names it in the schedule entry of the pass's first layer.  One kernel, in float.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Injection, register_part
from .plan import ParamSpec


@register_part("injection", "pass_input")
class PassInput(Injection):
    graph_safe = True

    def __init__(self, hidden_size: int, index: int, times: int, tensor: Optional[str] = None, add_embedding: bool = False,
                 init_std: float = 0.02):
        self.hidden_size, self.index, self.times = int(hidden_size), int(index), int(times)
        if not 0 <= self.index < self.times:
            raise ValueError(f"pass_input: pass {index} of {times}")
        self.tensor, self.needs_embedding, self.init_std = tensor, bool(add_embedding), init_std
        self.vec: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor: ParamSpec((self.times, self.hidden_size), ("normal", self.init_std))} if self.tensor else {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        if self.tensor:
            self.vec = tensors[self.tensor][self.index].contiguous()

    def forward(self, residual, ctx, embedded) -> None:
        if not isinstance(residual, torch.Tensor):
            raise ValueError("pass_input: the stream it is given is not one float32 stream")
        if self.needs_embedding and embedded is None:
            raise ValueError("pass_input: the embedding's output was not kept for this step")
        ops.stream_add(residual, embedded if self.needs_embedding else None, self.vec)
