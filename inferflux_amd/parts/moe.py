"""Mixture of experts: a router picks a few small gated feed-forwards per row and weighs their outputs.

    z = W_r h (float), s = sigmoid(z) (or softmax(z) over the experts)
    the experts lie in ``groups`` equal groups of neighbours; a group's score is the sum of its ``group_top`` highest
    s; only experts of the ``keep_groups`` best groups can be chosen; the ``top`` highest s among them are
    out = sum over the chosen e of w_e * W_down[e] (silu(W_gate[e] h) * (W_up[e] h)),
    w_e = s_e, divided by the sum of the chosen s with ``renormalize``, times ``route_scale``

With ``n_identity`` the router has that many outputs more than there are experts with weights: the last ``n_identity`` of
its n_experts + n_identity outputs are identity experts, whose output is the row h itself (times its weight); they take part in
the scores, the softmax and the choice like every other.  With ``choice_bias`` a tensor ``correction`` [n_experts + n_identity]
is added to the scores for the choice alone; the weights stay the scores.  ``activation`` "clamped_swish" with ``limit`` L makes
an expert W_down (g sigmoid(1.702 g) (u + 1)) with g = min(W_gate h, L), u = clamp(W_up h, -L, L); the shared expert has the same
form with ``shared_limit``.

With ``router_bias`` a bias b_r joins the logits, z = W_r h + b_r (it counts for the choice and for the weights).  Scoring
"softmax" with ``renormalize`` is the softmax over the chosen logits alone.  With ``shared_ff`` a further gated feed-forward
of that inner size runs for every row and is added, times sigmoid(w_sg . h) (one number per row) with ``shared_gate``.

Tensors (``<name>.``): router [experts + identity, H] (router.b [experts], correction [experts + identity]), e<j>.gate and e<j>.up [ff, H], e<j>.down [H, ff]; shared.gate,
shared.up, shared.down, shared.sg [1, H]; no other biases.  The experts' matrices are stacked at load into [experts, ff, H]
and [experts, H, ff].

The router and the choice run on the device, and the experts' products read each (row, choice)'s expert from device
memory: the launches of a step depend on its layout alone, so a decode step is captured and replayed like any other.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import FeedForward, register_part
from .ffn import GATED_ACTIVATIONS, SwiGLU
from .plan import ParamSpec


# (row, choice) items of a step from which the experts' products go to the matrix cores, tiles of items of one expert
# against that expert's weights; below, every item streams its expert's weights by itself
GROUPED_MIN_ITEMS = 64


@register_part("ffn", "moe")
class MixtureOfExperts(FeedForward):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, n_experts: int, top: int, ff: int, groups: int = 1, keep_groups: int = 1,
                 group_top: int = 2, scoring: str = "sigmoid", renormalize: bool = False, route_scale: float = 1.0,
                 init_std: float = 0.02, router_bias: bool = False, shared_ff: int = 0, shared_gate: bool = False,
                 n_identity: int = 0, choice_bias: bool = False, activation: str = "silu", limit: Optional[float] = None,
                 shared_limit: Optional[float] = None):
        if scoring not in ("sigmoid", "softmax"):
            raise ValueError(f"{name}: scoring '{scoring}' unknown (sigmoid or softmax)")
        self.n_identity = int(n_identity or 0)
        self.n_routed = int(n_experts) + self.n_identity          # what the router scores: the experts and the identity experts
        if self.n_identity < 0 or (self.n_identity and groups != 1):
            raise ValueError(f"{name}: {n_identity} identity experts (not negative, and not together with groups)")
        if self.n_routed % groups or not 0 < keep_groups <= groups or not 0 < top <= keep_groups * (self.n_routed // groups):
            raise ValueError(f"{name}: top {top} of {self.n_routed} experts in {groups} groups of which {keep_groups} are kept")
        if activation not in GATED_ACTIVATIONS:
            raise ValueError(f"{name}: activation '{activation}' unknown (one of {sorted(GATED_ACTIVATIONS)})")
        self.activation, self.act = activation, GATED_ACTIVATIONS[activation]
        self.limit = float(limit) if limit is not None else 0.0
        if (self.act == ops.ACT_CLAMPED_SWISH) != (self.limit > 0):
            raise ValueError(f"{name}: the activation '{activation}' and a limit of {limit} do not go together")
        self.choice_bias, self.correction = bool(choice_bias), None
        self.name, self.hidden_size = name, int(hidden_size)
        self.n_experts, self.top, self.ff = int(n_experts), int(top), int(ff)
        self.groups, self.keep_groups, self.group_top = int(groups), int(keep_groups), int(group_top)
        self.scoring, self.renormalize, self.route_scale, self.init_std = scoring, bool(renormalize), float(route_scale), init_std
        self.router = self.gate = self.up = self.down = None
        self.router_bias, self.bias = bool(router_bias), None
        self.shared_gate, self.shared_gate_w = bool(shared_gate), None
        self.shared = None
        if shared_ff:
            n = f"{name}.shared"
            self.shared = SwiGLU(n, hidden_size, int(shared_ff), init_std, activation,
                                 {"gate": f"{n}.gate", "up": f"{n}.up", "down": f"{n}.down"},
                                 limit=(shared_limit if shared_limit is not None else limit) if self.limit > 0 else None)
        elif shared_gate:
            raise ValueError(f"{name}: a gate on a shared expert that does not exist")

    def children(self):
        return (self.shared,) if self.shared is not None else ()

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, H, s = self.name, self.hidden_size, ("normal", self.init_std)
        out = {f"{n}.router": ParamSpec((self.n_routed, H), s)}
        if self.choice_bias:
            out[f"{n}.correction"] = ParamSpec((self.n_routed,), ("normal", 0.01))
        for e in range(self.n_experts):
            out[f"{n}.e{e}.gate"] = ParamSpec((self.ff, H), s)
            out[f"{n}.e{e}.up"] = ParamSpec((self.ff, H), s)
            out[f"{n}.e{e}.down"] = ParamSpec((H, self.ff), s)
        if self.router_bias:
            out[f"{n}.router.b"] = ParamSpec((self.n_routed,), s)
        if self.shared_gate:
            out[f"{n}.shared.sg"] = ParamSpec((1, H), s)
        return out

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.name
        mats = [tensors[f"{n}.e{e}.{p}"] for e in range(self.n_experts) for p in ("gate", "up", "down")] + [tensors[f"{n}.router"]]
        dtype = mats[0].dtype if len({m.dtype for m in mats}) == 1 else torch.float32     # mixed storage is widened
        stack = lambda p: torch.stack([tensors[f"{n}.e{e}.{p}"].to(dtype) for e in range(self.n_experts)]).contiguous()
        self.gate, self.up, self.down = stack("gate"), stack("up"), stack("down")
        self.router = ops.prepare_linear(tensors[f"{n}.router"].to(dtype).contiguous())     # (steps of many rows take its product from ``linear``)
        if self.gate.is_cuda and ops.grouped_takes(dtype, self.hidden_size, self.ff):
            # one tensor that both products read: rows of gate and up in turns of 16
            self.gate, self.up = ops.pair_gate_up(self.gate, self.up), None

        if self.router_bias:
            self.bias = tensors[f"{n}.router.b"].float().contiguous()        # the router is float whatever the file holds
        if self.choice_bias:
            self.correction = tensors[f"{n}.correction"].float().contiguous()
        if self.shared_gate:
            self.shared_gate_w = tensors[f"{n}.shared.sg"].to(dtype).reshape(-1).contiguous()

    def route(self, h):
        return ops.moe_route(h, self.router, self.top, self.groups, self.keep_groups, self.group_top,
                             self.scoring == "softmax", self.renormalize, self.route_scale, self.bias, self.correction)

    def _with_shared(self, out, x, ctx):
        """The chosen experts' sum plus the shared expert's output (times its gate of one number per row)."""
        if self.shared is None:
            return out
        extra = self.shared.forward(x, ctx)
        return ops.gated_add(out, extra, x, self.shared_gate_w if self.shared_gate else None)     # (one kernel, also for partial sums)

    def forward(self, h, ctx):
        x = h if h.dtype == self.router.dtype else h.to(self.router.dtype)
        ids, weights = self.route(x)
        if ctx.timer is not None:
            ctx.timer.mark("ffn.route")
        if self.up is None and x.shape[0] * self.top >= GROUPED_MIN_ITEMS:
            return self._with_shared(ops.moe_experts_grouped(x, self.gate, self.down, ids, weights, self.act, self.limit,
                                                             self.n_identity), x, ctx)      # (partial sums, one per choice)
        out = self._with_shared(ops.moe_experts(x, self.gate, self.up, self.down, ids, weights, self.act, self.limit,
                                                self.n_identity), x, ctx)
        return out if out.dtype == h.dtype else out.to(h.dtype)
