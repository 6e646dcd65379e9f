"""Position encodings applied to queries and keys before the cache write.

A position part hands the mixer what its fused kernel needs: ``kernel_args(ctx)`` returns
(style, rotary_dim, cos, sin), the last two being the step's table [T, rotary_dim / 2] of
angle = float(position) * inv_freq[p], computed in float once per step and shared by every
layer with the same constants.  The kernel rotates pair p of every head by it.  A position part
that cannot be expressed this way sets ``needs_apply`` and implements ``apply(q, k, positions)``.

Rotary, split-half ("NeoX") pairing as the reference applies it to qwen2
(runtime/backends/cuda/native/model_loader.h:39-61 chooses the pairing;
cuda_kernels.cu:71-117): pair p joins elements p and p + d/2, f_p = 1 / theta^(2p/d),
(x_p, x_{p+d/2}) <- (x_p cos a - x_{p+d/2} sin a, x_p sin a + x_{p+d/2} cos a).  The reference
evaluates powf per element; here the d/2 frequencies are computed once in double precision
and rounded to float.

Frequencies scaled for contexts longer than the model was trained on ("YaRN", ``scaling`` = factor, original, fast,
slow): with dim(t) = dims ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)),
dims - 1) and ramp_p = clamp((p - lo) / max(hi - lo, 0.001), 0, 1), pair p turns with f_p / factor * ramp_p +
f_p (1 - ramp_p): the fast pairs keep their frequency, the slow ones are stretched by the factor, and cos and sin are
both multiplied by 0.1 ln(factor) + 1.

Frequencies scaled in bands of wavelength (``scaling`` = factor, original, low, high): with l_p = 2 pi / f_p, a pair with
l_p < original / high keeps f_p; one with l_p > original / low turns with f_p / factor; between the two, with
s = (original / l_p - low) / (high - low), it turns with (1 - s) f_p / factor + s f_p.  cos and sin keep their size.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from ..kernels import ops
from .base import Part, register_part


class PositionEncoding(Part):
    def kernel_args(self, ctx) -> Tuple[int, int, Optional[torch.Tensor], Optional[torch.Tensor]]:
        return ops.ROPE_NONE, 0, None, None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], positions: torch.Tensor):
        """Transform q [T, nH, d] and k [T, nKV, d] (or None) outside the fused kernel."""
        return q, k

    needs_apply = False


@register_part("position", "none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim


@register_part("position", "rotary")
class RotaryPosition(PositionEncoding):
    graph_safe = True

    """``style``: "split_half" pairs (p, p + rot/2); "consecutive" pairs (2p, 2p+1)."""

    STYLES = {"split_half": ops.ROPE_SPLIT_HALF, "consecutive": ops.ROPE_CONSECUTIVE}

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None, style: str = "split_half",
                 scaling: Optional[dict] = None):
        """``scaling``: None, {"factor", "original", "fast", "slow"} (a ramp over the pairs) or {"factor", "original", "low",
        "high"} (bands of wavelength); see the module's text."""
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.theta = float(theta)
        if style not in self.STYLES:
            raise ValueError(f"rotary style '{style}' unknown (one of {sorted(self.STYLES)})")
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.style = style
        self.scaling = None
        self.magnitude = 1.0
        self.bands = bool(scaling) and ("low" in scaling or "high" in scaling)
        if self.bands:
            missing = [k for k in ("factor", "original", "low", "high") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling in bands needs {missing}")
            self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "low", "high")}
            if self.scaling["factor"] <= 0 or self.scaling["original"] <= 0 or not 0 < self.scaling["low"] < self.scaling["high"]:
                raise ValueError(f"rotary scaling: factor and original must be positive and 0 < low < high, got {self.scaling}")
        elif scaling:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling needs {missing}")
            self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "fast", "slow")}
            if self.scaling["factor"] <= 0 or self.scaling["original"] <= 0 or self.scaling["fast"] <= 0 or self.scaling["slow"] <= 0:
                raise ValueError(f"rotary scaling: factor, original, fast and slow must be positive, got {self.scaling}")
            self.magnitude = 0.1 * math.log(self.scaling["factor"]) + 1.0
        self._inv_freq = {}

    def frequencies(self) -> torch.Tensor:
        """The pairs' frequencies in double precision."""
        n = self.rotary_dim // 2
        p = torch.arange(n, dtype=torch.float64)
        f = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), 2.0 * p / self.rotary_dim)
        if self.scaling is None:
            return f
        sc, dims = self.scaling, self.rotary_dim
        if self.bands:
            wavelength = 2.0 * math.pi / f
            s = torch.clamp((sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"]), 0.0, 1.0)
            blended = (1.0 - s) * f / sc["factor"] + s * f
            return torch.where(wavelength < sc["original"] / sc["high"], f,
                               torch.where(wavelength > sc["original"] / sc["low"], f / sc["factor"], blended))
        dim_of = lambda turns: dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
        ramp = torch.clamp((p - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / sc["factor"] * ramp + f * (1.0 - ramp)

    def inv_freq(self, device) -> torch.Tensor:
        key = str(device)
        t = self._inv_freq.get(key)
        if t is None:
            t = self.frequencies().to(torch.float32).to(device)
            self._inv_freq[key] = t
        return t

    def kernel_args(self, ctx):
        key = ("rotary_table", self.theta, self.rotary_dim, tuple(sorted(self.scaling.items())) if self.scaling else None)
        cos, sin = ctx.derived(key, lambda: ops.rope_table(ctx.positions, self.inv_freq(ctx.device), self.magnitude))
        return self.STYLES[self.style], self.rotary_dim, cos, sin
