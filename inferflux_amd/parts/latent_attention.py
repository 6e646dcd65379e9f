"""Attention through a latent: queries, keys and values are projected down to narrow latents first, and only the
key/value latent and one shared rotated key part are cached.

With H heads of ``dim`` unrotated and ``rot_dim`` rotated query/key dimensions, values of ``vdim``, a query latent of
``q_rank`` and a key/value latent of ``kv_rank``:

    c_q = rmsnorm(W_dq h) * g_q              q   = W_uq c_q, per head [q_n (dim) | q_r (rot_dim)]
    c   = rmsnorm((W_dkv h)[:kv_rank]) * g_kv      k_r = (W_dkv h)[kv_rank:], one for all heads
    per head: k_n = W_uk c, v = W_uv c
    score(i, j) = (q_n(i) . k_n(j) + rot(q_r(i), i) . rot(k_r(j), j)) * scale,  j <= i (and within the window)
    out = W_o [softmax-weighted sums of v, head by head]

Neither k_n nor v is ever formed.  Since q_n . (W_uk c) = (W_uk^T q_n) . c, a head's query becomes
[W_uk^T q_n | rot(q_r)] (kv_rank + rot_dim wide) and scores against the cached row [c | rot(k_r)], which all heads
share; the weighted sum is taken over c itself and W_uv is applied to it afterwards.  To the paged attention kernels
this is attention with one kv head whose keys are kv_rank + rot_dim and whose values kv_rank wide, so the cache, its
pages, windows and block tables are those of every other attention layer (``CacheSpec`` with ``v_head_dim``), and a
step's rows may be prompt portions and decoded tokens alike.

Without a query latent (``q_rank`` None) the queries are one product of the mixer's input, q = W_q h (tensor ``q``
[heads (dim + rot_dim), H]).  With ``sinks`` every head has a learned score (tensor ``sink`` [heads]) that joins its
softmax's denominator as a key without value: p_j = exp(s_j) / (exp(sink_h) + sum_j exp(s_j)).  ``pairing`` says which
elements of the rotated parts the position part's rotation pairs: "split_half" (p, p + dims / 2), as the kernels turn
them, or "interleaved" (2p, 2p + 1); for the latter the rows of the weights that produce the rotated parts are reordered
at load so that pair (2p, 2p + 1) lies at (p, p + dims / 2), which leaves every score as it was since queries and keys are
reordered alike.

Tensors (``<name>.``): dq [q_rank, H], dq.norm [q_rank], uq [heads (dim + rot_dim), q_rank], dkv [kv_rank + rot_dim, H],
dkv.norm [kv_rank], uk [heads dim, kv_rank], uv [heads vdim, kv_rank], o [H, heads vdim].  The two down projections
are one product (their weights are stacked at load), and W_uk is kept transposed per head.

Norms, rotation angles, scores and softmax are computed in float whatever the activation type.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import Mixer, MixerBinding, build_part, register_part
from .ffn import concat_weights
from .plan import CacheSpec, ParamSpec, PartSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, n_heads: int, dim: int, rot_dim: int, v_dim: int, q_rank: Optional[int],
                 kv_rank: int, scale: float, eps: float, position: PartSpec, window: Optional[int] = None,
                 init_std: float = 0.02, sinks: bool = False, pairing: str = "split_half"):
        self.name, self.hidden_size = name, int(hidden_size)
        self.n_heads, self.dim, self.rot_dim, self.v_dim = int(n_heads), int(dim), int(rot_dim), int(v_dim)
        self.q_rank, self.kv_rank = int(q_rank or 0), int(kv_rank)
        if pairing not in ("split_half", "interleaved"):
            raise ValueError(f"{name}: pairing '{pairing}' unknown (split_half or interleaved)")
        self.sinks, self.pairing, self.sink_scores = bool(sinks), pairing, None
        self.scale, self.eps, self.init_std = float(scale), float(eps), init_std
        self.window = int(window) if window else None
        self.position = build_part("position", position)
        if self.position.needs_apply:
            raise ValueError(f"{name}: latent attention needs a position part that gives the kernels a rotation table")
        self.w_down = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = self.q_norm = self.kv_norm = None

    @property
    def value_width(self) -> int:
        """Width of a cached value.  The latent's, unless the matrix-core attention kernels take the key's size (they
        are written for values as wide as keys): then the rotated key part is stored behind the latent on the value
        side too, rot_dim / (kv_rank + rot_dim) more bytes and products on that side, and what comes back behind a
        head's kv_rank sums is left unread."""
        d = self.kv_rank + self.rot_dim
        return d if (d % 16 == 0 and d <= ops.MFMA_MAX_HEAD_DIM) else self.kv_rank

    def cache_spec(self) -> CacheSpec:
        d, dv = self.kv_rank + self.rot_dim, self.value_width
        return CacheSpec(1, d, self.window, dv if dv != d else None)

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, H, s = self.name, self.hidden_size, ("normal", self.init_std)
        nh, d, r, dv = self.n_heads, self.dim, self.rot_dim, self.v_dim
        if self.q_rank:
            out = {f"{n}.dq": ParamSpec((self.q_rank, H), s), f"{n}.dq.norm": ParamSpec((self.q_rank,), ("ones",)),
                   f"{n}.uq": ParamSpec((nh * (d + r), self.q_rank), s)}
        else:
            out = {f"{n}.q": ParamSpec((nh * (d + r), H), s)}
        if self.sinks:
            out[f"{n}.sink"] = ParamSpec((nh,), ("normal", 1.0))
        return {
            **out,
            f"{n}.dkv": ParamSpec((self.kv_rank + r, H), s), f"{n}.dkv.norm": ParamSpec((self.kv_rank,), ("ones",)),
            f"{n}.uk": ParamSpec((nh * d, self.kv_rank), s), f"{n}.uv": ParamSpec((nh * dv, self.kv_rank), s),
            f"{n}.o": ParamSpec((H, nh * dv), s),
        }

    def _pair_order(self, device) -> torch.Tensor:
        """Where each element of a rotated part comes from so that the pairs (2p, 2p + 1) of the first ``dims`` elements lie
        at (p, p + dims / 2); the elements behind them stay."""
        dims = self.position.rotary_dim
        idx = list(range(0, dims, 2)) + list(range(1, dims, 2)) + list(range(dims, self.rot_dim))
        return torch.tensor(idx, dtype=torch.long, device=device)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n, nh = self.name, self.n_heads
        w_q, w_dkv = tensors[f"{n}.uq" if self.q_rank else f"{n}.q"], tensors[f"{n}.dkv"]
        if self.pairing == "interleaved":
            order = self._pair_order(w_q.device)
            w_q = w_q.view(nh, self.dim + self.rot_dim, -1)
            w_q = torch.cat([w_q[:, :self.dim], w_q[:, self.dim:][:, order]], dim=1).reshape(nh * (self.dim + self.rot_dim), -1).contiguous()
            w_dkv = torch.cat([w_dkv[:self.kv_rank], w_dkv[self.kv_rank:][order]], dim=0).contiguous()
        if self.q_rank:
            self.w_down = ops.prepare_linear(concat_weights([tensors[f"{n}.dq"], w_dkv]))
        else:
            self.w_down = ops.prepare_linear(w_dkv)
        self.w_uq = ops.prepare_linear(w_q)
        if self.sinks:
            self.sink_scores = tensors[f"{n}.sink"].float().contiguous()        # scores are float whatever the file holds
        self.w_o = ops.prepare_linear(tensors[f"{n}.o"])
        dtype = self.w_uq.dtype
        # per head [kv_rank, dim]: the product that moves W_uk over to the query's side
        self.w_uk_t = tensors[f"{n}.uk"].to(dtype).view(nh, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[f"{n}.uv"].to(dtype).view(nh, self.v_dim, self.kv_rank).contiguous()
        norms = [tensors[f"{n}.dq.norm"] if self.q_rank else None, tensors[f"{n}.dkv.norm"]]
        if self.q_rank and norms[0].dtype != norms[1].dtype:
            norms = [w.float() for w in norms]
        self.q_norm, self.kv_norm = norms

    def forward(self, h, ctx, binding: MixerBinding):
        cache = binding.cache
        T, nh, t = h.shape[0], self.n_heads, ctx.timer
        _, rot_dims, cos, sin = self.position.kernel_args(ctx)
        slots = ctx.write_slots(cache.group) if binding.writes_cache else None
        y = ops.linear(h, self.w_down, keep_slices=True)              # [T, q_rank + kv_rank + rot_dim]
        cq = ops.latent_finish(y, self.q_norm, self.kv_norm, self.eps, cos, sin, rot_dims, slots, self.q_rank, self.kv_rank,
                               self.rot_dim, cache.k, cache.v, cache.page_size, h.dtype)
        q = ops.linear(cq if self.q_rank else h, self.w_uq)           # [T, heads (dim + rot_dim)]
        w_dtype = self.w_uk_t.dtype
        qa = ops.headwise(q if q.dtype == w_dtype else q.to(w_dtype), self.w_uk_t, nh, self.dim + self.rot_dim, self.rot_dim,
                          cos, sin, rot_dims)                         # [T, heads, kv_rank + rot_dim]
        if t is not None:
            t.mark("mixer.qkv")
        a = paged_attention(qa if qa.dtype == h.dtype else qa.to(h.dtype), cache, ctx, self.window, self.scale,
                            sinks=self.sink_scores)                    # [T, heads value_width]
        if t is not None:
            t.mark("mixer.attention")
        v = ops.headwise(a if a.dtype == w_dtype else a.to(w_dtype), self.w_uv, nh, self.value_width)    # [T, heads, vdim]
        v = v.view(T, nh * self.v_dim)
        return ops.linear(v if v.dtype == h.dtype else v.to(h.dtype), self.w_o, keep_slices=True)
