"""Grouped-query attention over the paged cache, with q/k/v bias, a position part and an
optional window.

Reference order (runtime/backends/cuda/native/transformer_forward.cu:1944-2135, 2145-2241):
q, k, v = h Wq^T + bq, h Wk^T + bk, h Wv^T + bv; position encoding of q and k; k and v are
written to the cache at the token's position; causal attention of head h over kv head
h / (nH / nKV) with scale 1/sqrt(d) applied after the dot product; delta = attn Wo^T.
The three projections are concatenated at load time into one [(nH + 2 nKV) d, H] product;
the bias is added in float inside the rotary kernel (the reference rounds the product to the
activation type first and adds the bias afterwards, cuda_kernels.cu:518-527).

An execution that reads another entry's cache (binding.writes_cache False) projects and
encodes only its queries.

Optional mechanisms, each a constructor argument that is off by default:
  ``keep_first``      a windowed query at position i also sees the request's first ``keep_first`` positions, at their true
                      places: j <= i and (i - j < window or j < keep_first); the cache keeps their pages.
  ``sink``            a key without value with this score joins the softmax's denominator: p_j = exp(s_j) /
                      (exp(sink) + sum_j exp(s_j)); with 0 that is "one added to the denominator".
  ``unit_norm_eps``   after the rotation every q and k head is divided by its root mean square (eps inside the root; an
                      RMS norm without weight).
  ``output_gate``     True: head h's output is multiplied by sigmoid(W_g x)_h before the output projection (W_g [heads, H], a
                      further block of rows of the fused projection).  "elementwise": the concatenated heads are multiplied
                      element by element with sigmoid(W_g x) (W_g [heads * v_head_dim, H]).
  ``qk_norm_eps``     before the rotation every q and k head becomes x / sqrt(mean(x^2) + eps) * w, with one weight of
                      head_dim for all q heads ("q_norm") and one for all k heads ("k_norm").
  ``value_mix``       "source": this layer hands the step's values (as projected) on to the layers after it; "mix": this
                      layer caches v <- (1 - lambda) v + lambda v_source instead of its own, lambda a scalar tensor.  The
                      layers must agree in kv heads and value width.
  ``chunk``           the sequence is cut into blocks of this many positions counted from its start, and a query sees only
                      the keys of its own block: j <= i and j // chunk == i // chunk.  The cache keeps a window of ``chunk``
                      positions (a block never reaches further back).
  ``differential``    {"diff": c, "eps": e}: differential attention.  Every query head and kv head holds two vectors of
                      ``head_dim`` elements, laid out one after the other; each pair is a softmax map of its own over the
                      same values a_1, a_2, and the head's output is o = a_1 - lambda a_2 with lambda =
                      exp(lq1 . lk1) - exp(lq2 . lk2) + c (four tensors of head_dim, one lambda for the layer), then
                      o / sqrt(mean(o^2) + e) over the head's values, times (1 - c).  Needs a position part that leaves q
                      and k alone.
  ``tensors``         full names of the tensors in the model file ("q", "k", "v", "o", "q_bias", "k_bias", "v_bias", "gate",
                      "mix", "q_norm", "k_norm", "lq1", "lk1", "lq2", "lk2") where they are not ``<name>.q_proj.weight`` and so on.
"""
from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import Mixer, MixerBinding, build_part, register_part
from .position import PositionEncoding
from .ffn import concat_weights
from .plan import CacheSpec, ParamSpec, PartSpec


@register_part("mixer", "paged_attention")
class PagedAttention(Mixer):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PartSpec, bias: bool = True, window: Optional[int] = None,
                 scale: Optional[float] = None, init_std: float = 0.02, v_head_dim: Optional[int] = None,
                 keep_first: int = 0, sink: Optional[float] = None, unit_norm_eps: Optional[float] = None,
                 output_gate=False, value_mix: Optional[str] = None, tensors: Optional[Mapping[str, str]] = None,
                 qk_norm_eps: Optional[float] = None, chunk: Optional[int] = None, differential: Optional[Mapping[str, float]] = None):
        """``v_head_dim``: the width of a value head where it differs from ``head_dim`` (such a layer runs on the
        kernels that take both widths: the plain attention kernel and the unfused projection path)."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{name}: {n_heads} query heads are not a multiple of {n_kv_heads} kv heads")
        self.name, self.hidden_size = name, int(hidden_size)
        self.chunk = int(chunk) if chunk else None
        self.differential = None
        self.map_dim = int(head_dim)                   # elements of one map's query or key
        if differential is not None:
            self.differential = (float(differential["diff"]), float(differential["eps"]))
            head_dim = 2 * int(head_dim)               # to the projection, the row kernel and the cache a head is both maps' vectors
        if v_head_dim is None and differential is not None:
            v_head_dim = self.map_dim
        self.n_heads, self.n_kv_heads, self.head_dim = int(n_heads), int(n_kv_heads), int(head_dim)
        self.v_head_dim = int(v_head_dim) if v_head_dim else self.head_dim
        self.bias, self.window, self.init_std = bool(bias), (int(window) if window else None), init_std
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.map_dim)
        self.position = build_part("position", position)
        self.keep_first = max(int(keep_first or 0), 0) if self.window else 0
        self.sink = None if sink is None else float(sink)
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        if output_gate not in (False, True, None, "head", "elementwise"):
            raise ValueError(f"{name}: output_gate '{output_gate}' unknown (False, True or 'elementwise')")
        self.output_gate = bool(output_gate)
        self.gate_elementwise = output_gate == "elementwise"
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.q_norm_w = self.k_norm_w = None
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"{name}: value_mix '{value_mix}' unknown (None, 'source' or 'mix')")
        self.value_mix, self.mix_weight = value_mix, 0.0
        self.names = {"q": f"{name}.q_proj.weight", "k": f"{name}.k_proj.weight", "v": f"{name}.v_proj.weight",
                      "o": f"{name}.o_proj.weight", "q_bias": f"{name}.q_proj.bias", "k_bias": f"{name}.k_proj.bias",
                      "v_bias": f"{name}.v_proj.bias", "gate": f"{name}.gate.weight", "mix": f"{name}.value_mix",
                      "q_norm": f"{name}.q_norm.weight", "k_norm": f"{name}.k_norm.weight",
                      "lq1": f"{name}.lambda_q1", "lk1": f"{name}.lambda_k1", "lq2": f"{name}.lambda_q2", "lk2": f"{name}.lambda_k2"}
        self.names.update(tensors or {})
        # (what the kernels fused for the plain case do not do: then the projection, the row kernel and attention run one by one)
        self._extras = (self.unit_norm_eps is not None or self.output_gate or self.value_mix is not None
                        or self.qk_norm_eps is not None or self.chunk is not None or self.differential is not None)
        if self.differential is not None and (self.unit_norm_eps is not None or self.qk_norm_eps is not None
                                              or self.position.kernel_args.__func__ is not PositionEncoding.kernel_args):
            raise ValueError(f"{name}: differential attention takes no norms on q and k and a position part that leaves them alone")
        self.lam = 0.0
        self.w_qkv = self.b_qkv = self.w_o = self._w_q = None

    @property
    def gate_rows(self) -> int:
        """Rows of the gate's weight: one per head, or one per element of the concatenated heads."""
        if not self.output_gate:
            return 0
        return self.n_heads * self.v_head_dim if self.gate_elementwise else self.n_heads

    def cache_spec(self) -> CacheSpec:
        window = self.window
        if self.chunk is not None:             # a block's query never reads further back than the block is long
            window = min(window, self.chunk) if window else self.chunk
        return CacheSpec(self.n_kv_heads, self.head_dim, window,
                         self.v_head_dim if self.v_head_dim != self.head_dim else None, self.keep_first)

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, d, dv, s = self.hidden_size, self.head_dim, self.v_head_dim, ("normal", self.init_std)
        nm = self.names
        out = {
            nm["q"]: ParamSpec((self.n_heads * d, H), s),
            nm["k"]: ParamSpec((self.n_kv_heads * d, H), s),
            nm["v"]: ParamSpec((self.n_kv_heads * dv, H), s),
            nm["o"]: ParamSpec((H, self.n_heads * dv), s),
        }
        if self.bias:
            out[nm["q_bias"]] = ParamSpec((self.n_heads * d,), s)
            out[nm["k_bias"]] = ParamSpec((self.n_kv_heads * d,), s)
            out[nm["v_bias"]] = ParamSpec((self.n_kv_heads * dv,), s)
        if self.output_gate:
            out[nm["gate"]] = ParamSpec((self.gate_rows, H), s)
        if self.qk_norm_eps is not None:
            out[nm["q_norm"]] = ParamSpec((d,), ("ones",))
            out[nm["k_norm"]] = ParamSpec((d,), ("ones",))
        if self.differential is not None:
            for k in ("lq1", "lk1", "lq2", "lk2"):
                out[nm[k]] = ParamSpec((self.map_dim,), ("normal", 0.1))
        if self.value_mix is not None:       # (the source layer's tensor is in the file too, where the file has it; nothing reads it)
            out[nm["mix"]] = ParamSpec((), ("uniform", 0.2, 0.8), optional=self.value_mix == "source")
        return out

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        nm = self.names
        blocks = [tensors[nm[p]] for p in "qkv"] + ([tensors[nm["gate"]]] if self.output_gate else [])
        self.w_qkv = self._prepare_qkv(concat_weights(blocks), self.n_heads + 2 * self.n_kv_heads)
        self.b_qkv = None
        if self.bias:
            biases = [tensors[nm[p + "_bias"]] for p in "qkv"]
            if self.output_gate:
                biases.append(torch.zeros(self.gate_rows, dtype=biases[0].dtype, device=biases[0].device))
            self.b_qkv = concat_weights(biases)
        self.w_o = ops.prepare_linear(tensors[nm["o"]])
        if self.value_mix == "mix":
            self.mix_weight = float(tensors[nm["mix"]].float().item())
        if self.qk_norm_eps is not None:
            self.q_norm_w, self.k_norm_w = tensors[nm["q_norm"]], tensors[nm["k_norm"]]
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.q_norm_w, self.k_norm_w = self.q_norm_w.float(), self.k_norm_w.float()
        if self.differential is not None:      # one number for the layer, formed once in double precision
            dot = lambda a, b: float((tensors[nm[a]].double() * tensors[nm[b]].double()).sum().item())
            self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.differential[0]
        self._w_q = None

    def _prepare_qkv(self, weight: torch.Tensor, heads: int):
        """The projection's weight with its decode copy; for head sizes that are multiples of 32 the copy's
        row tiles are ordered so that the fused projection + rotation kernel finds both halves of a rotation
        pair in one lane (plain products read the same copy through the order)."""
        order = None
        if (self.head_dim % 32 == 0 and self.v_head_dim == self.head_dim and weight.is_cuda and weight.dtype == torch.bfloat16
                and not self._extras):
            order = torch.tensor(ops.pair_tile_order(heads, self.head_dim), dtype=torch.int32, device=weight.device)
        return ops.prepare_linear(weight, order)

    adds_to_stream = True

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return not self.position.needs_apply and ops.takes_scaled_rows(n_rows, self.w_qkv)

    def _project_out(self, out, sink):
        if sink is not None and ops.adds_into_stream(out.shape[0], self.w_o, sink.norm_weight):
            return ops.linear_into_stream(out, self.w_o, sink.stream, sink.norm_weight, sink.eps, sink.mult)
        return ops.linear(out, self.w_o, keep_slices=sink is not None)   # an RMS norm's kernel adds partial sums itself

    def _attend(self, q, cache, ctx, gate=None):
        if self.differential is None:
            return paged_attention(q, cache, ctx, self.window, self.scale, self.keep_first, self.sink, gate, block=self.chunk)
        lam, out_scale, eps = self.lam, 1.0 - self.differential[0], self.differential[1]
        if (self.v_head_dim == self.head_dim and gate is None and self.sink is None and not self.keep_first
                and ops.mfma_attention_supported(q.dtype, self.head_dim, cache.page_size)):
            # Values as wide as both maps' keys together: each map becomes a head of its own whose query is padded with
            # zeros over the other map's half, which the matrix-core kernels score against the keys' whole rows; a small
            # kernel joins the two outputs.
            a = paged_attention(ops.diff_expand(q), cache, ctx, self.window, self.scale, block=self.chunk)
            return ops.diff_combine(a, self.n_heads, self.v_head_dim, lam, out_scale, eps)
        # any other sizes, and 32-bit: the kernel that knows two maps, one wave per (row, head), float math
        return ops.attention_plain(q, cache.k, cache.v, ctx.row_req, ctx.positions, ctx.block_table(cache.group), self.window,
                                   self.scale, self.keep_first, self.sink, gate, chunk=self.chunk, differential=(lam, out_scale, eps))

    def _forward_extras(self, h, ctx, binding: MixerBinding, sink):
        """The step with the optional mechanisms: the fused projection (with the gate's rows), one row kernel for bias,
        rotation, unit norms, value mixing and the cache write, attention with the gate as a factor on its output."""
        if not binding.writes_cache:
            raise ValueError(f"{self.name}: a layer with unit norms, an output gate or value mixing owns its cache")
        cache, nH, nKV, d, dv, T = binding.cache, self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, h.shape[0]
        style, rotary_dim, cos, sin = self.position.kernel_args(ctx)
        if self.position.needs_apply:
            raise ValueError(f"{self.name}: these mechanisms need a position part that gives the kernels a rotation table")
        t = ctx.timer
        qkv = ops.linear(h, self.w_qkv, keep_slices=True)
        dtype = qkv.dtype
        per_head_gate = self.output_gate and not self.gate_elementwise
        gate = torch.empty((T, nH), dtype=torch.float32, device=ctx.device) if per_head_gate else None
        qk_norm = (self.q_norm_w, self.k_norm_w, self.qk_norm_eps) if self.qk_norm_eps is not None else None
        key = ("value_mix", nKV, dv)
        v_first = v_out = None
        if self.value_mix == "source":
            v_out = torch.empty((T, nKV * dv), dtype=dtype, device=ctx.device)
            ctx.share(key, v_out)
        elif self.value_mix == "mix":
            v_first = ctx.shared(key)
            if v_first is None:
                raise ValueError(f"{self.name}: mixes in the values of an earlier layer, but none has handed any on in this step")
        q = ops.rope_append(qkv, self.b_qkv, ctx.write_slots(cache.group), cos, sin, style, rotary_dim, nH, nKV, d, cache.k, cache.v,
                            cache.page_size, dv, self.unit_norm_eps, gate, v_first, self.mix_weight, v_out, qk_norm,
                            self.gate_rows if self.gate_elementwise else 0)
        if t is not None:
            t.mark("mixer.qkv")
        a = self._attend(q, cache, ctx, gate)
        if self.gate_elementwise:         # the gate's columns lie behind q, k and v in the projected rows
            a = ops.sigmoid_gate(a, qkv, (nH + nKV) * d + nKV * dv)
        if t is not None:
            t.mark("mixer.attention")
        return self._project_out(a, sink)

    def forward(self, h, ctx, binding: MixerBinding, sink=None):
        if self._extras:
            return self._forward_extras(h, ctx, binding, sink)
        cache = binding.cache
        nH, d = self.n_heads, self.head_dim
        nKV = self.n_kv_heads if binding.writes_cache else 0
        width = (nH + nKV) * d + nKV * self.v_head_dim
        style, rotary_dim, cos, sin = self.position.kernel_args(ctx)
        w, b = self.w_qkv, self.b_qkv
        if not binding.writes_cache:  # only the queries: the first nH*d rows of the fused matrix
            if self._w_q is None:
                self._w_q = self._prepare_qkv(w.rows[:width], self.n_heads)
            w, b = self._w_q, (b[:width] if b is not None else None)
        slots = ctx.write_slots(cache.group) if binding.writes_cache else None
        t = ctx.timer
        if (style == ops.ROPE_SPLIT_HALF and rotary_dim == d and w.order is not None and h.dtype == torch.bfloat16
                and h.shape[0] <= 16 and not self.position.needs_apply):
            # few tokens: the rotation and the cache write are the projection's epilogue
            q = ops.qkv_rope_append(h, w, b, slots, cos, sin, nH, nKV, d, cache.k if slots is not None else None,
                                    cache.v if slots is not None else None, cache.page_size)
            if t is not None:
                t.mark("mixer.qkv")
            a = self._attend(q, cache, ctx)
            if t is not None:
                t.mark("mixer.attention")
            return self._project_out(a, sink)
        qkv = ops.linear(h, w, keep_slices=not self.position.needs_apply)     # the rotary kernel adds partial sums itself
        if self.position.needs_apply:
            qkv, b = self._encode_outside(qkv, b, ctx, nKV), None
        q = ops.rope_append(qkv, b, slots, cos, sin, style, rotary_dim, nH, nKV, d,
                            cache.k if slots is not None else None, cache.v if slots is not None else None,
                            cache.page_size, self.v_head_dim)
        if t is not None:
            t.mark("mixer.qkv")
        a = self._attend(q, cache, ctx)
        if t is not None:
            t.mark("mixer.attention")
        return self._project_out(a, sink)

    def _encode_outside(self, qkv, bias, ctx, nKV):
        """For a position part that transforms q and k itself: add the bias, let the part encode,
        and hand the kernel rows it only has to copy."""
        nH, d, T = self.n_heads, self.head_dim, qkv.shape[0]
        if bias is not None:
            qkv = (qkv.float() + bias.float()).to(qkv.dtype)
        q = qkv[:, : nH * d].reshape(T, nH, d)
        k = qkv[:, nH * d: (nH + nKV) * d].reshape(T, nKV, d) if nKV else None
        q, k = self.position.apply(q, k, ctx.positions)
        cols = [q.reshape(T, nH * d)]
        if nKV:
            cols += [k.reshape(T, nKV * d), qkv[:, (nH + nKV) * d:]]
        return torch.cat(cols, dim=1).contiguous()
