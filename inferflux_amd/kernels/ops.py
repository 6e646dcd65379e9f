"""Python faces of the HIP kernels.

Every function checks on the host that the operands are on the GPU, contiguous, of the
expected type and of shapes that fit what the kernel and its grid assume, and only then
launches on torch's current stream.  Nothing here falls back to another implementation: a
missing library or a refused size raises.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Iterable, Optional, Tuple

import torch

from .. import log
from .device import ARCH, COMPUTE_UNITS, N_XCD
from .library import KernelModule, Variant, load_module

P = ctypes.c_void_p
I = ctypes.c_int
F = ctypes.c_float
LL = ctypes.c_longlong

DT_F32, DT_BF16 = 0, 1
_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16}

ROPE_NONE, ROPE_SPLIT_HALF, ROPE_CONSECUTIVE = 0, 1, 2
ACT_SILU, ACT_GELU_TANH = 0, 1          # gated activations of a feed-forward: act(gate) * up
ACT_CLAMPED_SWISH = 2                   # ... and min(gate, L) sigmoid(1.702 min(gate, L)) (clamp(up, -L, L) + 1), which takes its limit L
_GATED_EPILOGUE = {ACT_SILU: 1, ACT_GELU_TANH: 3}    # ... as the epilogue number of the streaming products

# The matrix-core attention module is compiled per head size, when a model with that head size
# first runs; these sizes are compiled ahead by build_all().
MFMA_HEAD_DIMS_PREBUILT = (16, 32, 64, 128)
MFMA_MAX_HEAD_DIM = 128
# The tile kernel's two tilings: 1 = tiles of 64 rows (four waves of 16), which give twice as many workgroups for
# short portions; 2 = tiles of 128 rows, in which every key and value fetched serves twice as many rows.  At head
# size 128 the tall tiles are the kernel of attn_prefill.hip (eight waves of 16 rows, tiles loaded straight into
# LDS), at the other head sizes attn_mfma.hip's with two query tiles per wave.
TILE_QTS = (1, 2)
# (that kernel is written in gfx950's own instructions, loads into LDS of 16 bytes a lane among them; built for anything
# else, the tall tiles of head size 128 are attn_mfma.hip's as well)
DIRECT_TILE_HEAD_DIM = 128 if ARCH == "gfx950" else None


class KernelError(RuntimeError):
    pass


def module_variants() -> Iterable[Tuple[str, Variant]]:
    yield ("cache_manager", ())       # host code: the cache's bookkeeping
    yield ("core", ())
    yield ("gemm_f32", ())
    yield ("attn_plain", ())
    yield ("sampling", ())
    yield ("gemm_bf16", ())
    yield ("gemm_wide", ())
    yield ("layernorm", ())
    yield ("latent", ())
    yield ("moe", ())
    yield ("ssm", ())
    yield ("gla", ())
    yield ("delta", ())
    yield ("hyper", ())
    yield ("rowwise", ())
    yield ("grouped_gemm", ())
    yield ("ceilings", ())            # measurement only: what the memory gives a kernel that just reads
    for d in MFMA_HEAD_DIMS_PREBUILT:
        for qt in TILE_QTS:
            yield _tile_module(d, qt)[:2]
    if DIRECT_TILE_HEAD_DIM is not None:      # (tall tiles with kept first keys, a sink or a gate at that head size)
        yield _tile_module(DIRECT_TILE_HEAD_DIM, 2, direct=False)[:2]
    for dk, dv in WIDE_DIMS_PREBUILT:
        yield ("attn_wide", (("K_DIM", dk), ("V_DIM", dv)))


def _tile_module(head_dim: int, qt: int, direct: bool = True):
    """(module, variant, entry point, the function that says its tile rows) of the tile kernel for a tiling.  ``direct``
    False: not the kernel that loads straight into LDS (it has no kept first keys, sink or gate)."""
    if qt == 2 and head_dim == DIRECT_TILE_HEAD_DIM and direct:
        return "attn_prefill", (("HEAD_DIM", head_dim),), "ifx_attn_prefill", "ifx_attn_prefill_tile_rows"
    return "attn_mfma", (("HEAD_DIM", head_dim), ("TILE_QT", qt)), "ifx_attn_tiles", "ifx_attn_tile_rows"


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported element type {t.dtype} (float32 or bfloat16)") from None


def _check(t: torch.Tensor, name: str, shape=None, dtype=None) -> None:
    # on every launch: written for the case that nothing is wrong
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous()):
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{name}: not a tensor")
        if not t.is_cuda:
            raise KernelError(f"{name}: tensor is on {t.device}; the kernels run on the GPU only")
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: element type {t.dtype}, expected {dtype}")
    if shape is not None:
        ts = t.shape
        ok = len(shape) == len(ts)
        if ok:
            for want, got in zip(shape, ts):
                if want is not None and want != got:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {tuple(ts)}, expected {tuple(shape)}")


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _stream() -> int:
    # torch's current stream as a raw handle; the accessor that skips building a Stream object is used
    # where this torch has it (it is called once per launch)
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _call(mod: KernelModule, fname: str, argtypes, *args) -> None:
    rc = mod.fn(fname, argtypes)(*args)
    if rc != 0:
        raise KernelError(f"{fname}: {mod.last_error()} (code {rc})")


# ----------------------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, H] rows of ``table`` [V, H] named by int32 ``ids`` [T] (ids are checked by the caller), times ``scale``."""
    _check(ids, "ids", (None,), torch.int32)
    _check(table, "table", (None, None))
    T, H = ids.shape[0], table.shape[1]
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _call(load_module("core"), "ifx_embedding", (P, P, I, P, I, I, F, P),
          ids.data_ptr(), table.data_ptr(), _dt(table), out.data_ptr(), T, H, float(scale), _stream())
    return out


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, norm_weight: torch.Tensor, eps: float, scale: float = 1.0):
    """``embedding`` (times ``scale``) for up to 16 tokens that also prepares the RMS norm (bfloat16 weight ``norm_weight`` [H]) which
    reads the stream first: returns (the float32 stream [T, H], that norm's rows up to the factor per row)."""
    _check(ids, "ids", (None,), torch.int32)
    _check(table, "table", (None, None))
    T, H = ids.shape[0], table.shape[1]
    _check(norm_weight, "norm_weight", (H,), torch.bfloat16)
    if T > 16:
        raise KernelError(f"embedding_scaled: {T} rows (at most 16)")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    rows = torch.empty((T, H), dtype=torch.bfloat16, device=table.device)
    pieces = torch.empty((-(-H // 4096), 16), dtype=torch.float32, device=table.device)
    _call(load_module("core"), "ifx_embedding_norm", (P, P, I, P, P, P, P, I, I, F, P),
          ids.data_ptr(), table.data_ptr(), _dt(table), norm_weight.data_ptr(), out.data_ptr(), rows.data_ptr(),
          pieces.data_ptr(), T, H, float(scale), _stream())
    return out, ScaledRows(rows, pieces, H, eps, norm_weight)


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, delta_scale: float = 1.0) -> torch.Tensor:
    """``residual`` [T, H] float32 (+= ``delta_scale`` * ``delta`` in place when given and no ``rows``), then RMSNorm.

    With ``rows`` (int32 [R]) only those rows are normalised, into [R, H], and the residual is
    left untouched.
    """
    _check(residual, "residual", (None, None), torch.float32)
    T, H = residual.shape
    _check(weight, "weight", (H,))
    n_slices = 1
    if isinstance(delta, ScaledDelta):             # a delta with its factor
        delta, delta_scale = delta.value, delta_scale * delta.scale
    if isinstance(delta, SliceSums):               # partial sums: the kernel adds them in slice order
        _check(delta.parts, "delta", (None, T, H), torch.float32)
        n_slices, delta = delta.parts.shape[0], delta.parts
    elif delta is not None:
        _check(delta, "delta", (T, H))
    n = T
    if rows is not None:
        _check(rows, "rows", (None,), torch.int32)
        n = rows.shape[0]
    out = torch.empty((n, H), dtype=out_dtype, device=residual.device)
    _call(load_module("core"), "ifx_add_rmsnorm", (P, P, I, P, I, P, I, P, I, I, F, I, I, LL, F, P),
          residual.data_ptr(), _ptr(delta), _dt(delta) if delta is not None else 0, weight.data_ptr(),
          _dt(weight), out.data_ptr(), _DT[out_dtype], _ptr(rows), n, H, float(eps),
          1 if (delta is not None and rows is None) else 0, n_slices, T * H, float(delta_scale), _stream())
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0):
    """``magnitude`` times cos and sin [T, pairs] of float(position) * inv_freq, computed in float."""
    _check(positions, "positions", (None,), torch.int32)
    _check(inv_freq, "inv_freq", (None,), torch.float32)
    T, n = positions.shape[0], inv_freq.shape[0]
    cs = torch.empty((T, n), dtype=torch.float32, device=positions.device)
    sn = torch.empty((T, n), dtype=torch.float32, device=positions.device)
    _call(load_module("core"), "ifx_rope_table", (P, P, P, P, I, I, F, P),
          positions.data_ptr(), inv_freq.data_ptr(), cs.data_ptr(), sn.data_ptr(), T, n, float(magnitude), _stream())
    return cs, sn


def rope_append(qkv: torch.Tensor, bias: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rope_style: int,
                rotary_dim: int, n_heads: int, n_kv_heads: int, head_dim: int,
                k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_size: int,
                v_head_dim: Optional[int] = None, unit_norm_eps: Optional[float] = None, gate_out: Optional[torch.Tensor] = None,
                v_first: Optional[torch.Tensor] = None, v_mix: float = 0.0, v_out: Optional[torch.Tensor] = None,
                qk_norm: Optional[Tuple[torch.Tensor, torch.Tensor, float]] = None, extra_cols: int = 0) -> torch.Tensor:
    """Bias, rotation and cache write of one step's projections; returns q [T, n_heads, head_dim].

    ``qk_norm`` (q weight [head_dim], k weight [head_dim], eps): before the rotation every q and k head becomes
    x / sqrt(mean(x^2) + eps) * weight.  ``extra_cols``: further columns at the end of every row of ``qkv`` that belong
    to another kernel (a gate that is applied elsewhere).

    Optionally: ``unit_norm_eps`` divides every q and k head by its root mean square (eps inside the root) after the
    rotation; ``gate_out`` (float32 [T, n_heads]) receives sigmoid(x + bias) of n_heads further columns behind q, k and v
    (a gate per head on the attention's output); ``v_first`` [T, n_kv_heads v_head_dim] is mixed into the values before
    they are cached, v <- (1 - v_mix) v + v_mix v_first; ``v_out`` receives the values as projected, before any mixing.

    ``qkv`` is [T, (n_heads + n_kv_heads) head_dim + n_kv_heads v_head_dim] when the keys and values are
    written (``slots`` int32 [T] = page * page_size + offset; ``v_head_dim`` None: as wide as the keys), or
    [T, n_heads head_dim] with ``n_kv_heads`` = 0 for a mixer that only reads another's cache.  ``cos`` / ``sin``
    are the step's rotation table [T, rotary_dim / 2] (from rope_table).
    """
    T = qkv.shape[0]
    dv = head_dim if v_head_dim is None else int(v_head_dim)
    gate_cols = n_heads if gate_out is not None else 0
    width = (n_heads + n_kv_heads) * head_dim + n_kv_heads * dv + gate_cols + int(extra_cols)
    n_slices = 1
    if isinstance(qkv, SliceSums):                  # partial sums: the kernel adds them in slice order
        _check(qkv.parts, "qkv", (None, T, width), torch.float32)
        n_slices, dtype, qkv = qkv.parts.shape[0], qkv.dtype, qkv.parts
    else:
        _check(qkv, "qkv", (T, width))
        dtype = qkv.dtype
    if bias is not None:
        _check(bias, "bias", (width,))
    if rope_style != ROPE_NONE:
        _check(cos, "cos", (T, rotary_dim // 2), torch.float32)
        _check(sin, "sin", (T, rotary_dim // 2), torch.float32)
    if slots is not None:
        _check(slots, "slots", (T,), torch.int32)
        _check(k_cache, "k_cache", (None, n_kv_heads, page_size, head_dim), dtype)
        _check(v_cache, "v_cache", (k_cache.shape[0], n_kv_heads, dv, page_size), dtype)
    elif n_kv_heads != 0:
        raise KernelError("rope_append: keys and values given but no slots to write them to")
    if gate_out is not None:
        _check(gate_out, "gate_out", (T, n_heads), torch.float32)
    for t, nm in ((v_first, "v_first"), (v_out, "v_out")):
        if t is not None:
            _check(t, nm, (T, n_kv_heads * dv), dtype)
    qn = kn = None
    if qk_norm is not None:
        qn, kn, pre_eps = qk_norm
        _check(qn, "q norm weight", (head_dim,))
        _check(kn, "k norm weight", (head_dim,), qn.dtype)
    q = torch.empty((T, n_heads, head_dim), dtype=dtype, device=qkv.device)
    _call(load_module("core"), "ifx_rope_append",
          (P, I, P, I, P, P, P, I, I, I, I, I, I, I, P, P, P, I, LL, I, I, P, I, F, P, F, P, P, P, I, F, I, P),
          qkv.data_ptr(), _DT[dtype], _ptr(bias), _dt(bias) if bias is not None else 0, _ptr(slots),
          _ptr(cos) if rope_style != ROPE_NONE else 0, _ptr(sin) if rope_style != ROPE_NONE else 0, rope_style,
          rotary_dim, T, n_heads, n_kv_heads, head_dim, page_size, q.data_ptr(), _ptr(k_cache), _ptr(v_cache),
          n_slices, T * width, dv, gate_cols, _ptr(gate_out), 1 if unit_norm_eps is not None else 0,
          float(unit_norm_eps or 0.0), _ptr(v_first), float(v_mix), _ptr(v_out), _ptr(qn), _ptr(kn),
          _dt(qn) if qn is not None else 0, float(pre_eps) if qn is not None else 0.0, int(extra_cols), _stream())
    return q


def swiglu(gate_up: torch.Tensor, interleaved: bool = False, act: int = ACT_SILU, limit: float = 0.0) -> torch.Tensor:
    """act(gate) * up [T, I] from [T, 2I] laid out [gate | up] or, interleaved, gate_0, up_0, gate_1, ...; ``act``:
    ACT_SILU (the default), ACT_GELU_TANH, or ACT_CLAMPED_SWISH with its ``limit`` L: g = min(gate, L),
    u = clamp(up, -L, L), g sigmoid(1.702 g) (u + 1)."""
    _check(gate_up, "gate_up", (None, None))
    T, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("swiglu: odd width")
    out = torch.empty((T, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _call(load_module("core"), "ifx_swiglu", (P, P, I, I, I, I, I, F, P),
          gate_up.data_ptr(), out.data_ptr(), _dt(gate_up), T, two_i // 2, 1 if interleaved else 0, int(act), float(limit), _stream())
    return out


def _delta_args(delta, shape, name):
    """(pointer, dtype code, slices, elements between slices) of a tensor or of a product left as ``SliceSums``."""
    if isinstance(delta, ScaledDelta):
        delta = delta.tensor()
    if isinstance(delta, SliceSums):
        _check(delta.parts, name, (None, *shape), torch.float32)
        return delta.parts.data_ptr(), DT_F32, delta.parts.shape[0], delta.parts[0].numel()
    _check(delta, name, shape)
    return delta.data_ptr(), _dt(delta), 1, 0


def layernorm(x: torch.Tensor, delta, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
              rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Layer norm with a weight and no bias of the rows of ``x`` [T, H] (float32 or bfloat16), in float:
    (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight.  A ``delta`` (a tensor or ``SliceSums``) is added first,
    and written back into ``x`` unless ``rows`` (int32 [R]) picks the rows to normalise."""
    _check(x, "x", (None, None))
    T, H = x.shape
    _check(weight, "weight", (H,))
    dp, dd, n_slices, stride = (0, 0, 1, 0) if delta is None else _delta_args(delta, (T, H), "delta")
    n = T
    if rows is not None:
        _check(rows, "rows", (None,), torch.int32)
        n = rows.shape[0]
    out = torch.empty((n, H), dtype=out_dtype, device=x.device)
    _call(load_module("layernorm"), "ifx_layernorm", (P, I, P, I, I, LL, P, I, P, I, P, I, I, F, P),
          x.data_ptr(), _dt(x), dp, dd, n_slices, stride, weight.data_ptr(), _dt(weight), out.data_ptr(), _DT[out_dtype],
          _ptr(rows), n, H, float(eps), _stream())
    return out


def add_layernorm(stream: torch.Tensor, delta, weight: torch.Tensor, eps: float,
                  cast_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """``stream`` [T, H] (float32) += layer norm (weight, no bias) of ``delta`` [T, H] (a tensor or ``SliceSums``), in
    place.  With ``cast_dtype`` the new stream rounded to that type is returned as well (what a sub-block that reads
    the stream itself takes as its input); with float32 that is the stream."""
    _check(stream, "stream", (None, None), torch.float32)
    T, H = stream.shape
    _check(weight, "weight", (H,))
    dp, dd, n_slices, stride = _delta_args(delta, (T, H), "delta")
    cast = torch.empty((T, H), dtype=cast_dtype, device=stream.device) if cast_dtype not in (None, torch.float32) else None
    _call(load_module("layernorm"), "ifx_add_layernorm", (P, P, I, I, LL, P, I, P, I, I, I, F, P),
          stream.data_ptr(), dp, dd, n_slices, stride, weight.data_ptr(), _dt(weight), _ptr(cast),
          _DT[cast_dtype] if cast is not None else 0, T, H, float(eps), _stream())
    return stream if cast_dtype == torch.float32 else cast


def cast_rows(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 rows ``x`` rounded to ``dtype`` (bfloat16)."""
    _check(x, "x", None, torch.float32)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _call(load_module("layernorm"), "ifx_cast_rows", (P, P, I, LL, P), x.data_ptr(), out.data_ptr(), _DT[dtype], x.numel(), _stream())
    return out


def latent_finish(y, q_norm: Optional[torch.Tensor], kv_norm: torch.Tensor, eps: float, cos: Optional[torch.Tensor],
                  sin: Optional[torch.Tensor], rot_dims: int, slots: Optional[torch.Tensor], q_rank: int, kv_rank: int,
                  rot_dim: int, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_size: int,
                  dtype: torch.dtype) -> Optional[torch.Tensor]:
    """What follows the down projections of attention through a latent.  ``y`` [T, q_rank + kv_rank + rot_dim] (a
    tensor or ``SliceSums``) holds per row the query latent, the key/value latent and the shared rotated key part.
    Returns the query latent under its RMS norm (weight ``q_norm``) [T, q_rank] (None when ``q_rank`` is 0); with
    ``slots`` (int32 [T] = page * page_size + offset) the key/value latent under its RMS norm (``kv_norm``) and the
    key part, its first ``rot_dims`` elements turned by the table ``cos`` / ``sin`` [T, rot_dims / 2], go into the
    cache: K rows [latent | key part] (``k_cache`` [pages, 1, page_size, kv_rank + rot_dim]) and V columns
    (``v_cache`` [pages, 1, kv_rank, page_size], or [pages, 1, kv_rank + rot_dim, page_size] for attention kernels that
    want values as wide as keys: the key part is then written there as well)."""
    width = q_rank + kv_rank + rot_dim
    T = y.shape[0]
    yp, yd, n_slices, stride = _delta_args(y, (T, width), "y")
    if q_rank:
        _check(q_norm, "q_norm", (q_rank,), kv_norm.dtype)
    _check(kv_norm, "kv_norm", (kv_rank,))
    if rot_dims:
        _check(cos, "cos", (T, rot_dims // 2), torch.float32)
        _check(sin, "sin", (T, rot_dims // 2), torch.float32)
    if slots is not None:
        _check(slots, "slots", (T,), torch.int32)
        _check(k_cache, "k_cache", (None, 1, page_size, kv_rank + rot_dim), dtype)
        _check(v_cache, "v_cache", (k_cache.shape[0], 1, None, page_size), dtype)
        if v_cache.shape[2] not in (kv_rank, kv_rank + rot_dim):
            raise KernelError(f"latent_finish: values of {v_cache.shape[2]} rows (the latent's {kv_rank}, or {kv_rank + rot_dim} with the key part)")
    cq = torch.empty((T, q_rank), dtype=dtype, device=kv_norm.device) if q_rank else None
    _call(load_module("latent"), "ifx_latent_finish", (P, I, I, LL, P, P, I, P, P, I, P, P, P, P, I, I, I, I, I, I, F, I, P),
          yp, yd, n_slices, stride, _ptr(q_norm), kv_norm.data_ptr(), _dt(kv_norm), _ptr(cos) if rot_dims else 0,
          _ptr(sin) if rot_dims else 0, rot_dims, _ptr(slots), _ptr(cq), _ptr(k_cache) if slots is not None else 0,
          _ptr(v_cache) if slots is not None else 0, _DT[dtype], T, q_rank, kv_rank, rot_dim, page_size, float(eps),
          v_cache.shape[2] if slots is not None else kv_rank, _stream())
    return cq


HEADWISE_GROUPED_MIN_ROWS = 32     # rows of a step from which the per-head products go to the matrix cores


def headwise(x: torch.Tensor, weight: torch.Tensor, n_heads: int, x_head: int, tail: int = 0,
             cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rot_dims: int = 0) -> torch.Tensor:
    """A product per head: out[t, h, :N] = ``weight``[h] x[t, h] with ``weight`` [H, N, K] and head h's input the K
    elements of row t of ``x`` [T, >= H * x_head] from h * x_head on.  The ``tail`` elements that follow a head's K
    inputs are appended to its output, the first ``rot_dims`` of them turned by the table ``cos`` / ``sin``
    [T, rot_dims / 2] in split-half pairs.  Returns [T, H, N + tail] in x's type; sums in float."""
    _check(x, "x", (None, None))
    T = x.shape[0]
    _check(weight, "weight", (n_heads, None, None), x.dtype)
    _, N, K = weight.shape
    if x_head < K + tail or x.shape[1] < (n_heads - 1) * x_head + K + tail:
        raise KernelError(f"headwise: {n_heads} heads of {K} + {tail} inputs, {x_head} apart, do not fit rows of {x.shape[1]}")
    if rot_dims:
        _check(cos, "cos", (T, rot_dims // 2), torch.float32)
        _check(sin, "sin", (T, rot_dims // 2), torch.float32)
    out = torch.empty((T, n_heads, N + tail), dtype=x.dtype, device=x.device)
    tail_only = 0
    if x.dtype == torch.bfloat16 and T >= HEADWISE_GROUPED_MIN_ROWS and K % 8 == 0 and x_head % 8 == 0 and x.shape[1] % 8 == 0:
        # many rows: the products on the matrix cores, and of the other kernel only the tails
        _call(load_module("grouped_gemm"), "ifx_headwise_grouped", (P, P, P, I, I, I, I, I, I, I, P),
              x.data_ptr(), weight.data_ptr(), out.data_ptr(), T, n_heads, K, N, x.shape[1], x_head, N + tail, _stream())
        if not tail:
            return out
        tail_only = 1
    _call(load_module("latent"), "ifx_headwise", (P, P, P, I, I, I, I, I, I, I, I, P, P, I, I, P),
          x.data_ptr(), weight.data_ptr(), out.data_ptr(), _dt(x), T, n_heads, K, N, x.shape[1], x_head, tail,
          _ptr(cos) if rot_dims else 0, _ptr(sin) if rot_dims else 0, rot_dims, tail_only, _stream())
    return out


ROUTE_FUSED_MAX_ROWS = 16       # rows up to which the router's kernel forms the logits itself


def moe_route(h: torch.Tensor, router, top: int, groups: int = 1, keep_groups: int = 1, group_top: int = 2,
              softmax: bool = False, renormalize: bool = False, scale: float = 1.0, bias: Optional[torch.Tensor] = None,
              choice_bias: Optional[torch.Tensor] = None):
    """The router of a mixture of experts, in float: scores of ``router`` [E, K] (a tensor or a ``LinearWeight``) times the
    rows of ``h`` [T, K] through a sigmoid (or a softmax over the experts), the ``top`` highest among the experts of the best
    ``keep_groups`` of ``groups`` equal groups of neighbours (a group scores the sum of its ``group_top`` highest).  Returns
    (ids int32 [T, top], weights float32 [T, top]): the chosen scores, divided by their sum with ``renormalize``, times
    ``scale``.  ``bias`` float32 [E] is added to the logits before anything else; ``choice_bias`` float32 [E] is added to the
    scores for the choice alone (the weights stay the scores themselves).  Up to ``ROUTE_FUSED_MAX_ROWS`` rows the kernel forms the logits itself; more rows in bfloat16 get them from
    ``linear`` with float32 sums and output."""
    _check(h, "h", (None, None))
    T, K = h.shape
    rows = router.rows if isinstance(router, LinearWeight) else router
    _check(rows, "router", (None, K), h.dtype)
    E = rows.shape[0]
    # (in 32-bit the kernel forms them whatever the rows: a row's sums then never depend on what shares its step)
    z = linear(h, router, out_dtype=torch.float32) if (T > ROUTE_FUSED_MAX_ROWS and h.dtype == torch.bfloat16) else None
    ids = torch.empty((T, top), dtype=torch.int32, device=h.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=h.device)
    if bias is not None:
        _check(bias, "bias", (E,), torch.float32)
    if choice_bias is not None:
        _check(choice_bias, "choice_bias", (E,), torch.float32)
    _call(load_module("moe"), "ifx_moe_route", (P, P, I, P, P, P, I, I, I, I, I, I, I, I, I, F, P, P, P),
          h.data_ptr(), rows.data_ptr(), _dt(h), _ptr(z), ids.data_ptr(), weights.data_ptr(), T, K, E, top, groups, keep_groups,
          group_top, 1 if softmax else 0, 1 if renormalize else 0, float(scale), _ptr(bias), _ptr(choice_bias), _stream())
    return ids, weights


def pair_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[E, ff, K] gate and up weights (ff a multiple of 16) as one tensor [E, 2 ff, K] whose rows alternate 16 of gate with
    the same 16 of up: a wave of the grouped product then holds a gate tile and its up tile, and the activation is its
    epilogue."""
    E, ff, K = gate.shape
    if ff % 16 or up.shape != gate.shape:
        raise KernelError(f"pair_gate_up: ff={ff} must be a multiple of 16 and both weights alike")
    return torch.stack([gate.view(E, ff // 16, 16, K), up.view(E, ff // 16, 16, K)], dim=2).reshape(E, 2 * ff, K).contiguous()


def moe_experts(h: torch.Tensor, gate: torch.Tensor, up: Optional[torch.Tensor], down: torch.Tensor, ids: torch.Tensor,
                weights: torch.Tensor, act: int = ACT_SILU, limit: float = 0.0, n_identity: int = 0) -> torch.Tensor:
    """sum_j weights[t, j] * down[e] (act(gate[e] h_t, up[e] h_t)), e = ids[t, j], row by row: every (row, choice)
    streams its expert's weights (``gate`` / ``up`` [E, ff, K], or ``gate`` [E, 2 ff, K] from ``pair_gate_up`` and ``up``
    None; ``down`` [E, N, ff]; all in h's type).  With ``n_identity`` an id from E upwards names an identity expert, whose
    output is the row itself (N = K then).  ``act``: ACT_SILU, ACT_GELU_TANH, or ACT_CLAMPED_SWISH with its ``limit``.  Returns [T, N]."""
    _check(h, "h", (None, None))
    T, K = h.shape
    paired = up is None
    _check(gate, "gate", (None, None, K), h.dtype)
    E, ff = gate.shape[0], gate.shape[1] // (2 if paired else 1)
    if not paired:
        _check(up, "up", (E, ff, K), h.dtype)
    _check(down, "down", (E, None, ff), h.dtype)
    N = down.shape[1]
    top = ids.shape[1]
    _check(ids, "ids", (T, top), torch.int32)
    _check(weights, "weights", (T, top), torch.float32)
    if n_identity and N != K:
        raise KernelError(f"moe_experts: identity experts hand back the row itself, so N={N} must equal K={K}")
    mod = load_module("moe")
    a = torch.empty((T, top, ff), dtype=h.dtype, device=h.device)
    _call(mod, "ifx_moe_gate_up", (P, P, P, P, P, I, I, I, I, I, I, I, I, F, P),
          h.data_ptr(), gate.data_ptr(), _ptr(up), ids.data_ptr(), a.data_ptr(), _dt(h), T, K, ff, top, 1 if paired else 0, E,
          int(act), float(limit), _stream())
    out = torch.empty((T, N), dtype=h.dtype, device=h.device)
    _call(mod, "ifx_moe_down", (P, P, P, P, P, I, I, I, I, I, I, P, P),
          a.data_ptr(), down.data_ptr(), ids.data_ptr(), weights.data_ptr(), out.data_ptr(), _dt(h), T, N, ff, top, E, h.data_ptr(), _stream())
    return out


def grouped_tile_items(n_items: int, n_experts: int) -> int:
    """Items of one expert to a workgroup of the grouped product: 128 where the experts get that many on average (every
    weight tile fetched then serves twice the items), else 64 (steps of few rows, whose tiles are mostly empty)."""
    return 128 if n_items >= 128 * n_experts else 64


def grouped_takes(dtype: torch.dtype, K: int, ff: int) -> bool:
    """Whether the grouped matrix-core product takes experts of these sizes."""
    return dtype == torch.bfloat16 and K % 8 == 0 and ff % 16 == 0


def moe_experts_grouped(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, ids: torch.Tensor,
                        weights: torch.Tensor, act: int = ACT_SILU, limit: float = 0.0, n_identity: int = 0) -> "SliceSums":
    """The same sum for steps of many rows, on the matrix cores: the (row, choice) items are ordered by expert on the
    device and every expert's weights meet tiles of its items (bfloat16; ``gate_up`` from ``pair_gate_up``).  Returns the
    choices' weighted outputs as ``SliceSums`` [top, T, N] (float32), which the kernel that adds them to the stream sums
    in the order of the choices.  ``n_identity``: ids from E up to E + n_identity name identity experts, whose output is
    the row itself (N = K then); ``act`` and ``limit`` as for ``moe_experts``."""
    _check(h, "h", (None, None), torch.bfloat16)
    T, K = h.shape
    _check(gate_up, "gate_up", (None, None, K), torch.bfloat16)
    E, ff = gate_up.shape[0], gate_up.shape[1] // 2
    _check(down, "down", (E, None, ff), torch.bfloat16)
    N, top = down.shape[1], ids.shape[1]
    _check(ids, "ids", (T, top), torch.int32)
    _check(weights, "weights", (T, top), torch.float32)
    if not grouped_takes(h.dtype, K, ff):
        raise KernelError(f"moe_experts_grouped: K={K} must be a multiple of 8 and ff={ff} of 16")
    mod = load_module("grouped_gemm")
    if n_identity and N != K:
        raise KernelError(f"moe_experts_grouped: identity experts hand back the row itself, so N={N} must equal K={K}")
    n_items = T * top
    n_real, E = E, E + int(n_identity)
    tile_items = grouped_tile_items(n_items, E)
    max_tiles = -(-n_items // tile_items) + E          # every expert may end on a tile that is not full
    lists = torch.empty((n_items + 3 * max_tiles + 1,), dtype=torch.int32, device=h.device)
    sorted_, te, ts, tc, nt = (lists[:n_items], lists[n_items:n_items + max_tiles], lists[n_items + max_tiles:n_items + 2 * max_tiles],
                               lists[n_items + 2 * max_tiles:n_items + 3 * max_tiles], lists[n_items + 3 * max_tiles:])
    _call(mod, "ifx_moe_sort", (P, I, I, I, P, P, P, P, P, P), ids.data_ptr(), n_items, E, tile_items, sorted_.data_ptr(), te.data_ptr(),
          ts.data_ptr(), tc.data_ptr(), nt.data_ptr(), _stream())
    a = torch.empty((n_items, ff), dtype=torch.bfloat16, device=h.device)
    _call(mod, "ifx_moe_gate_up_grouped", (P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, P),
          h.data_ptr(), gate_up.data_ptr(), a.data_ptr(), sorted_.data_ptr(), te.data_ptr(), ts.data_ptr(), tc.data_ptr(),
          nt.data_ptr(), max_tiles, tile_items, K, ff, top, n_real, int(act), float(limit), _stream())
    parts = torch.empty((top, T, N), dtype=torch.float32, device=h.device)
    _call(mod, "ifx_moe_down_grouped", (P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P, P),
          a.data_ptr(), down.data_ptr(), parts.data_ptr(), weights.data_ptr(), sorted_.data_ptr(), te.data_ptr(), ts.data_ptr(),
          tc.data_ptr(), nt.data_ptr(), max_tiles, tile_items, T, N, ff, top, n_real, h.data_ptr(), _stream())
    return SliceSums(parts, torch.bfloat16)


# ----------------------------------------------------------------------------------------
def gemm_f32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] (float32 or bfloat16) times float32 ``weight`` [N, K] transposed, true 32-bit math."""
    _check(x, "x", (None, None))
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.float32)
    N = weight.shape[0]
    if bias is not None:
        _check(bias, "bias", (N,), torch.float32)
    out_dtype = out_dtype or x.dtype
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _call(load_module("gemm_f32"), "ifx_gemm_f32", (P, I, P, P, P, I, I, I, I, P),
          x.data_ptr(), _dt(x), weight.data_ptr(), _ptr(bias), out.data_ptr(), _DT[out_dtype], M, N, K, _stream())
    return out


SKINNY_MAX_M = 64
WIDE_MAX_M = 128           # rows the product that shares x through LDS takes at most ...
WIDE_MANY_ROWS_MAX_N = 16384   # ... beyond 64 of them only for weights of up to this many rows (see _small_m_kernel)


def enable_library_gemm_tuning(max_ms_per_shape: int = 300, filename: Optional[str] = None) -> None:
    """Let the library pick, by timing, the fastest of its kernels for every matrix-product shape it
    meets (torch's TunableOp over hipBLASLt and rocBLAS).  The first product of a shape then takes
    up to ``max_ms_per_shape`` longer; worth it when shapes repeat (a fixed prefill portion, a steady
    decode batch), not for one-off shapes, so it is off unless asked for."""
    import torch.cuda.tunable as tunable
    tunable.enable(True)
    tunable.tuning_enable(True)
    tunable.set_max_tuning_duration(int(max_ms_per_shape))
    if not filename:
        import os
        from .library import _fallback_dir
        # this user's private folder under the temporary directory (refused if somebody else made it or may write it)
        filename = os.path.join(_fallback_dir(create=True), "tunableop.csv")
    tunable.set_filename(filename)     # choices are kept there and reused by later runs


def pause_library_gemm_tuning(paused: bool) -> None:
    """While paused, shapes already timed keep their chosen kernel and new shapes take the default."""
    import torch.cuda.tunable as tunable
    if tunable.is_enabled():
        tunable.tuning_enable(not paused)


def tile_weights(weight: torch.Tensor, order: Optional[torch.Tensor] = None, tile_rows: int = 16) -> torch.Tensor:
    """The tiled form of a bfloat16 ``weight`` [N, K] that the weight-streaming product reads in
    contiguous runs: a flat tensor of ceil(N / tile_rows) row tiles of ``tile_rows`` rows (even, 8 to 16) by
    cols64(K) k-values (zeros in the padding).  ``order`` (int32, a permutation of the row tiles, tiles of 16
    only): tile t of the copy is row tile order[t] of the weight."""
    _check(weight, "weight", (None, None), torch.bfloat16)
    N, K = weight.shape
    if K % 8:
        raise KernelError(f"tile_weights: K={K} must be a multiple of 8")
    if tile_rows not in TILE_ROWS or (order is not None and tile_rows != 16):
        raise KernelError(f"tile_weights: {tile_rows} rows to a tile (one of {TILE_ROWS}; 16 with a tile order)")
    mod = load_module("gemm_bf16")
    n_tiles = -(-N // tile_rows)
    if order is not None:
        _check(order, "order", (n_tiles,), torch.int32)
        if sorted(order.tolist()) != list(range(n_tiles)):
            raise KernelError("tile_weights: order is not a permutation of the weight's row tiles")
    out = torch.empty((_tiled_size(N, K, tile_rows),), dtype=torch.bfloat16, device=weight.device)
    _call(mod, "ifx_tile_weights", (P, P, I, I, P, I, P), weight.data_ptr(), out.data_ptr(), N, K, _ptr(order), tile_rows, _stream())
    return out


TILE_ROWS = (8, 10, 12, 14, 16)      # rows a tile of the copy may hold


def _tiled_size(N: int, K: int, tile_rows: int) -> int:
    return -(-N // tile_rows) * tile_rows * (-(-K // 64) * 64)


def choose_tile_rows(N: int) -> int:
    """Rows to a tile of a weight's streamed copy.  A workgroup of the products for few rows of x owns whole row
    tiles, and a compute unit can have only so many bytes on their way: a weight of 3,584 rows in tiles of 16
    gives 224 of the 256 units a tile and takes as long as one of 4,096 rows.  Where 16-row tiles leave units
    without one, the tiles are made as low as still gives every unit at most one (3,584 rows: 14; 2,048: 8).
    Measured at 1-64 rows of x: 3,584 x 18,944 takes 24.8 us instead of 25.9 at 8 rows, 2,048 x 11,008 16.3
    instead of 20.1 at 16 rows; weights with more tiles than units gain nothing from lower tiles or lose."""
    if N > 16 * COMPUTE_UNITS:
        return 16
    rows = -(-N // COMPUTE_UNITS)
    return min(16, max(8, rows + rows % 2))


class LinearWeight:
    """A projection's weight as the products want it: ``rows`` [N, K] as the model file has it, and for
    bfloat16 weights ``tiled``, the copy that products with few rows of x (decoding) stream from.  The
    copy doubles the weight's memory; it is left out when ``decode_weight_copy`` is off or when the
    card has no room for it, and products with few rows then read ``rows``."""

    __slots__ = ("rows", "tiled", "order", "tile_rows")

    def __init__(self, rows: torch.Tensor, tiled: Optional[torch.Tensor] = None, order: Optional[torch.Tensor] = None,
                 tile_rows: int = 16):
        # order: the copy's row-tile order, tile_rows: the rows to a tile of the copy (see tile_weights)
        self.rows, self.tiled, self.order, self.tile_rows = rows, tiled, order, tile_rows

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


# Whether prepare_linear makes tiled copies, and how much memory it leaves free when it does.
decode_weight_copy = True
DECODE_COPY_RESERVE_BYTES = 8 << 30


def prepare_linear(weight: torch.Tensor, order: Optional[torch.Tensor] = None, tile_rows: int = 0) -> LinearWeight:
    """Wrap a projection's weight for ``linear`` / ``linear_swiglu``, with the tiled copy if wanted and possible
    (its row tiles in ``order``, if given, and then of 16 rows; else of ``tile_rows`` rows, 0: ``choose_tile_rows``)."""
    tiled = None
    if order is not None:
        tile_rows = 16
    elif tile_rows == 0:
        tile_rows = choose_tile_rows(weight.shape[0]) if weight.dim() == 2 else 16
    if (decode_weight_copy and weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] % 8 == 0):
        free, _ = torch.cuda.mem_get_info(weight.device)
        if free >= weight.numel() * 2 + DECODE_COPY_RESERVE_BYTES:
            tiled = tile_weights(weight.contiguous(), order, tile_rows)
        else:
            log.warn("kernels", f"no room for the decode copy of a {tuple(weight.shape)} weight "
                                f"({free / 2**30:.1f} GiB free): decoding reads the plain rows")
    return LinearWeight(weight, tiled, order if tiled is not None else None, tile_rows if tiled is not None else 16)


class ScaledRows:
    """Rows of a normalised activation up to one factor per row: row t stands for
    ``rows[t] * rsqrt(sum(pieces[:, t]) / width + eps)``.  ``rows`` is bfloat16 [T <= 16, width] (the stream times
    the norm's weight), ``pieces`` float32 [n, 16] (sums of squares of the stream over runs of columns, one run
    per row tile of the product that made them; rows past T hold zeros).  A weight-streaming product that takes these multiplies its sums by the factor, which
    saves the norm a kernel of its own; ``linear_into_stream`` makes them."""

    __slots__ = ("rows", "pieces", "width", "eps", "norm_weight")

    def __init__(self, rows: torch.Tensor, pieces: torch.Tensor, width: int, eps: float,
                 norm_weight: Optional[torch.Tensor] = None):
        self.rows, self.pieces, self.width, self.eps = rows, pieces, int(width), float(eps)
        self.norm_weight = norm_weight      # the weight the rows were multiplied by: whose norm they stand for

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


class ScaledDelta:
    """A sub-block's output that is added to the stream times ``scale`` (a model's factor on every sub-block's output):
    ``value`` is a tensor or ``SliceSums``.  ``add_rmsnorm`` takes it as its delta; ``tensor()`` forms it for everyone
    else."""

    __slots__ = ("value", "scale")

    def __init__(self, value, scale: float):
        self.value, self.scale = value, float(scale)

    @property
    def shape(self):
        return self.value.shape

    def tensor(self) -> torch.Tensor:
        v = self.value.sum(torch.float32) if isinstance(self.value, SliceSums) else self.value.float()
        return v * self.scale


class SliceSums:
    """A product left as partial sums over slices of K: it stands for ``parts.sum(0)`` (float32 [S, M, N], added in
    slice order).  ``add_rmsnorm`` takes it as its delta and ``rope_append`` as its q/k/v, which saves the kernel
    that would add the slices; ``sum()`` adds them for everyone else."""

    __slots__ = ("parts", "dtype")

    def __init__(self, parts: torch.Tensor, dtype: torch.dtype):
        self.parts, self.dtype = parts, dtype      # dtype: what the sum would be rounded to

    @property
    def shape(self):
        return self.parts.shape[1:]

    def sum(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        S, M, N = self.parts.shape
        out = torch.empty((M, N), dtype=dtype or self.dtype, device=self.parts.device)
        _call(load_module("gemm_wide"), "ifx_sum_slices", (P, P, I, I, LL, P),
              self.parts.data_ptr(), out.data_ptr(), _DT[out.dtype], S, M * N, _stream())
        return out


def _scale_args(x):
    """(rows, the four row-factor arguments of the kernels) of a tensor or a ``ScaledRows``."""
    if isinstance(x, ScaledRows):
        _check(x.pieces, "pieces", (None, 16), torch.float32)
        if not 1 <= x.pieces.shape[0] <= x.width:
            raise KernelError(f"scaled rows: {x.pieces.shape[0]} pieces for a width of {x.width}")
        _check(x.rows, "rows", (None, x.width), torch.bfloat16)
        if x.rows.shape[0] > 16:
            raise KernelError(f"scaled rows: {x.rows.shape[0]} rows, at most 16")
        return x.rows, (x.pieces.data_ptr(), x.pieces.shape[0], float(x.width), x.eps)
    return x, (0, 0, 0.0, 0.0)


def takes_scaled_rows(n_rows: int, weight) -> bool:
    """Whether ``linear`` / ``linear_swiglu`` / ``qkv_rope_append`` take ``ScaledRows`` of ``n_rows`` rows with this weight."""
    if not isinstance(weight, LinearWeight):
        return False
    N, K = weight.rows.shape
    return (weight.rows.dtype == torch.bfloat16 and n_rows <= 16
            and _small_m_kernel(n_rows, N, K, weight.tiled is not None) in ("skinny", "wide"))


def adds_into_stream(n_rows: int, weight, norm_weight: torch.Tensor) -> bool:
    """Whether ``linear_into_stream`` takes this shape."""
    if not isinstance(weight, LinearWeight) or weight.order is not None:
        return False
    N, K = weight.rows.shape
    if norm_weight is None:           # (a reader that takes partial sums but keeps the addition to itself)
        return False
    return (weight.rows.dtype == torch.bfloat16 and norm_weight.dtype == torch.bfloat16 and n_rows <= 16 and N % 4 == 0
            and _small_m_kernel(n_rows, N, K, weight.tiled is not None) == "skinny")


def linear_into_stream(x: torch.Tensor, weight: LinearWeight, stream: torch.Tensor, norm_weight: torch.Tensor,
                       eps: float, mult: float = 1.0) -> ScaledRows:
    """``stream`` [M <= 16, N] (float32) += ``mult`` * x [M, K] W^T in place, as the product's epilogue, which also prepares
    the RMS norm that follows (weight ``norm_weight`` [N] bfloat16): returns its rows up to the factor per row."""
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    N = weight.rows.shape[0]
    if not adds_into_stream(M, weight, norm_weight) or weight.rows.shape[1] != K:
        raise KernelError(f"linear_into_stream: not for {M} rows times a {tuple(weight.rows.shape)} weight")
    _check(stream, "stream", (M, N), torch.float32)
    _check(norm_weight, "norm_weight", (N,), torch.bfloat16)
    rows = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    tile_rows = 16 if weight.tiled is None else weight.tile_rows
    pieces = torch.empty((-(-N // tile_rows), 16), dtype=torch.float32, device=x.device)    # one piece per row tile
    w = weight.rows if weight.tiled is None else weight.tiled
    _call(load_module("gemm_bf16"), "ifx_skinny_gemm", _SKINNY_ARGS,
          x.data_ptr(), w.data_ptr(), 0, DT_F32, M, N, K, 0, 0, 0, 2, 0 if weight.tiled is None else tile_rows, 0,
          0, 0, 0.0, 0.0, stream.data_ptr(), norm_weight.data_ptr(), rows.data_ptr(), pieces.data_ptr(), float(mult), _stream())
    return ScaledRows(rows, pieces, N, eps, norm_weight)


_SKINNY_ARGS = (P, P, P, I, I, I, I, I, I, I, I, I, P, P, I, F, F, P, P, P, P, F, P)


def pair_tile_order(n_heads: int, head_dim: int) -> list:
    """Row-tile order of a projection whose rows are ``n_heads`` heads of ``head_dim`` (a multiple of 32) that
    puts the two halves of 16 split-half rotation pairs into consecutive tiles: for head h and j < d / 32,
    tiles h d/16 + j and h d/16 + j + d/32.  What ``qkv_rope_append`` expects of its tiled copy."""
    per, half = head_dim // 16, head_dim // 32
    return [h * per + j + s * half for h in range(n_heads) for j in range(half) for s in (0, 1)]


def qkv_rope_append(x: torch.Tensor, weight: LinearWeight, bias: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                    cos: torch.Tensor, sin: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_size: int,
                    waves: int = 0, unroll: int = 0) -> torch.Tensor:
    """For up to 16 tokens: q, k, v = x W^T + bias from the pair-ordered tiled copy of the concatenated
    weight, q and k rotated (split-half pairs over the whole head, table cos/sin [M, d/2]), k and v written
    into the paged cache at ``slots``, q returned [M, nH, d] -- one kernel, the rotation and the cache
    write being the product's epilogue.  With ``slots`` None the weight holds the query rows only.
    ``x`` may be ``ScaledRows``."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    heads = n_heads + (2 * n_kv_heads if slots is not None else 0)
    if weight.tiled is None or weight.order is None or tuple(weight.rows.shape) != (heads * head_dim, K):
        raise KernelError(f"qkv_rope_append: needs the pair-ordered tiled copy of a [{heads * head_dim}, {K}] weight")
    if M > 16 or head_dim % 32 or K % 8:
        raise KernelError(f"qkv_rope_append: M={M} must be <= 16, head_dim={head_dim} a multiple of 32, K={K} of 8")
    _check(cos, "cos", (M, head_dim // 2), torch.float32)
    _check(sin, "sin", (M, head_dim // 2), torch.float32)
    if bias is not None:
        _check(bias, "bias", (heads * head_dim,))
    if slots is not None:
        _check(slots, "slots", (M,), torch.int32)
        _check(k_cache, "k_cache", (None, n_kv_heads, page_size, head_dim), torch.bfloat16)
        _check(v_cache, "v_cache", (k_cache.shape[0], n_kv_heads, head_dim, page_size), torch.bfloat16)
    q = torch.empty((M, n_heads, head_dim), dtype=torch.bfloat16, device=x.device)
    _call(load_module("gemm_bf16"), "ifx_qkv_rope", (P, P, I, I, P, I, P, P, P, I, I, I, I, P, P, P, I, I, P, I, F, F, P),
          x.data_ptr(), weight.tiled.data_ptr(), M, K, _ptr(bias), _dt(bias) if bias is not None else 0, _ptr(slots),
          cos.data_ptr(), sin.data_ptr(), n_heads, n_kv_heads, head_dim, page_size, q.data_ptr(), _ptr(k_cache),
          _ptr(v_cache), waves, unroll, *scale, _stream())
    return q


def skinny_gemm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                nt: int = 0, waves: int = 0, unroll: int = 0, swiglu_pairs: bool = False,
                tiled: Optional[torch.Tensor] = None, order: Optional[torch.Tensor] = None, tile_rows: int = 16,
                act: int = ACT_SILU) -> torch.Tensor:
    """bfloat16 x [M <= 64, K] times bfloat16 ``weight`` [N, K] transposed on the matrix cores, float
    accumulation, output bfloat16 or float32.  ``nt``, ``waves``, ``unroll`` = 0 lets the kernel choose.
    With ``swiglu_pairs`` the weight's rows alternate gate and up and the output is act(gate) * up [M, N/2] (``act``:
    ACT_SILU or ACT_GELU_TANH).  With ``tiled`` (``tile_weights(weight, order, tile_rows)``) the kernel streams that copy instead of the rows.
    ``x`` may be ``ScaledRows``."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.bfloat16)
    N = weight.shape[0]
    if tiled is not None:
        if tile_rows not in TILE_ROWS or (order is not None and tile_rows != 16):
            raise KernelError(f"skinny_gemm: {tile_rows} rows to a tile (one of {TILE_ROWS}; 16 with a tile order)")
        _check(tiled, "tiled", (_tiled_size(N, K, tile_rows),), torch.bfloat16)
    if M > SKINNY_MAX_M or K % 8:
        raise KernelError(f"skinny_gemm: M={M} must be <= {SKINNY_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and N % 2:
        raise KernelError("skinny_gemm: gate/up pairs need an even number of weight rows")
    out = torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    if order is not None and (tiled is None or swiglu_pairs):
        raise KernelError("skinny_gemm: a tile order goes with a tiled copy and a plain product")
    _call(load_module("gemm_bf16"), "ifx_skinny_gemm", _SKINNY_ARGS,
          x.data_ptr(), (weight if tiled is None else tiled).data_ptr(), out.data_ptr(), _DT[out_dtype], M, N, K, nt, waves,
          unroll, _GATED_EPILOGUE[act] if swiglu_pairs else 0, 0 if tiled is None else tile_rows, _ptr(order), *scale, 0, 0, 0, 0,
          1.0, _stream())
    return out


def wide_gemm(x, weight: LinearWeight, out_dtype: torch.dtype = torch.bfloat16, waves: int = 0,
              slices: int = 0, swiglu_pairs: bool = False, keep_slices: bool = False, act: int = ACT_SILU):
    """bfloat16 x [M <= 128, K] times ``weight`` transposed from its tiled copy, x shared through LDS by the waves
    of a workgroup: the product for 17-64 rows, for 65-128 rows of weights with few rows, and for 9-16 rows of large
    tall weights.  ``waves`` (4-16 per workgroup, 8 beyond 64 rows; one tile of weight rows each) and ``slices`` of K
    (added in a fixed order): 0 lets the kernel choose.  With ``keep_slices`` a product of several slices comes back as
    ``SliceSums``.  ``x`` may be ``ScaledRows`` (up to 16 rows)."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    N = weight.rows.shape[0]
    if weight.tiled is None or weight.rows.shape[1] != K or weight.rows.dtype != torch.bfloat16:
        raise KernelError(f"wide_gemm: needs the tiled copy of a bfloat16 [N, {K}] weight")
    if M > WIDE_MAX_M or K % 8:
        raise KernelError(f"wide_gemm: M={M} must be <= {WIDE_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and (N % 2 or weight.order is not None):
        raise KernelError("wide_gemm: gate/up pairs need an even number of weight rows in their natural order")
    mod = load_module("gemm_wide")
    if _tiled_size(N, K, weight.tile_rows) != weight.tiled.numel():
        raise KernelError(f"wide_gemm: the copy is not that of a [{N}, {K}] weight in tiles of {weight.tile_rows} rows")
    plan = mod.fn("ifx_wide_gemm_plan", (I, I, I, I, I, I, I))(M, N, K, waves, slices, 1 if swiglu_pairs else 0, weight.tile_rows)
    n_waves, n_slices = plan // 256, plan % 256
    part = torch.empty((n_slices, M, N), dtype=torch.float32, device=x.device) if n_slices > 1 else None
    keep = keep_slices and n_slices > 1
    out = None if keep else torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    _call(mod, "ifx_wide_gemm", (P, P, P, I, P, I, I, I, I, I, I, P, I, P, I, F, F, P),
          x.data_ptr(), weight.tiled.data_ptr(), _ptr(out), _DT[out_dtype], _ptr(part), M, N, K, n_waves, n_slices,
          _GATED_EPILOGUE[act] if swiglu_pairs else 0, _ptr(weight.order), weight.tile_rows, *scale, _stream())
    return SliceSums(part, out_dtype) if keep else out


def staged_gemm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                slices: int = 0, unroll: int = 0, swiglu_pairs: bool = False, act: int = ACT_SILU) -> torch.Tensor:
    """The same product as skinny_gemm with x staged in LDS and shared by the waves of a workgroup
    (64 weight rows per workgroup, K cut into ``slices``; 0 lets the kernel choose)."""
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.bfloat16)
    N = weight.shape[0]
    if M > SKINNY_MAX_M or K % 8:
        raise KernelError(f"staged_gemm: M={M} must be <= {SKINNY_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and N % 2:
        raise KernelError("staged_gemm: gate/up pairs need an even number of weight rows")
    mod = load_module("gemm_bf16")
    n_slices = 1 if swiglu_pairs else mod.fn("ifx_staged_gemm_slices", (I, I, I, I))(M, N, K, slices)
    part = torch.empty((n_slices, M, N), dtype=torch.float32, device=x.device) if n_slices > 1 else None
    out = torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    _call(mod, "ifx_staged_gemm", (P, P, P, I, P, I, I, I, I, I, I, P),
          x.data_ptr(), weight.data_ptr(), out.data_ptr(), _DT[out_dtype], _ptr(part), M, N, K, slices, unroll,
          _GATED_EPILOGUE[act] if swiglu_pairs else 0, _stream())
    return out


def linear(x: torch.Tensor, weight, out_dtype: Optional[torch.dtype] = None, keep_slices: bool = False):
    """x [M, K] times ``weight`` [N, K] transposed (a tensor or a ``LinearWeight``), chosen by the weight's
    type and by M.  With ``keep_slices`` the result may be ``SliceSums`` (the caller hands it to ``add_rmsnorm`` or
    ``rope_append``, or calls its ``sum()``).

    A float32 weight takes the true 32-bit kernel whatever the activation's type.  A bfloat16
    weight with bfloat16 activations takes the weight-streaming kernel for up to 64 rows and the
    library product with float accumulation beyond, as the reference does for every dense
    projection (runtime/backends/cuda/native/cublas_gemm.cpp:99-117).  float32 output (logits)
    always comes from float accumulators, never through a bfloat16 rounding.
    """
    tiled = order = None
    tile_rows = 16
    if isinstance(x, ScaledRows) and not takes_scaled_rows(x.shape[0], weight):
        raise KernelError(f"linear: scaled rows are not taken for {x.shape[0]} rows and this weight")
    if isinstance(weight, LinearWeight):
        weight, tiled, order, tile_rows = weight.rows, weight.tiled, weight.order, weight.tile_rows
    if weight.dtype == torch.float32:
        return gemm_f32(x, weight, None, out_dtype or x.dtype)
    if weight.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise KernelError(f"linear: weight {weight.dtype} with activation {x.dtype} is not supported")
    _check(x if not isinstance(x, ScaledRows) else x.rows, "x", (None, weight.shape[1]))
    _check(weight, "weight", (None, None))
    out_dtype = out_dtype or torch.bfloat16
    M, K = x.shape
    kind = _small_m_kernel(M, weight.shape[0], K, tiled is not None)
    if kind == "skinny":
        return skinny_gemm(x, weight, out_dtype, tiled=tiled, order=order, tile_rows=tile_rows)
    if kind == "wide":
        return wide_gemm(x, LinearWeight(weight, tiled, order, tile_rows), out_dtype, keep_slices=keep_slices)
    if kind == "staged":
        return staged_gemm(x, weight, out_dtype)
    if out_dtype == torch.float32:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    if keep_slices:
        S = library_k_slices(M, weight.shape[0], K)
        if S > 1 and not torch.cuda.is_current_stream_capturing():
            # K cut into S slices as one batched product of the library with float32 results: [S, M, N] partial sums
            xs = x.view(M, S, K // S).transpose(0, 1)
            ws = weight.view(weight.shape[0], S, K // S).permute(1, 2, 0)
            return SliceSums(torch.bmm(xs, ws, out_dtype=torch.float32), out_dtype)
    return torch.matmul(x, weight.t())


LIBRARY_SLICE_MIN_K = 2048      # k-values a slice of a library product keeps at least
LIBRARY_MAX_SLICES = 8


def library_k_slices(M: int, N: int, K: int) -> int:
    """Into how many slices of K a product that goes to the library is cut when the caller adds partial sums anyway.
    A product of many rows with a deep, narrow weight (down: 3,584 x 18,944) has few output tiles (the library's are
    about 256 x 256: 28 at 512 rows) and leaves most of the chip idle; cut into slices that still hold a few
    thousand k-values each, the same library fills it: at 512 rows 65 us instead of 124 (196 without tuning), at
    1,024 rows 112 instead of 188, at 2,048 rows 210 instead of 265.  A power of two, 1: not cut."""
    tiles = -(-M // 256) * -(-N // 256)
    S = 1
    while (2 * S <= LIBRARY_MAX_SLICES and 2 * S * tiles <= 256 and K % (16 * S) == 0
           and K // (2 * S) >= LIBRARY_SLICE_MIN_K):
        S *= 2
    return S


WIDE_FEW_ROWS_MIN_N = 16384               # rows of a weight (tall enough to fill the chip without slices of K) and ...
WIDE_FEW_ROWS_MIN_WEIGHT = 100_000_000    # ... its elements from which 9-16 rows take the product that shares x through LDS


def _tile_pairs_fit(N: int) -> bool:
    """Whether the product that splits K over a workgroup's waves takes the 16-row tiles of a weight of ``N`` rows in
    pairs (the rule of ifx_skinny_gemm: pairs halve its reads of x, and it takes them where they do not give the fullest
    of the 256 compute units more tiles than single tiles would)."""
    n_tiles = -(-N // 16)
    fullest = lambda nt: -(-(-(-n_tiles // nt)) // 256) * nt
    return -(-n_tiles // 2) >= 128 and fullest(2) <= fullest(1)


def _wide_for_few_rows(M: int, N: int, K: int) -> bool:
    """Whether up to 16 rows go to the product that shares x through LDS instead of the one that splits K over a
    workgroup's waves.  From 9 rows on the latter reads as much of x from the L2 as of W from memory; for large tall
    weights, which fill the chip without slices of K, the former then wins (both with the norm's factor per row; gate/up
    of the 7B shape at 9-16 rows 44.4 against 46.9 us, of the 14B shape 46 against 47-49, 32B 87 against 88-94 from 12
    rows, 72B 145 against 157-164; the heads of the 7B, 3B and 72B shapes from 12 rows: 177 against 185, 99 against 105
    and 385 against 414 at 16).  Where the other product cannot take tiles in pairs (gate/up of the 14B and 72B shapes)
    it reads x twice as often and loses from 6 rows on (14B 44.6 against 46.6-47.3 us at 6-8 rows, 72B 143-145 against
    146-149).  Smaller weights (gate/up of the 3B shape: 20 against 17 us) stay where they are."""
    if N < WIDE_FEW_ROWS_MIN_N:
        return _few_rows_in_slices(M, N, K)
    if N * K < WIDE_FEW_ROWS_MIN_WEIGHT:
        return False
    if M >= (12 if N >= 65536 else 9):
        return True
    return M >= 6 and N < 65536 and not _tile_pairs_fit(N)


UNEVEN_TILES_MIN_WEIGHT = 64_000_000      # elements from which a weight whose tiles lie unevenly on the chip is cut into slices of K


def _few_rows_in_slices(M: int, N: int, K: int) -> bool:
    """Whether 8-16 rows times a large weight of few rows go to the product that shares x through LDS and cuts K into slices
    (their sum left to the norm's kernel) instead of the one that adds into the stream itself.  The latter gives a
    workgroup whole row tiles: 5,120 rows are 320 tiles, two for 64 of the 256 compute units and one for the others,
    and the product takes as long as one of 8,192 rows (lower tiles do not help it: measured).  Slices of K fill the
    chip evenly whatever the number of tiles, at the price of the kernel that adds them (5.6 us).  down of the 32B shape
    (5,120 x 27,648) at 8 / 12 / 16 rows: 55 / 61 / 67 us against 43 + 5.6; of the 14B shape (5,120 x 13,824) 29 / 33 / 36
    against 24 + 5.6; its o (5,120 x 5,120: 14-17 against 11 + 5.6) is too small to gain, and weights whose tiles lie
    evenly (3,584 rows in tiles of 14, 8,192 rows) lose.  Decode steps: 8 requests at the 32B shape 13.4 -> 12.9 ms, 16 at
    the 14B shape 11.5 -> 11.3."""
    if M < (8 if N * K >= 2 * UNEVEN_TILES_MIN_WEIGHT else 9) or N * K < UNEVEN_TILES_MIN_WEIGHT:   # (8 rows: the smaller weight ties)
        return False
    tile_rows = choose_tile_rows(N)
    n_tiles = -(-N // tile_rows)
    return N < 0.7 * (-(-n_tiles // COMPUTE_UNITS) * COMPUTE_UNITS * tile_rows)


def _small_m_kernel(M: int, N: int, K: int, has_tiled: bool = False) -> Optional[str]:
    """Which of the streaming kernels takes a bfloat16 product of this shape, or None for the library.
    Measured on the 7B shapes: up to 16 rows the product that splits K over the waves of a workgroup (with x
    staged in LDS for very tall weights such as the head's when there is no tiled copy; 9-16 rows of large tall
    weights as from 17 rows, see _wide_for_few_rows); from 17 to 64 rows
    the product that shares x through LDS, which needs the tiled copy (without it, the first kernel up to 32
    rows on narrow weights); from 65 to 128 rows the same product for weights of few rows, whose K it cuts into
    slices to fill the chip where the library has too few output tiles to (down, o and q/k/v of the 7B shape:
    37-50, 15-21 and 16-22 us against 58-66, 30-34 and 30-37); beyond that, and for tall weights such as gate/up
    and the head, the library's tiles reuse the rows better."""
    if K % 8:
        return None
    if M <= 16:
        if has_tiled and _wide_for_few_rows(M, N, K):
            return "wide"
        return "staged" if N >= 65536 and not has_tiled else "skinny"
    if has_tiled and (M <= SKINNY_MAX_M or (M <= WIDE_MAX_M and N <= WIDE_MANY_ROWS_MAX_N)):
        return "wide"
    if M <= 32 and N <= 4096:
        return "skinny"
    return None


def linear_swiglu(x: torch.Tensor, weight_pairs, act: int = ACT_SILU, limit: float = 0.0) -> torch.Tensor:
    """act(x Wg^T) * (x Wu^T) (``act``: ACT_SILU, ACT_GELU_TANH, or ACT_CLAMPED_SWISH with its ``limit``, which is applied by
    a kernel of its own after the product whatever the number of rows) where ``weight_pairs`` [2I, K] (a tensor or a
    ``LinearWeight``) alternates the rows of Wg and Wu.  For few rows the activation is the product's epilogue; otherwise a second kernel
    applies it."""
    M, K = x.shape
    if isinstance(x, ScaledRows) and not takes_scaled_rows(M, weight_pairs):
        raise KernelError(f"linear_swiglu: scaled rows are not taken for {M} rows and this weight")
    rows, tiled, tile_rows = ((weight_pairs.rows, weight_pairs.tiled, weight_pairs.tile_rows) if isinstance(weight_pairs, LinearWeight)
                              else (weight_pairs, None, 16))
    if isinstance(weight_pairs, LinearWeight) and weight_pairs.order is not None:
        raise KernelError("linear_swiglu: a tile order is not supported for gate/up pairs")
    if act == ACT_CLAMPED_SWISH:
        return swiglu(linear(x, weight_pairs), interleaved=True, act=act, limit=limit)
    if rows.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
        kind = _small_m_kernel(M, rows.shape[0], K, tiled is not None)
        if kind == "skinny":
            return skinny_gemm(x, rows, torch.bfloat16, swiglu_pairs=True, tiled=tiled, tile_rows=tile_rows, act=act)
        if kind == "wide":
            return wide_gemm(x, weight_pairs, torch.bfloat16, swiglu_pairs=True, act=act)
        if kind == "staged":
            return staged_gemm(x, rows, torch.bfloat16, swiglu_pairs=True, act=act)
    return swiglu(linear(x, rows), interleaved=True, act=act)


# ----------------------------------------------------------------------------------------
def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, row_req: torch.Tensor,
                    positions: torch.Tensor, block_table: torch.Tensor, window: Optional[int],
                    scale: float, keep_first: int = 0, sink: Optional[float] = None,
                    gate: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None, chunk: Optional[int] = None,
                    differential: Optional[Tuple[float, float, float]] = None) -> torch.Tensor:
    """Causal (optionally windowed) attention of q [T, nH, d] over the paged cache (K [pages, nKV, page, d],
    V [pages, nKV, dv, page]; dv may differ from d); returns [T, nH*dv].  ``keep_first``: a windowed query also sees
    the first so many positions of its request; ``sink``: the score of a key without value that is added to the
    softmax's denominator (None: no such key), ``sinks`` float32 [nH]: such a score for every head; ``gate`` float32
    [T, nH]: a factor on every head's output; ``chunk``: a query sees only keys of its own block of that many positions,
    counted from the sequence's start.  ``differential`` (lambda, out_scale, eps): q and the keys hold two vectors of
    d / 2 elements per head, each pair a softmax map of its own over the same values; a head's output is map 1 minus
    lambda times map 2, divided by its root mean square (eps inside the root), times out_scale."""
    _check(q, "q", (None, None, None))
    T, nH, d = q.shape
    maps = 2 if differential is not None else 1
    if d % maps:
        raise KernelError(f"attention_plain: two maps need an even row, got {d}")
    lam, out_scale, norm_eps = differential if differential is not None else (0.0, 1.0, 0.0)
    if sinks is not None:
        _check(sinks, "sinks", (nH,), torch.float32)
    _check(k_cache, "k_cache", (None, None, None, d), q.dtype)
    n_pages, nKV, page_size, _ = k_cache.shape
    _check(v_cache, "v_cache", (n_pages, nKV, None, page_size), q.dtype)
    dv = v_cache.shape[2]
    _check(row_req, "row_req", (T,), torch.int32)
    _check(positions, "positions", (T,), torch.int32)
    _check(block_table, "block_table", (None, None), torch.int32)
    if gate is not None:
        _check(gate, "gate", (T, nH), torch.float32)
    out = torch.empty((T, nH * dv), dtype=q.dtype, device=q.device)
    _call(load_module("attn_plain"), "ifx_attn_plain", (P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, I, I, F, P, P, I, I, F, F, F, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _dt(q), row_req.data_ptr(),
          positions.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, nH, nKV, d // maps, dv, page_size,
          int(window or 0), float(scale), int(keep_first or 0), 0 if sink is None else 1, float(sink or 0.0), _ptr(gate),
          _ptr(sinks), int(chunk or 0), maps, float(lam), float(out_scale), float(norm_eps), _stream())
    return out


# ----------------------------------------------------------------------------------------
DELTA_THREAD_CHANNELS = (4, 8, 16, 32, 64)  # key channels of a column of S a thread may hold
DELTA_MAX_PADDED_DIM, DELTA_MAX_COLS, DELTA_THREADS = 256, 128, 256
DELTA_DECODE_MAX_CHANNELS = 8               # ... at most this many in steps of single tokens (64 decoded rows at 16 heads of 64 x 128: 62.8 us with 8, 70.2 with 16)


def delta_padded_dim(d: int) -> int:
    """The key channels of a head padded to a power of two (at least 4): what a column of S takes in a request's state."""
    p = 4
    while p < d:
        p *= 2
    if p > DELTA_MAX_PADDED_DIM:
        raise KernelError(f"delta rule: heads of {d} key channels (at most {DELTA_MAX_PADDED_DIM})")
    return p


def delta_layout(d: int, dv: int, single_tokens: bool = False) -> Tuple[int, int, int]:
    """(channels a thread, threads a column, columns a workgroup) of the delta rule's kernel for heads of ``d`` key channels
    and ``dv`` values.  The threads of a column are a power of two of neighbouring lanes that share the padded channels; a
    workgroup has up to 256 threads and a head's columns are dealt to as many workgroups as that takes.  The state's layout
    does not depend on the choice, so a step takes the one that suits it: a prompt's portion is a chain from token to token,
    which is shortest with the fewest channels a thread; steps of single tokens are many short workgroups, of which there
    should be few (``single_tokens``)."""
    dpad = delta_padded_dim(d)
    found = []
    for ch in DELTA_THREAD_CHANNELS:
        if ch > dpad or dpad // ch > 64:
            continue
        ks = dpad // ch
        cols = max(1, min(dv, DELTA_THREADS // ks, DELTA_MAX_COLS))
        threads = -(-cols * ks // 64) * 64
        if dpad <= threads and 2 * cols <= threads:         # (each thread fetches its share of a stage of sixteen tokens)
            found.append((ch, ks, cols))
    if not found:
        raise KernelError(f"delta rule: heads of {d} key channels and {dv} values fit no layout of the kernel")
    if single_tokens:
        few = [f for f in found if f[0] <= DELTA_DECODE_MAX_CHANNELS] or found
        return min(few, key=lambda f: (-(-dv // f[2]), f[0]))
    return found[0]


def delta_state_floats(n_heads: int, d: int, dv: int) -> int:
    delta_layout(d, dv)
    return n_heads * dv * delta_padded_dim(d)


def delta_rule(u: torch.Tensor, rows: torch.Tensor, cols: Tuple[int, int, int], A_log: torch.Tensor, dt_bias: torch.Tensor,
               norm_w: torch.Tensor, eps: float, n_heads: int, n_kv_heads: int, d: int, dv: int, state: torch.Tensor,
               state_offset: int, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
               single_tokens: bool = False) -> torch.Tensor:
    """The gated delta rule over a step's rows (see csrc/delta.hip).  ``u`` [T, >= 2 G d + H dv] holds per row the q heads,
    the k heads and the v heads (after their convolution), ``rows`` [T, ld] the gate's H dv columns from ``cols[0]``, beta's
    H from ``cols[1]`` and the decay's H from ``cols[2]``, both in the activation type.  ``A_log``, ``dt_bias`` float32 [H],
    ``norm_w`` [dv].  A request's S lies ``state_offset`` floats into its row of ``state`` [slots, n] (float32), zero for a
    request that starts.  ``single_tokens``: every request brings one row (the launch then takes few, larger workgroups).
    Returns [T, H dv] in u's type."""
    _check(u, "u", (None, None))
    T, ldu = u.shape
    _check(rows, "rows", (T, None), u.dtype)
    ldr = rows.shape[1]
    H, G = n_heads, n_kv_heads
    col_g, col_b, col_a = cols
    if ldu < 2 * G * d + H * dv or col_g + H * dv > ldr or col_b + H > ldr or col_a + H > ldr:
        raise KernelError("delta_rule: the rows are narrower than the columns named")
    _check(A_log, "A_log", (H,), torch.float32)
    _check(dt_bias, "dt_bias", (H,), torch.float32)
    _check(norm_w, "norm_w", (dv,))
    _check(state, "state", (None, None), torch.float32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _check(t, nm, (R,), torch.int32)
    ch, ks, cols = delta_layout(d, dv, single_tokens)
    if state_offset + H * dv * ch * ks > state.shape[1]:
        raise KernelError("delta_rule: the state rows are too short")
    out = torch.empty((T, H * dv), dtype=u.dtype, device=u.device)
    o_raw = torch.empty((T, H * dv), dtype=torch.float32, device=u.device)
    _call(load_module("delta"), "ifx_delta_rule", (P, I, P, I, I, I, I, I, P, P, P, I, F, P, LL, LL, P, P, P, P, P, I, I, I, I, I, I, I, I, I, P),
          u.data_ptr(), ldu, rows.data_ptr(), ldr, col_g, col_b, col_a, _dt(u), A_log.data_ptr(), dt_bias.data_ptr(),
          norm_w.data_ptr(), _dt(norm_w), float(eps), state.data_ptr(), state.shape[1], int(state_offset), q_start.data_ptr(),
          q_len.data_ptr(), slots.data_ptr(), out.data_ptr(), o_raw.data_ptr(), T, R, H, G, d, dv, ch, ks, cols, _stream())
    return out


def diff_expand(q: torch.Tensor) -> torch.Tensor:
    """q [T, H, 2 d] -> [T, 2 H, 2 d]: head 2 h is [q1 | 0], head 2 h + 1 is [0 | q2] (the two maps of differential attention as
    heads of their own against keys whose rows hold both maps' vectors)."""
    _check(q, "q", (None, None, None))
    T, H, two_d = q.shape
    if two_d % 2:
        raise KernelError("diff_expand: a row of two maps has an even number of elements")
    out = torch.empty((T, 2 * H, two_d), dtype=q.dtype, device=q.device)
    _call(load_module("rowwise"), "ifx_diff_expand", (P, P, I, LL, I, P), q.data_ptr(), out.data_ptr(), _dt(q), T * H, two_d // 2, _stream())
    return out


def diff_combine(a: torch.Tensor, n_heads: int, dv: int, lam: float, out_scale: float, eps: float) -> torch.Tensor:
    """a [T, 2 H dv] (per head the two maps' outputs, one after the other) -> [T, H dv]: o = a1 - lam a2, divided by its root
    mean square over dv (eps inside the root), times out_scale."""
    _check(a, "a", (None, 2 * n_heads * dv))
    T = a.shape[0]
    out = torch.empty((T, n_heads * dv), dtype=a.dtype, device=a.device)
    _call(load_module("rowwise"), "ifx_diff_combine", (P, P, I, LL, I, F, F, F, P), a.data_ptr(), out.data_ptr(), _dt(a), T * n_heads, dv,
          float(lam), float(out_scale), float(eps), _stream())
    return out


def stream_add(stream: torch.Tensor, rows: Optional[torch.Tensor] = None, vec: Optional[torch.Tensor] = None) -> torch.Tensor:
    """stream [T, H] (float32) += rows [T, H] (float32) + vec [H], in place; either operand may be None."""
    _check(stream, "stream", (None, None), torch.float32)
    T, H = stream.shape
    if rows is not None:
        _check(rows, "rows", (T, H), torch.float32)
    if vec is not None:
        _check(vec, "vec", (H,))
    _call(load_module("rowwise"), "ifx_stream_add", (P, P, P, I, I, I, P), stream.data_ptr(), _ptr(rows), _ptr(vec),
          _dt(vec) if vec is not None else 0, T, H, _stream())
    return stream


# ----------------------------------------------------------------------------------------
def causal_conv_silu(x: torch.Tensor, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                     row_req: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """silu of a causal convolution per channel over each request's rows: the first ``channels`` columns of ``x``
    [T, >= channels] with ``weight`` [channels, taps] (the last column is the current token's) and ``bias``.  A request's
    last taps - 1 inputs live in the first channels * (taps - 1) floats of its row of ``state`` [slots, n] (float32,
    zero for a request that starts), are read as the inputs before this step's and replaced by this step's last.
    ``row_req`` [T], ``q_start`` / ``q_len`` / ``slots`` [R] (int32) describe the step.  Returns [T, channels]."""
    _check(x, "x", (None, None))
    T, ld = x.shape
    _check(weight, "weight", (channels, None))
    taps = weight.shape[1]
    if bias is not None:
        _check(bias, "bias", (channels,), weight.dtype)
    _check(state, "state", (None, None), torch.float32)
    _check(row_req, "row_req", (T,), torch.int32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _check(t, nm, (R,), torch.int32)
    out = torch.empty((T, channels), dtype=x.dtype, device=x.device)
    _call(load_module("ssm"), "ifx_causal_conv", (P, I, I, P, P, I, P, LL, P, P, P, P, P, I, I, I, I, P),
          x.data_ptr(), _dt(x), ld, weight.data_ptr(), _ptr(bias), _dt(weight), state.data_ptr(), state.shape[1],
          row_req.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), slots.data_ptr(), out.data_ptr(), T, R, channels, taps, _stream())
    return out


def selective_scan(u: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, A: torch.Tensor, bc: torch.Tensor,
                   D: torch.Tensor, z: torch.Tensor, state: torch.Tensor, state_offset: int, q_start: torch.Tensor,
                   q_len: torch.Tensor, slots: torch.Tensor, chunks: Optional[Dict[str, object]] = None) -> torch.Tensor:
    """The recurrence of a selective state-space mixer over each request's rows, then the gate:
    dt = softplus(dt_raw + dt_bias); S[c, n] <- exp(dt A[c, n]) S[c, n] + dt u[c] B[n]; y[c] = sum_n S[c, n] C[n] + D[c] u[c];
    out = y * silu(z).  ``u`` [T, C], ``dt_raw`` float32 [T, C], ``A`` float32 [C, N] (negative), ``bc`` [T, >= 2N] with B
    then C, ``z`` a view [T, C] of rows that may be wider (its row stride is taken), ``state`` float32 [slots, n] with a
    request's S at ``state_offset`` of its row.  All of the recurrence is float.  Returns [T, C] in u's type.

    ``chunks`` (from ``scan_chunks``): the requests' rows cut into chunks that run side by side, each first from a zero
    state, then from the state that the chunks before it leave (the recurrence is linear in S); the same function up to
    the rounding of float sums taken in another order."""
    _check(u, "u", (None, None))
    T, C = u.shape
    _check(dt_raw, "dt_raw", (T, C), torch.float32)
    _check(A, "A", (C, None), torch.float32)
    N = A.shape[1]
    _check(dt_bias, "dt_bias", (C,))
    _check(D, "D", (C,), dt_bias.dtype)
    _check(bc, "bc", (T, None), u.dtype)
    if not (isinstance(z, torch.Tensor) and z.is_cuda and z.dtype == u.dtype and tuple(z.shape) == (T, C) and z.stride(1) == 1):
        raise KernelError("selective_scan: z must be a [T, C] view with contiguous rows in u's type")
    _check(state, "state", (None, None), torch.float32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _check(t, nm, (R,), torch.int32)
    out = torch.empty((T, C), dtype=u.dtype, device=u.device)
    n_chunks, max_chunk, lists = 0, 0, (0, 0, 0, 0, 0, 0)
    if chunks is not None:
        n_chunks, max_chunk = chunks["req"].shape[0], int(chunks["rows"])
        for nm in ("req", "t0", "len"):
            _check(chunks[nm], f"chunks.{nm}", (n_chunks,), torch.int32)
        _check(chunks["req_chunk0"], "chunks.req_chunk0", (R + 1,), torch.int32)
        chunk_state = torch.empty((n_chunks, C, N), dtype=torch.float32, device=u.device)
        chunk_dt = torch.empty((n_chunks, C), dtype=torch.float32, device=u.device)
        lists = (chunks["req"].data_ptr(), chunks["t0"].data_ptr(), chunks["len"].data_ptr(), chunks["req_chunk0"].data_ptr(),
                 chunk_state.data_ptr(), chunk_dt.data_ptr())
    _call(load_module("ssm"), "ifx_selective_scan",
          (P, I, P, P, P, P, I, P, I, P, I, P, LL, LL, P, P, P, P, I, I, I, I, I, I, P, P, P, P, P, P, P),
          u.data_ptr(), _dt(u), dt_raw.data_ptr(), dt_bias.data_ptr(), A.data_ptr(), bc.data_ptr(), bc.shape[1], D.data_ptr(),
          _dt(D), z.data_ptr(), z.stride(0) if T else C, state.data_ptr(), state.shape[1], int(state_offset), q_start.data_ptr(),
          q_len.data_ptr(), slots.data_ptr(), out.data_ptr(), T, R, C, N, n_chunks, max_chunk, *lists, _stream())
    return out


def scan_chunks(q_start, q_len, chunk: int, device) -> Dict[str, object]:
    """The lists ``selective_scan`` takes as ``chunks``: every request's rows (host arrays ``q_start`` / ``q_len`` of the
    step) cut into chunks of up to ``chunk`` rows, in one upload."""
    import numpy as np
    req, t0, ln, first = [], [], [], [0]
    for r, (s0, n) in enumerate(zip(q_start.tolist(), q_len.tolist())):
        for at in range(0, n, chunk):
            req.append(r); t0.append(s0 + at); ln.append(min(chunk, n - at))
        first.append(len(req))
    n = len(req)
    pad = lambda v: v + [0] * (-len(v) % 4)
    packed = torch.from_numpy(np.asarray(pad(req) + pad(t0) + pad(ln) + first, dtype=np.int32)).to(device)
    w = n + -n % 4
    return {"req": packed[:n], "t0": packed[w:w + n], "len": packed[2 * w:2 * w + n], "req_chunk0": packed[3 * w:3 * w + len(first)],
            "rows": int(chunk)}       # (the most rows a chunk has: the kernels keep a chunk's B and C in LDS)


# ----------------------------------------------------------------------------------------
GLA_THREAD_CHANNELS = ((16, 512), (32, 1024), (64, 512), (128, 256))   # channels of S a thread may hold, and the threads a workgroup may then have


def gla_layout(d: int, dv: int) -> Tuple[int, int]:
    """(channels a thread holds, threads per column) for a head of d key channels and dv values: the first pairing whose
    workgroup (dv columns times the threads of a column) fits; failing that, the first in which a thread holds several
    columns (4 with 16 channels, 2 with 32: what its registers take).  A request's S takes heads * dv * parts * channels
    floats."""
    def parts_for(dp):
        parts = 1
        while parts * dp < d:
            parts *= 2
        return parts
    for dp, max_threads in GLA_THREAD_CHANNELS:
        parts = parts_for(dp)
        if parts <= 64 and max(dv * parts, d) <= max_threads:     # (a thread per key channel loads a stage's q, k and decays)
            return dp, parts
    for dp, cols in ((16, 4), (32, 2)):
        parts = parts_for(dp)
        if parts <= 64 and max(-(-dv // cols) * parts, d) <= 1024:
            return dp, parts
    raise KernelError(f"gla: a head of {d} key channels and {dv} values does not fit a workgroup")


def gla_state_floats(n_heads: int, d: int, dv: int) -> int:
    dp, parts = gla_layout(d, dv)
    return n_heads * dv * parts * dp


def gla_scan(rows: torch.Tensor, cols: Tuple[int, int, int, int], z: torch.Tensor, z_bias: Optional[torch.Tensor], tau: float,
             q_scale: float, norm_weight: torch.Tensor, eps: float, n_heads: int, d: int, dv: int, state: torch.Tensor,
             state_offset: int, q_start: torch.Tensor, q_len: torch.Tensor, slots: torch.Tensor,
             chunks: Optional[Dict[str, object]] = None) -> torch.Tensor:
    """Gated linear attention over each request's rows, with the output's norm and gate:
    alpha = sigmoid(z + z_bias) ^ (1 / tau) per key channel; per head S <- diag(alpha) S + k v^T; o = S^T q * q_scale;
    y = o / sqrt(mean(o^2) + eps) * norm_weight * silu(g).  ``rows`` [T, ld] holds q, k (n_heads * d each), v and g
    (n_heads * dv each) at the columns ``cols`` = (q, k, v, g); ``z`` float32 [T, n_heads * d]; ``state`` float32
    [slots, n] with a request's S (``gla_state_floats`` numbers, laid out for the kernel) at ``state_offset`` of its row.
    Decays, S, o, norm and gate are float.  Returns y [T, n_heads * dv] in the rows' type.

    ``chunks`` (from ``scan_chunks``): the requests' rows cut into chunks that run side by side, first from a zero state,
    then from the state the chunks before leave (the recurrence is linear in S); the same function up to the rounding of
    float sums taken in another order."""
    _check(rows, "rows", (None, None))
    T, ld = rows.shape
    HD, HV = n_heads * d, n_heads * dv
    q_col, k_col, v_col, g_col = (int(c) for c in cols)
    for c, w, nm in ((q_col, HD, "q"), (k_col, HD, "k"), (v_col, HV, "v"), (g_col, HV, "g")):
        if c < 0 or c + w > ld:
            raise KernelError(f"gla_scan: the {nm} columns {c}..{c + w} lie outside rows of {ld}")
    _check(z, "z", (T, HD), torch.float32)
    if z_bias is not None:
        _check(z_bias, "z_bias", (HD,), torch.float32)
    _check(norm_weight, "norm_weight", (dv,))
    _check(state, "state", (None, None), torch.float32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (slots, "slots")):
        _check(t, nm, (R,), torch.int32)
    dp, parts = gla_layout(d, dv)
    out = torch.empty((T, HV), dtype=rows.dtype, device=rows.device)
    n_chunks, lists = 0, (0, 0, 0, 0, 0, 0)
    if chunks is not None:
        n_chunks = chunks["req"].shape[0]
        for nm in ("req", "t0", "len"):
            _check(chunks[nm], f"chunks.{nm}", (n_chunks,), torch.int32)
        _check(chunks["req_chunk0"], "chunks.req_chunk0", (R + 1,), torch.int32)
        chunk_state = torch.empty((n_chunks, HV * parts * dp), dtype=torch.float32, device=rows.device)
        chunk_loga = torch.empty((n_chunks, HD), dtype=torch.float32, device=rows.device)
        lists = (chunks["req"].data_ptr(), chunks["t0"].data_ptr(), chunks["len"].data_ptr(), chunks["req_chunk0"].data_ptr(),
                 chunk_state.data_ptr(), chunk_loga.data_ptr())
    _call(load_module("gla"), "ifx_gla_scan",
          (P, I, I, I, I, I, I, P, P, F, F, F, P, I, P, LL, LL, P, P, P, P, I, I, I, I, I, I, I, I, P, P, P, P, P, P, P),
          rows.data_ptr(), _dt(rows), ld, q_col, k_col, v_col, g_col, z.data_ptr(), _ptr(z_bias), 1.0 / float(tau), float(q_scale),
          float(eps), norm_weight.data_ptr(), _dt(norm_weight), state.data_ptr(), state.shape[1], int(state_offset),
          q_start.data_ptr(), q_len.data_ptr(), slots.data_ptr(), out.data_ptr(), T, R, n_heads, d, dv, dp, parts, n_chunks,
          *lists, _stream())
    return out


HYPER_MAX_STREAMS = 8


def hyper_step(src: torch.Tensor, n_streams: int, y=None, mix: Optional[torch.Tensor] = None, out_weights: Optional[torch.Tensor] = None,
               in_weights: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
               out_dtype: Optional[torch.dtype] = None, y_scale: float = 1.0):
    """One step of hyper-connections on the streams of a step's rows, in float.

    ``src`` float32: the streams [T, S, H], or one stream [T, H] that all S start as.  With ``y`` [T, H] (a tensor of any
    activation type or ``SliceSums``) the streams become x_t <- sum_s mix[s, t] x_s + out_weights[t] * y * y_scale, in
    place (copies of a single stream are written to a new tensor).  With ``in_weights`` the sub-block that follows reads
    u = sum_t in_weights[t] x_t of the new streams: returned normalised, u / sqrt(mean(u^2) + eps) * norm_weight in
    ``out_dtype``, or as it is in float32 without ``norm_weight``.  Returns (streams, rows or None)."""
    S = int(n_streams)
    single = src.dim() == 2
    if single:
        _check(src, "src", (None, None), torch.float32)
        T, H = src.shape
    else:
        _check(src, "src", (None, S, None), torch.float32)
        T, _, H = src.shape
    if not 0 < S <= HYPER_MAX_STREAMS:
        raise KernelError(f"hyper_step: {S} streams (1 to {HYPER_MAX_STREAMS})")
    for t, nm, shape in ((mix, "mix", (S, S)), (out_weights, "out_weights", (S,)), (in_weights, "in_weights", (S,))):
        if t is not None:
            _check(t, nm, shape, torch.float32)
    n_slices, stride, y_ptr, y_dt = 1, 0, 0, 0
    if y is not None:
        if mix is None or out_weights is None:
            raise KernelError("hyper_step: an update needs the mixing matrix and the output weights")
        if isinstance(y, SliceSums):
            _check(y.parts, "y", (None, T, H), torch.float32)
            n_slices, stride, y_ptr, y_dt = y.parts.shape[0], T * H, y.parts.data_ptr(), DT_F32
        else:
            _check(y, "y", (T, H))
            y_ptr, y_dt = y.data_ptr(), _dt(y)
    dst = torch.empty((T, S, H), dtype=torch.float32, device=src.device) if single else src
    rows = None
    if in_weights is not None:
        if norm_weight is not None:
            _check(norm_weight, "norm_weight", (H,))
            rows = torch.empty((T, H), dtype=out_dtype or torch.float32, device=src.device)
        else:
            rows = torch.empty((T, H), dtype=torch.float32, device=src.device)
    _call(load_module("hyper"), "ifx_hyper_step", (P, I, P, P, I, I, LL, F, P, P, P, P, I, F, P, I, I, I, I, P),
          src.data_ptr(), 1 if single else 0, dst.data_ptr(), y_ptr, y_dt, n_slices, stride, float(y_scale), _ptr(mix), _ptr(out_weights),
          _ptr(in_weights), _ptr(norm_weight), _dt(norm_weight) if norm_weight is not None else 0, float(eps), _ptr(rows),
          _DT[rows.dtype] if rows is not None else 0, T, S, H, _stream())
    return dst, rows


def linear_act(x, weight, act: int) -> torch.Tensor:
    """act(x W^T) for a feed-forward without a gate (``act``: ACT_SILU or ACT_GELU_TANH, formed in float on the product's
    output)."""
    return activation(linear(x, weight, keep_slices=True), act)


def activation(x, act: int) -> torch.Tensor:
    """act(x) element by element in float: ACT_SILU or ACT_GELU_TANH (a feed-forward without a gate).  ``x`` may be
    ``SliceSums``: the partial sums are added in slice order first, and the result has the type they stand for."""
    if isinstance(x, SliceSums):
        parts = x.parts
        _check(parts, "x", (None, None, None), torch.float32)
        n = parts.shape[1] * parts.shape[2]
        if n % 4:
            return activation(x.sum(x.dtype), act)
        out = torch.empty(parts.shape[1:], dtype=x.dtype, device=parts.device)
        _call(load_module("rowwise"), "ifx_activation_slices", (P, I, LL, P, I, LL, I, P), parts.data_ptr(), parts.shape[0], n,
              out.data_ptr(), _DT[x.dtype], n, int(act), _stream())
        return out
    _check(x, "x")
    out = torch.empty_like(x)
    _call(load_module("rowwise"), "ifx_activation", (P, P, I, LL, I, P), x.data_ptr(), out.data_ptr(), _dt(x), x.numel(), int(act), _stream())
    return out


def sigmoid_gate(x: torch.Tensor, rows, g_col: int) -> torch.Tensor:
    """x [T, C] times sigmoid of the columns ``g_col`` .. ``g_col`` + C - 1 of ``rows`` [T, ld] (x's type, or ``SliceSums``),
    element by element, the sigmoid in float."""
    _check(x, "x", (None, None))
    T, C = x.shape
    n_slices, stride = 1, 0
    if isinstance(rows, SliceSums):
        _check(rows.parts, "rows", (None, T, None), torch.float32)
        n_slices, ld, stride, ptr = rows.parts.shape[0], rows.parts.shape[2], T * rows.parts.shape[2], rows.parts.data_ptr()
    else:
        _check(rows, "rows", (T, None), x.dtype)
        ld, ptr = rows.shape[1], rows.data_ptr()
    if g_col < 0 or g_col + C > ld:
        raise KernelError(f"sigmoid_gate: columns {g_col}..{g_col + C} lie outside rows of {ld}")
    out = torch.empty_like(x)
    _call(load_module("rowwise"), "ifx_sigmoid_gate", (P, P, I, I, I, LL, P, I, I, I, P),
          x.data_ptr(), ptr, ld, int(g_col), n_slices, stride, out.data_ptr(), _dt(x), T, C, _stream())
    return out


def gated_add(base, extra, h: torch.Tensor, gate_weight: Optional[torch.Tensor]) -> torch.Tensor:
    """base + sigmoid(h . gate_weight) * extra row by row: ``base`` and ``extra`` [T, N] (h's type, or ``SliceSums``, which are
    added in slice order), ``h`` [T, K], ``gate_weight`` [K] (one number per row, formed in float; None: the gate is 1, and
    ``h`` only says the type and the number of rows).  Returns [T, N] in h's type."""
    _check(h, "h", (None, None))
    T, K = h.shape
    if gate_weight is not None:
        _check(gate_weight, "gate_weight", (K,), h.dtype)

    def operand(v, nm):
        if isinstance(v, SliceSums):
            _check(v.parts, nm, (None, T, None), torch.float32)
            return v.parts.data_ptr(), 1, v.parts.shape[0], T * v.parts.shape[2], v.parts.shape[2]
        _check(v, nm, (T, None), h.dtype)
        return v.data_ptr(), 1 if v.dtype == torch.float32 else 0, 1, 0, v.shape[1]

    bp, bf, bn, bs, N = operand(base, "base")
    ep, ef, en, es, N2 = operand(extra, "extra")
    if N != N2:
        raise KernelError(f"gated_add: base is {N} wide, extra {N2}")
    out = torch.empty((T, N), dtype=h.dtype, device=h.device)
    _call(load_module("rowwise"), "ifx_gated_add", (P, I, I, LL, P, I, I, LL, P, P, I, P, I, I, I, P),
          bp, bf, bn, bs, ep, ef, en, es, h.data_ptr(), _ptr(gate_weight), K, out.data_ptr(), _dt(h), T, N, _stream())
    return out


def scale_softcap(logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """In place on float32 ``logits``: x <- x * scale, then (cap > 0) x <- cap * tanh(x / cap)."""
    _check(logits, "logits", None, torch.float32)
    _call(load_module("rowwise"), "ifx_scale_softcap", (P, LL, F, F, P), logits.data_ptr(), logits.numel(), float(scale), float(cap or 0.0), _stream())
    return logits


WIDE_MAX_K_DIM, WIDE_MAX_V_DIM = 1024, 512
WIDE_DIMS_PREBUILT = ((576, 512),)      # compiled ahead by build_all(); any other pair of widths when a model first needs it


def wide_attention_supported(dtype: torch.dtype, n_kv_heads: int, k_dim: int, v_dim: int, page_size: int) -> bool:
    """Whether ``attention_wide`` takes this cache: bfloat16, one kv head that all query heads share, keys of a multiple
    of 8 and values of a multiple of 16 elements, pages of a power of two from 16."""
    return (dtype == torch.bfloat16 and n_kv_heads == 1 and k_dim % 8 == 0 and 0 < k_dim <= WIDE_MAX_K_DIM and v_dim % 16 == 0
            and 0 < v_dim <= WIDE_MAX_V_DIM and page_size >= 16 and page_size & (page_size - 1) == 0)


def wide_launch_shape(n_rows: int, n_heads: int, max_kv: int):
    """(keys per split, splits) of a launch of ``attention_wide``: one wave per (row, 16 heads, split), splits as long as
    still give the chip about 2,048 waves, and no shorter than 64 keys."""
    groups = -(-n_heads // 16)
    splits = max(1, min(2048 // max(n_rows * groups, 1), -(-max_kv // 64)))
    chunk = max(64, -(-(-(-max_kv // splits)) // 32) * 32)
    return chunk, max(1, -(-max_kv // chunk))


def attention_wide(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, row_req: torch.Tensor, positions: torch.Tensor,
                   block_table: torch.Tensor, window: Optional[int], scale: float, chunk: int, max_splits: int,
                   sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal (optionally windowed) attention of q [T, nH, d] over one shared kv head with keys of d and values of dv
    elements (K [pages, 1, page, d], V [pages, 1, dv, page]) on the matrix cores, for widths the other matrix-core kernels
    do not take; returns [T, nH * dv].  Every row's keys are cut into splits of ``chunk`` (``max_splits`` * chunk must
    reach past the largest position) and merged by a second launch.  ``sinks`` float32 [nH]: a score per head that joins
    its softmax's denominator."""
    _check(q, "q", (None, None, None), torch.bfloat16)
    T, nH, d = q.shape
    if sinks is not None:
        _check(sinks, "sinks", (nH,), torch.float32)
    _check(k_cache, "k_cache", (None, 1, None, d), torch.bfloat16)
    n_pages, _, page_size, _ = k_cache.shape
    _check(v_cache, "v_cache", (n_pages, 1, None, page_size), torch.bfloat16)
    dv = v_cache.shape[2]
    if not wide_attention_supported(q.dtype, 1, d, dv, page_size):
        raise KernelError(f"attention_wide: keys of {d} (a multiple of 8 up to {WIDE_MAX_K_DIM}), values of {dv} (of 16 up to "
                          f"{WIDE_MAX_V_DIM}), pages of {page_size} (a power of two from 16)")
    _check(row_req, "row_req", (T,), torch.int32)
    _check(positions, "positions", (T,), torch.int32)
    _check(block_table, "block_table", (None, None), torch.int32)
    out = torch.empty((T, nH * dv), dtype=torch.bfloat16, device=q.device)
    part_o = torch.empty((T, nH, max_splits, dv), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((T, nH, max_splits, 2), dtype=torch.float32, device=q.device)
    _call(load_module("attn_wide", (("K_DIM", d), ("V_DIM", dv))), "ifx_attn_wide",
          (P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, F, P, P, P, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), 0, row_req.data_ptr(), positions.data_ptr(),
          block_table.data_ptr(), block_table.shape[1], T, nH, d, dv, page_size, int(window or 0), int(chunk), int(max_splits),
          float(scale), part_o.data_ptr(), part_ml.data_ptr(), _ptr(sinks), _stream())
    return out


def mfma_attention_supported(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= MFMA_MAX_HEAD_DIM
            and page_size >= 16 and page_size & (page_size - 1) == 0)


def _attn_common(q, k_cache, v_cache, qt=1, direct=True):
    _check(q, "q", (None, None, None), torch.bfloat16)
    T, nH, d = q.shape
    _check(k_cache, "k_cache", (None, None, None, d), torch.bfloat16)
    n_pages, nKV, page_size, _ = k_cache.shape
    _check(v_cache, "v_cache", (n_pages, nKV, d, page_size), torch.bfloat16)
    if not mfma_attention_supported(q.dtype, d, page_size):
        raise KernelError(f"matrix-core attention needs bfloat16, head_dim a multiple of 16 up to {MFMA_MAX_HEAD_DIM} and "
                          f"page_size a power of two from 16; got head_dim {d}, page_size {page_size}")
    name, variant, _, _ = _tile_module(d, qt, direct)
    return T, nH, d, nKV, page_size, load_module(name, variant)


def _attn_extras(T, nH, keep_first, sink, gate, sinks=None, block=None):
    """The six optional arguments of the matrix-core attention kernels: kept first keys, whether there is a sink, its
    score, the gate's pointer, the pointer to a sink score per head, the size of the blocks a row sees its own of."""
    if gate is not None:
        _check(gate, "gate", (T, nH), torch.float32)
    if sinks is not None:
        _check(sinks, "sinks", (nH,), torch.float32)
    return int(keep_first or 0), 0 if sink is None else 1, float(sink or 0.0), _ptr(gate), _ptr(sinks), int(block or 0)


ROW_MAX_WAVES = 8


def row_waves_fit(n_heads: int, n_kv_heads: int, head_dim: int, waves: int) -> int:
    """The most waves per workgroup, up to ``waves``, whose results fit the row kernel's 64 KB of LDS."""
    nc = min(16, n_heads // n_kv_heads)
    while waves > 1 and waves * nc * (head_dim + 6) * 4 > 65536:
        waves //= 2
    return waves


def attention_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                   rows: Optional[torch.Tensor], n_rows: int, row_req: torch.Tensor, positions: torch.Tensor,
                   block_table: torch.Tensor, window: Optional[int], scale: float, chunk: int, max_splits: int,
                   waves: int = 0, req_is_row: bool = False, keep_first: int = 0, sink: Optional[float] = None,
                   gate: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None, block: Optional[int] = None) -> None:
    """Attention of single rows (``rows`` int32, or None for rows 0..n_rows-1) into ``out`` [T, nH*d].  ``keep_first``,
    ``sink``, ``gate``: as for ``attention_plain``.

    ``waves`` 0: split s of a row covers key positions [s*chunk, (s+1)*chunk), one wave each, and a second launch
    merges a row's splits; ``max_splits`` * chunk must reach past the largest position among the rows.
    ``waves`` 1-8: one workgroup of that many waves per (row, kv head) shares the row's keys evenly and writes the
    output itself (``chunk`` and ``max_splits`` are not used): for launches with pairs enough to fill the chip.
    ``req_is_row``: the caller vouches that ``row_req`` is 0, 1, 2, ... (every request brings one row), which lets
    a wave ask for its block-table entries before it knows anything else."""
    T, nH, d, nKV, page_size, mod = _attn_common(q, k_cache, v_cache)
    _check(out, "out", (T, nH * d), torch.bfloat16)
    _check(row_req, "row_req", (T,), torch.int32)
    _check(positions, "positions", (T,), torch.int32)
    _check(block_table, "block_table", (None, None), torch.int32)
    if rows is not None:
        _check(rows, "rows", (n_rows,), torch.int32)
    elif n_rows != T:
        raise KernelError("attention_rows: without a row list every row of the batch is handled")
    if not 0 <= waves <= ROW_MAX_WAVES or row_waves_fit(nH, nKV, d, waves) != waves:
        raise KernelError(f"attention_rows: {waves} waves per workgroup (0-{ROW_MAX_WAVES}, and their results within 64 KB of LDS: "
                          f"up to {row_waves_fit(nH, nKV, d, ROW_MAX_WAVES)} at these head counts)")
    part_o = part_ml = None
    if waves == 0:
        part_o = torch.empty((n_rows, nH, max_splits, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_rows, nH, max_splits, 2), dtype=torch.float32, device=q.device)
    if req_is_row and block_table.shape[0] < T:
        raise KernelError("attention_rows: req_is_row needs a block-table row for every row of the step")
    _call(mod, "ifx_attn_rows", (P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, F, P, P, I, I, I, I, F, P, P, I, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(rows), row_req.data_ptr(),
          positions.data_ptr(), block_table.data_ptr(), block_table.shape[1], n_rows, nH, nKV, d, page_size,
          int(window or 0), chunk, max_splits, float(scale), _ptr(part_o), _ptr(part_ml), waves, 1 if req_is_row else 0,
          *_attn_extras(T, nH, keep_first, sink, gate, sinks, block), _stream())


def attention_tile_rows(head_dim: int, qt: int = 1) -> int:
    """Rows per tile of the tile kernel in tiling ``qt`` (see TILE_QTS; the compiled module says the same; asking it
    would compile a variant that a short step never runs)."""
    return 64 * qt


def attention_tiles(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                    tile_req: torch.Tensor, tile_q0: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                    kv_len: torch.Tensor, block_table: torch.Tensor, window: Optional[int], scale: float,
                    qt: int = 1, chunk: int = 0, max_splits: int = 1, rows: Optional[torch.Tensor] = None,
                    row_req: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                    order: Optional[torch.Tensor] = None, keep_first: int = 0, sink: Optional[float] = None,
                    gate: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None, block: Optional[int] = None) -> None:
    """Attention of tiles of ``attention_tile_rows(d, qt)`` consecutive rows of one request each (tile t:
    request tile_req[t], rows from tile_q0[t] of that request's rows in this step) into ``out`` [T, nH*d].

    With ``max_splits`` > 1 every tile's keys are cut into splits of ``chunk`` keys (a multiple of 64;
    ``max_splits`` * chunk must reach past the largest position) that run as workgroups of their own, and
    the rows named by ``rows`` (int32: every row of every tiled request) are merged at the end; this
    needs the step's ``row_req`` and ``positions`` [T].

    ``order`` (int32 [8 * n], from ``attention.tile_order``) says which work item each workgroup of the launch
    takes; every item must appear exactly once (-1: a workgroup without work).  The result does not depend on it."""
    extras = bool(keep_first) or sink is not None or gate is not None or sinks is not None or bool(block)      # (the kernel that loads straight into LDS has none of them)
    T, nH, d, nKV, page_size, mod = _attn_common(q, k_cache, v_cache, qt, not extras)
    _, _, entry, rows_fn = _tile_module(d, qt, not extras)
    if mod.fn(rows_fn, ())() != attention_tile_rows(d, qt):
        raise KernelError("attention_tiles: the compiled module's tile rows differ from attention_tile_rows()")
    _check(out, "out", (T, nH * d), torch.bfloat16)
    n_tiles = tile_req.shape[0]
    _check(tile_req, "tile_req", (n_tiles,), torch.int32)
    _check(tile_q0, "tile_q0", (n_tiles,), torch.int32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (kv_len, "kv_len")):
        _check(t, nm, (R,), torch.int32)
    _check(block_table, "block_table", (R, None), torch.int32)
    part_o = part_ml = None
    n_rows = 0
    if max_splits > 1:
        if chunk <= 0 or chunk % 64:
            raise KernelError(f"attention_tiles: splits need a chunk that is a multiple of 64, got {chunk}")
        if rows is None or row_req is None or positions is None:
            raise KernelError("attention_tiles: splits need the rows to merge, row_req and positions")
        n_rows = rows.shape[0]
        _check(rows, "rows", (n_rows,), torch.int32)
        _check(row_req, "row_req", (T,), torch.int32)
        _check(positions, "positions", (T,), torch.int32)
        part_o = torch.empty((T, nH, max_splits, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nH, max_splits, 2), dtype=torch.float32, device=q.device)
    per_xcd = 0
    if order is not None:
        _check(order, "order", (None,), torch.int32)
        if order.shape[0] % N_XCD:
            raise KernelError(f"attention_tiles: the order has a place for each of {N_XCD} XCDs' workgroups")
        per_xcd = order.shape[0] // N_XCD
    args = (q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), tile_req.data_ptr(), tile_q0.data_ptr(),
            n_tiles, q_start.data_ptr(), q_len.data_ptr(), kv_len.data_ptr(), block_table.data_ptr(),
            block_table.shape[1], nH, nKV, d, page_size, int(window or 0), float(scale), int(chunk), int(max_splits),
            _ptr(part_o), _ptr(part_ml), _ptr(rows), n_rows, _ptr(row_req), _ptr(positions), _ptr(order), per_xcd, N_XCD)
    types = (P, P, P, P, P, P, I, P, P, P, P, I, I, I, I, I, I, F, I, I, P, P, P, I, P, P, P, I, I)
    if entry == "ifx_attn_tiles":
        _call(mod, entry, types + (I, I, F, P, P, I, P), *args, *_attn_extras(T, nH, keep_first, sink, gate, sinks, block), _stream())
    else:
        _call(mod, entry, types + (P,), *args, _stream())


# ----------------------------------------------------------------------------------------
def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index of the maximum of each row of float32 ``logits`` [R, V]; int32 [R]."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    pv = torch.empty((R, 32), dtype=torch.float32, device=logits.device)
    pi = torch.empty((R, 32), dtype=torch.int32, device=logits.device)
    _call(load_module("sampling"), "ifx_argmax", (P, I, I, P, P, P, P), logits.data_ptr(), R, V, out.data_ptr(),
          pv.data_ptr(), pi.data_ptr(), _stream())
    return out


def apply_penalties(logits: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor,
                    rep: torch.Tensor, freq: torch.Tensor, pres: torch.Tensor) -> None:
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    n = rows.shape[0]
    for t, nm in ((rows, "rows"), (ids, "ids"), (counts, "counts")):
        _check(t, nm, (n,), torch.int32)
    for t, nm in ((rep, "rep"), (freq, "freq"), (pres, "pres")):
        _check(t, nm, (R,), torch.float32)
    _call(load_module("sampling"), "ifx_apply_penalties", (P, I, P, P, P, I, P, P, P, P),
          logits.data_ptr(), V, rows.data_ptr(), ids.data_ptr(), counts.data_ptr(), n, rep.data_ptr(),
          freq.data_ptr(), pres.data_ptr(), _stream())


def add_logit_bias(logits: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, bias: torch.Tensor) -> None:
    _check(logits, "logits", (None, None), torch.float32)
    n = rows.shape[0]
    _check(rows, "rows", (n,), torch.int32)
    _check(ids, "ids", (n,), torch.int32)
    _check(bias, "bias", (n,), torch.float32)
    _call(load_module("sampling"), "ifx_add_logit_bias", (P, I, P, P, P, I, P),
          logits.data_ptr(), logits.shape[1], rows.data_ptr(), ids.data_ptr(), bias.data_ptr(), n, _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: Optional[torch.Tensor] = None, draws: Optional[torch.Tensor] = None,
           any_greedy: bool = True, any_filters: bool = True) -> torch.Tensor:
    """One token per row of float32 ``logits`` [R, V]; rows with temperature <= 0 take the argmax (``any_greedy``
    False: the caller knows that there is no such row; ``any_filters`` False: that no row has top-k or top-p; both
    save launches that would find nothing to do).  The number in
    [0, 1) that a row's draw uses is either given (``uniform`` [R]) or made by the kernel from ``draws`` (int32
    [R, 4]: the row's seed and the count of its draws so far, 64 bits each, low word first), as
    ``sampling.params.philox_uniform`` makes it."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    _check(temperature, "temperature", (R,), torch.float32)
    _check(top_k, "top_k", (R,), torch.int32)
    _check(top_p, "top_p", (R,), torch.float32)
    _check(min_p, "min_p", (R,), torch.float32)
    if (uniform is None) == (draws is None):
        raise KernelError("sample: either uniform numbers or seeds and counters")
    if uniform is not None:
        _check(uniform, "uniform", (R,), torch.float32)
    else:
        _check(draws, "draws", (R, 4), torch.int32)
    mod = load_module("sampling")
    weights = torch.empty_like(logits)
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    # large vocabularies are drawn by several workgroups a row, which hand each other their results in scratch memory
    n_scratch = mod.fn("ifx_sample_scratch_blocks", (I, I, I))(R, V, 1 if any_filters else 0)
    scratch = torch.empty((n_scratch * 256,), dtype=torch.uint8, device=logits.device) if n_scratch else None
    _call(mod, "ifx_sample", (P, P, P, P, P, P, P, P, P, I, I, P, I, I, P),
          logits.data_ptr(), weights.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
          min_p.data_ptr(), uniform.data_ptr() if uniform is not None else None,
          draws.data_ptr() if draws is not None else None, out.data_ptr(), R, V, _ptr(scratch), 1 if any_greedy else 0,
          1 if any_filters else 0, _stream())
    return out


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, top_n: int):
    """log-softmax of the chosen token of each row and the row's ``top_n`` (<= 20) most probable tokens:
    (lp [R], top_ids [R, top_n] int32, top_lp [R, top_n]), descending, lowest index first among equals."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    _check(chosen, "chosen", (R,), torch.int32)
    lp = torch.empty((R,), dtype=torch.float32, device=logits.device)
    top_ids = torch.empty((R, top_n), dtype=torch.int32, device=logits.device)
    top_lp = torch.empty((R, top_n), dtype=torch.float32, device=logits.device)
    _call(load_module("sampling"), "ifx_logprobs", (P, P, I, I, I, P, P, P, P),
          logits.data_ptr(), chosen.data_ptr(), R, V, top_n, lp.data_ptr(), top_ids.data_ptr(), top_lp.data_ptr(), _stream())
    return lp, top_ids, top_lp


# ----------------------------------------------------------------------------------------
_SINKS: Dict[int, torch.Tensor] = {}


def stream_read(region: torch.Tensor, waves: int, streaming: bool) -> None:
    """Measurement only: ``waves`` single-wave workgroups read the whole of ``region`` (a multiple of 8 KB) once."""
    _check(region, "region")
    sink = _SINKS.get(region.device.index)
    if sink is None:
        sink = _SINKS[region.device.index] = torch.zeros(1, dtype=torch.float32, device=region.device)
    _call(load_module("ceilings"), "ifx_stream_read", (P, LL, I, I, P, P),
          region.data_ptr(), region.numel() * region.element_size(), waves, int(streaming), sink.data_ptr(), _stream())


def stream_copy(src: torch.Tensor, dst: torch.Tensor, waves: int, streaming: bool) -> None:
    """Measurement only: copies ``src`` to ``dst`` (same size, a multiple of 8 KB) with ``waves`` single-wave workgroups."""
    _check(src, "src")
    _check(dst, "dst")
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size():
        raise KernelError(f"stream_copy: {n} bytes into {dst.numel() * dst.element_size()}")
    _call(load_module("ceilings"), "ifx_stream_copy", (P, P, LL, I, I, P), src.data_ptr(), dst.data_ptr(), n, waves, int(streaming), _stream())
