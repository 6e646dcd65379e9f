"""Configuration of the Vavadra decoder, from its config.json.

The file is nested: the model's own sizes and constants at the top (``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``logit_scale``, ``loop``) and a list ``layers`` whose entries each give the layer's ``type`` (its
mixer), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null for a layer without one).
Layers need not be alike: the plan is built layer by layer.

    attention          differential attention: heads, kv_heads (absent: heads), dim (query/key size of one map of a head),
                       vdim (absent: dim), scale, diff (the constant of lambda), mask.size (positions are seen within blocks
                       of this many, counted from the sequence's start; absent: everything before)
    delta              the gated delta rule: heads (value heads), kv_heads (query/key heads; absent: heads), dim, vdim
                       (absent: dim), conv (taps of the short convolution; a file that leaves it out leaves it to the
                       tensor's shape)
    latent_attention   heads, dim (unrotated), rot_dim (rotated), vdim (absent: dim), kv_rank, scale, rot.base, rot.dims
                       (absent: rot_dim), mask.size (a sliding window; absent: everything before)
    mlp                kind "moe": expert.ff / limit, router.experts / identity (absent: 0) / top / scale (absent: 1),
                       shared.ff / limit (absent: no shared expert)
    loop               start, stop, times: layers start .. stop - 1 run ``times`` times in a row with the same weights

A missing or mistyped key is an error that names it by its path.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, Mapping, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, read_key
from .mumusun import _read, _section
from .tabatar import LoopConfig

MIXER_TYPES = ("attention", "delta", "latent_attention")
MLP_KINDS = ("moe",)


def _positive(obj, names, where):
    for name in names:
        if getattr(obj, name) <= 0:
            raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(obj, name)}")


@dataclasses.dataclass(frozen=True)
class DifferentialAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    chunk: Optional[int]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DifferentialAttentionConfig":
        mask = _section(d, "mask", where, optional=True) or {}
        dim, heads = _read(d, "dim", int, where), _read(d, "heads", int, where)
        return cls(heads=heads, kv_heads=_read(d, "kv_heads", int, where, heads), dim=dim, vdim=_read(d, "vdim", int, where, dim),
                   scale=_read(d, "scale", float, where), diff=_read(d, "diff", float, where),
                   chunk=_read(mask, "size", int, where + "mask.", None))

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
               "diff": self.diff}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        return out

    def validate(self, where: str) -> None:
        _positive(self, ("heads", "kv_heads", "dim", "vdim"), where)
        if self.heads % self.kv_heads:
            raise ConfigError(f"config.json: '{where}heads' = {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.chunk is not None and self.chunk <= 0:
            raise ConfigError(f"config.json: '{where}mask.size' must be positive, got {self.chunk}")


@dataclasses.dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: Optional[int]        # None: the model file's tensors say (``with_tensor_shapes``)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DeltaConfig":
        dim, heads = _read(d, "dim", int, where), _read(d, "heads", int, where)
        return cls(heads=heads, kv_heads=_read(d, "kv_heads", int, where, heads), dim=dim, vdim=_read(d, "vdim", int, where, dim),
                   conv=_read(d, "conv", int, where, None))

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim}
        if self.conv is not None:
            out["conv"] = self.conv
        return out

    def validate(self, where: str) -> None:
        _positive(self, ("heads", "kv_heads", "dim", "vdim"), where)
        if self.heads % self.kv_heads:
            raise ConfigError(f"config.json: '{where}heads' = {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.conv is not None and self.conv <= 0:
            raise ConfigError(f"config.json: '{where}conv' must be positive, got {self.conv}")


@dataclasses.dataclass(frozen=True)
class SinkLatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "SinkLatentAttentionConfig":
        rot = _section(d, "rot", where)
        mask = _section(d, "mask", where, optional=True) or {}
        dim, rot_dim = _read(d, "dim", int, where), _read(d, "rot_dim", int, where)
        return cls(heads=_read(d, "heads", int, where), dim=dim, rot_dim=rot_dim, vdim=_read(d, "vdim", int, where, dim),
                   kv_rank=_read(d, "kv_rank", int, where), scale=_read(d, "scale", float, where),
                   rot_base=_read(rot, "base", float, where + "rot."), rot_dims=_read(rot, "dims", int, where + "rot.", rot_dim),
                   window=_read(mask, "size", int, where + "mask.", None))

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
               "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out

    def validate(self, where: str) -> None:
        _positive(self, ("heads", "dim", "rot_dim", "vdim", "kv_rank"), where)
        if self.rot_dims <= 0 or self.rot_dims % 2 or self.rot_dims > self.rot_dim:
            raise ConfigError(f"config.json: '{where}rot.dims' = {self.rot_dims} must be even and within rot_dim {self.rot_dim}")
        if not self.rot_base > 1:
            raise ConfigError(f"config.json: '{where}rot.base' must be above 1, got {self.rot_base}")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"config.json: '{where}mask.size' must be positive, got {self.window}")


@dataclasses.dataclass(frozen=True)
class ClampedMoeConfig:
    ff: int
    limit: float
    experts: int
    identity: int
    top: int
    route_scale: float
    shared_ff: int             # 0: no shared expert
    shared_limit: float
    kind: ClassVar[str] = "moe"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "ClampedMoeConfig":
        expert, router = _section(d, "expert", where), _section(d, "router", where)
        shared = _section(d, "shared", where, optional=True)
        limit = _read(expert, "limit", float, where + "expert.")
        return cls(ff=_read(expert, "ff", int, where + "expert."), limit=limit,
                   experts=_read(router, "experts", int, where + "router."), identity=_read(router, "identity", int, where + "router.", 0),
                   top=_read(router, "top", int, where + "router."), route_scale=_read(router, "scale", float, where + "router.", 1.0),
                   shared_ff=_read(shared, "ff", int, where + "shared.") if shared is not None else 0,
                   shared_limit=_read(shared, "limit", float, where + "shared.", limit) if shared is not None else limit)

    def to_dict(self) -> Dict[str, Any]:
        out = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
               "router": {"experts": self.experts, "identity": self.identity, "top": self.top, "scale": self.route_scale}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out

    def validate(self, where: str) -> None:
        _positive(self, ("ff", "experts", "top"), where)
        if self.identity < 0:
            raise ConfigError(f"config.json: '{where}router.identity' must not be negative, got {self.identity}")
        if self.top > self.experts + self.identity:
            raise ConfigError(f"config.json: '{where}router.top' = {self.top} exceeds the {self.experts} + {self.identity} experts")
        if self.shared_ff < 0:
            raise ConfigError(f"config.json: '{where}shared.ff' must be positive, got {self.shared_ff}")
        if not (self.limit > 0 and self.shared_limit > 0):
            raise ConfigError(f"config.json: '{where}expert.limit' and 'shared.limit' must be positive")


_MIXERS = {"attention": DifferentialAttentionConfig, "delta": DeltaConfig, "latent_attention": SinkLatentAttentionConfig}


@dataclasses.dataclass(frozen=True)
class VavadraLayer:
    type: str
    mixer: Union[DifferentialAttentionConfig, DeltaConfig, SinkLatentAttentionConfig]
    mlp: Optional[ClampedMoeConfig]

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None}


@dataclasses.dataclass(frozen=True)
class VavadraConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    loop: Optional[LoopConfig]
    layers: Tuple[VavadraLayer, ...]
    # The file names no longest sequence: positions are formed in 32-bit floats like every other angle of the
    # engine, which counts integers exactly up to 2^24.
    max_positions: int = 1 << 24

    model_type: ClassVar[str] = "vavadra"
    architectures: ClassVar[Tuple[str, ...]] = ("Vavadra",)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "VavadraConfig":
        layers_in = d.get("layers")
        if not isinstance(layers_in, list) or not layers_in:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, L in enumerate(layers_in):
            where = f"layers[{i}]."
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: 'layers[{i}]' must be an object")
            kind = _read(L, "type", str, where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: '{where}type' = '{kind}' is not a known mixer (one of {MIXER_TYPES})")
            mixer = _MIXERS[kind].from_dict(_section(L, "mixer", where), where + "mixer.")
            mlp_in = _section(L, "mlp", where, optional=True)
            mlp = None
            if mlp_in is not None:
                mlp_kind = _read(mlp_in, "kind", str, where + "mlp.", "moe")
                if mlp_kind not in MLP_KINDS:
                    raise ConfigError(f"config.json: '{where}mlp.kind' = '{mlp_kind}' is not supported (one of {MLP_KINDS})")
                mlp = ClampedMoeConfig.from_dict(mlp_in, where + "mlp.")
            layers.append(VavadraLayer(kind, mixer, mlp))
        norm = _section(d, "norm", "")
        emb = _section(d, "embedding", "", optional=True) or {}
        lp = _section(d, "loop", "", optional=True)
        loop = None
        if lp is not None:
            loop = LoopConfig(_read(lp, "start", int, "loop."), _read(lp, "stop", int, "loop."), _read(lp, "times", int, "loop.", 1))
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int), norm_eps=_read(norm, "eps", float, "norm."),
                  embedding_scale=_read(emb, "scale", float, "embedding.", 1.0), logit_scale=read_key(d, "logit_scale", float, 1.0),
                  loop=loop, layers=tuple(layers), max_positions=read_key(d, "max_positions", int, 1 << 24))
        cfg.validate()
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architectures[0], "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
               "layers": [L.to_dict() for L in self.layers]}
        if self.loop is not None:
            out["loop"] = self.loop.to_dict()
        if self.max_positions != 1 << 24:
            out["max_positions"] = self.max_positions
        return out

    def validate(self) -> None:
        _positive(self, ("vocab", "width", "max_positions"), "")
        if not self.norm_eps >= 0:
            raise ConfigError(f"config.json: 'norm.eps' must be >= 0, got {self.norm_eps}")
        if self.loop is not None:
            lp = self.loop
            if not 0 <= lp.start < lp.stop <= len(self.layers):
                raise ConfigError(f"config.json: 'loop' = layers {lp.start} .. {lp.stop} - 1 does not lie within the {len(self.layers)} layers")
            if lp.times <= 0:
                raise ConfigError(f"config.json: 'loop.times' must be positive, got {lp.times}")
        for i, L in enumerate(self.layers):
            L.mixer.validate(f"layers[{i}].mixer.")
            if L.mlp is not None:
                L.mlp.validate(f"layers[{i}].mlp.")

    def run_order(self) -> Tuple[Tuple[int, Optional[int]], ...]:
        """(layer, pass) in the order the layers run: the looped span ``times`` times in a row, the others once.  ``pass`` is
        the number of the pass on the first layer of every pass of the loop and None everywhere else."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, None) for i in range(n))
        lp = self.loop
        out = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            out += [(i, t if i == lp.start else None) for i in range(lp.start, lp.stop)]
        return tuple(out + [(i, None) for i in range(lp.stop, n)])

    def open_sizes(self) -> Tuple[str, ...]:
        return tuple(f"layers[{i}].mixer.conv" for i, L in enumerate(self.layers) if L.type == "delta" and L.mixer.conv is None)

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "VavadraConfig":
        """The config with the sizes it leaves open taken from the model file: a delta layer's taps are the columns of its
        ``l<i>.mix.q.conv``."""
        layers = []
        for i, L in enumerate(self.layers):
            if L.type == "delta" and L.mixer.conv is None:
                shape = shapes.get(f"l{i}.mix.q.conv")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"config.json: 'layers[{i}].mixer' names no conv and the model file has no matrix 'l{i}.mix.q.conv' to take it from")
                L = dataclasses.replace(L, mixer=dataclasses.replace(L.mixer, conv=int(shape[1])))
            layers.append(L)
        out = dataclasses.replace(self, layers=tuple(layers))
        out.validate()
        return out
