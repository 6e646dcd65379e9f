"""Configuration of the Tabatar decoder, from its config.json.

The file is nested: the model's own sizes and constants at the top (``vocab``, ``width``, ``norm.eps``,
``embedding.scale``, ``streams``, ``logit_scale``, ``logit_softcap``, ``loop``) and a list ``layers`` whose entries each
give the layer's ``type`` (its mixer: "attention" or "gla"), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``, or null for a layer without one).  Layers need not be alike: the plan is built layer by layer.

    attention   heads, kv_heads (absent: heads), dim (query/key size per head), vdim (value size per head; absent: dim),
                scale (the factor on the scores), rot.base / rot.dims (the rotation's base and how many of a head's
                dimensions turn; absent: all), rot.scaling {factor, low, high, original} (frequencies scaled in bands of
                wavelength; absent: none), mask.size (how many positions, its own included, a query sees; absent or
                null: all before it)
    gla         heads, dim (key/query channels per head), vdim (values per head), tau (the decay's root), rank (the
                width of the decay's low-rank projection; a file that leaves it out leaves it to the tensor's shape)
    mlp         kind "dense": ff (inner size of a feed-forward without a gate)
                kind "moe": expert.ff, router.experts / top, shared.ff (a further expert every token takes; absent: none)
    loop        start, stop, times: layers start .. stop - 1 run ``times`` times in a row with the same weights (each pass
                with a cache or state of its own); absent: every layer runs once
    streams     the number of residual streams with learned connections between them; absent: one plain residual stream

A missing or mistyped key is an error that names it by its path.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, Mapping, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, read_key
from .mumusun import _read, _section

MIXER_TYPES = ("attention", "gla")
MLP_KINDS = ("dense", "moe")
MAX_STREAMS = 8


@dataclasses.dataclass(frozen=True)
class BandScaling:
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self) -> Dict[str, Any]:
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclasses.dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[BandScaling]
    window: Optional[int]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "AttentionConfig":
        rot = _section(d, "rot", where)
        mask = _section(d, "mask", where, optional=True) or {}
        sc = _section(rot, "scaling", where + "rot.", optional=True)
        scaling = None
        if sc is not None:
            w = where + "rot.scaling."
            scaling = BandScaling(_read(sc, "factor", float, w), _read(sc, "low", float, w), _read(sc, "high", float, w),
                                  _read(sc, "original", float, w))
        dim, heads = _read(d, "dim", int, where), _read(d, "heads", int, where)
        return cls(heads=heads, kv_heads=_read(d, "kv_heads", int, where, heads), dim=dim, vdim=_read(d, "vdim", int, where, dim),
                   scale=_read(d, "scale", float, where), rot_base=_read(rot, "base", float, where + "rot."),
                   rot_dims=_read(rot, "dims", int, where + "rot.", dim), rot_scaling=scaling,
                   window=_read(mask, "size", int, where + "mask.", None))

    def to_dict(self) -> Dict[str, Any]:
        rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale, "rot": rot}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out

    def validate(self, where: str) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.heads % self.kv_heads:
            raise ConfigError(f"config.json: '{where}heads' = {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if self.dim % 2:
            raise ConfigError(f"config.json: '{where}dim' = {self.dim} must be even")
        if self.rot_dims <= 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"config.json: '{where}rot.dims' = {self.rot_dims} must be even and within dim {self.dim}")
        if not self.rot_base > 1:
            raise ConfigError(f"config.json: '{where}rot.base' must be above 1, got {self.rot_base}")
        s = self.rot_scaling
        if s is not None and (min(s.factor, s.original, s.low) <= 0 or not s.low < s.high):
            raise ConfigError(f"config.json: '{where}rot.scaling' needs positive factor and original and 0 < low < high")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"config.json: '{where}mask.size' must be positive, got {self.window}")


@dataclasses.dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int]        # None: the model file's tensors say (``with_tensor_shapes``)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "GlaConfig":
        dim = _read(d, "dim", int, where)
        return cls(heads=_read(d, "heads", int, where), dim=dim, vdim=_read(d, "vdim", int, where, dim),
                   tau=_read(d, "tau", float, where), rank=_read(d, "rank", int, where, None))

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.rank is not None:
            out["rank"] = self.rank
        return out

    def validate(self, where: str) -> None:
        for name in ("heads", "dim", "vdim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if not self.tau > 0:
            raise ConfigError(f"config.json: '{where}tau' must be positive, got {self.tau}")
        if self.rank is not None and self.rank <= 0:
            raise ConfigError(f"config.json: '{where}rank' must be positive, got {self.rank}")


@dataclasses.dataclass(frozen=True)
class DenseMlpConfig:
    ff: int
    kind: ClassVar[str] = "dense"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DenseMlpConfig":
        return cls(ff=_read(d, "ff", int, where))

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}

    def validate(self, where: str) -> None:
        if self.ff <= 0:
            raise ConfigError(f"config.json: '{where}ff' must be positive, got {self.ff}")


@dataclasses.dataclass(frozen=True)
class MoeMlpConfig:
    ff: int
    experts: int
    top: int
    shared_ff: int             # 0: no shared expert
    kind: ClassVar[str] = "moe"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "MoeMlpConfig":
        expert, router = _section(d, "expert", where), _section(d, "router", where)
        shared = _section(d, "shared", where, optional=True)
        return cls(ff=_read(expert, "ff", int, where + "expert."), experts=_read(router, "experts", int, where + "router."),
                   top=_read(router, "top", int, where + "router."),
                   shared_ff=_read(shared, "ff", int, where + "shared.") if shared is not None else 0)

    def to_dict(self) -> Dict[str, Any]:
        out = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out

    def validate(self, where: str) -> None:
        for name in ("ff", "experts", "top"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{where}{name}' must be positive, got {getattr(self, name)}")
        if self.top > self.experts:
            raise ConfigError(f"config.json: '{where}router.top' = {self.top} exceeds the {self.experts} experts")
        if self.shared_ff < 0:
            raise ConfigError(f"config.json: '{where}shared.ff' must be positive, got {self.shared_ff}")


def _mlp_from_dict(d: Mapping[str, Any], where: str):
    kind = _read(d, "kind", str, where, "dense")
    if kind not in MLP_KINDS:
        raise ConfigError(f"config.json: '{where}kind' = '{kind}' is not supported (one of {MLP_KINDS})")
    return (DenseMlpConfig if kind == "dense" else MoeMlpConfig).from_dict(d, where)


@dataclasses.dataclass(frozen=True)
class TabatarLayer:
    type: str
    mixer: Union[AttentionConfig, GlaConfig]
    mlp: Union[None, DenseMlpConfig, MoeMlpConfig]

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None}


@dataclasses.dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int

    def to_dict(self) -> Dict[str, Any]:
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclasses.dataclass(frozen=True)
class TabatarConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    streams: Optional[int]              # None: one plain residual stream
    logit_scale: float
    logit_softcap: Optional[float]
    loop: Optional[LoopConfig]
    layers: Tuple[TabatarLayer, ...]
    # The file names no longest sequence: positions are formed in 32-bit floats like every other angle of the
    # engine, which counts integers exactly up to 2^24.
    max_positions: int = 1 << 24

    model_type: ClassVar[str] = "tabatar"
    architectures: ClassVar[Tuple[str, ...]] = ("Tabatar",)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TabatarConfig":
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
            mixer_cls = AttentionConfig if kind == "attention" else GlaConfig
            mixer = mixer_cls.from_dict(_section(L, "mixer", where), where + "mixer.")
            mlp = _section(L, "mlp", where, optional=True)
            layers.append(TabatarLayer(kind, mixer, _mlp_from_dict(mlp, where + "mlp.") if mlp is not None else None))
        norm = _section(d, "norm", "")
        emb = _section(d, "embedding", "", optional=True) or {}
        lp = _section(d, "loop", "", optional=True)
        loop = None
        if lp is not None:
            loop = LoopConfig(_read(lp, "start", int, "loop."), _read(lp, "stop", int, "loop."), _read(lp, "times", int, "loop.", 1))
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int), norm_eps=_read(norm, "eps", float, "norm."),
                  embedding_scale=_read(emb, "scale", float, "embedding.", 1.0), streams=read_key(d, "streams", int, None),
                  logit_scale=read_key(d, "logit_scale", float, 1.0), logit_softcap=read_key(d, "logit_softcap", float, None),
                  loop=loop, layers=tuple(layers), max_positions=read_key(d, "max_positions", int, 1 << 24))
        cfg.validate()
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architectures[0], "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
               "layers": [L.to_dict() for L in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.loop is not None:
            out["loop"] = self.loop.to_dict()
        if self.max_positions != 1 << 24:
            out["max_positions"] = self.max_positions
        return out

    def validate(self) -> None:
        for name in ("vocab", "width", "max_positions"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: '{name}' must be positive, got {getattr(self, name)}")
        if not self.norm_eps >= 0:
            raise ConfigError(f"config.json: 'norm.eps' must be >= 0, got {self.norm_eps}")
        if self.streams is not None and not 0 < self.streams <= MAX_STREAMS:
            raise ConfigError(f"config.json: 'streams' = {self.streams} (1 to {MAX_STREAMS})")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"config.json: 'logit_softcap' must be positive, got {self.logit_softcap}")
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

    def run_order(self) -> Tuple[int, ...]:
        """The layers in the order they run: the looped span ``times`` times in a row, the others once."""
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        lp = self.loop
        return tuple(range(lp.start)) + tuple(range(lp.start, lp.stop)) * lp.times + tuple(range(lp.stop, n))

    def open_sizes(self) -> Tuple[str, ...]:
        return tuple(f"layers[{i}].mixer.rank" for i, L in enumerate(self.layers) if L.type == "gla" and L.mixer.rank is None)

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "TabatarConfig":
        """The config with the sizes it leaves open taken from the model file: a gla layer's decay rank is the number of
        rows of its ``l<i>.mix.a1``."""
        layers = []
        for i, L in enumerate(self.layers):
            if L.type == "gla" and L.mixer.rank is None:
                shape = shapes.get(f"l{i}.mix.a1")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"config.json: 'layers[{i}].mixer' names no rank and the model file has no matrix 'l{i}.mix.a1' to take it from")
                L = dataclasses.replace(L, mixer=dataclasses.replace(L.mixer, rank=int(shape[0])))
            layers.append(L)
        out = dataclasses.replace(self, layers=tuple(layers))
        out.validate()
        return out
