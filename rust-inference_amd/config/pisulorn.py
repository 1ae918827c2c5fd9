"""Configuration of the Pisulorn decoder, from its config.json.

A Pisulorn model is a list of layers, each with a mixer of its own kind and sizes (softmax attention without
rotation, with a distance bias and an optional sliding window and query temperature; or the gated delta rule
with short convolutions) and an optional feed-forward (dense, or a mixture of experts); a stretch of the layers may
run several times in a row with the same weights; the residual may be kept in several streams; every sublayer's
output enters the residual times ``residual_mult``.  config.json names the design in ``"architecture"`` and gives
every size and constant:

    vocab, width, norm: {eps}, residual_mult (absent: 1), streams (absent: one plain residual),
    loop: {start, stop, times} (absent: every layer once),
    layers: [{type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, mask: {size}, q_temp: {coef, every}},
              mlp: {kind: "dense", ff} or {kind: "moe", expert: {ff, limit}, router: {experts, top}} or null},
             {type: "delta", mixer: {heads, kv_heads, dim, vdim, conv}, mlp: ...}, ...]

``max_positions`` is no key of the design (positions enter through distances alone); where it is given it is the
default length of a cache that is given none.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar, Optional

from ..errors import ConfigError, UnsupportedError
from .base import ModelConfig, f32, whole

MIXER_KINDS = ("attention", "delta")
DEFAULT_MAX_POSITIONS = 1 << 20


def _section(raw, key: str, where: str) -> dict:
    v = raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: {key!r} must be an object, got {v!r}")
    return v


def _heads(m: dict, where: str) -> tuple[int, int]:
    for key in ("heads", "dim"):
        if key not in m:
            raise ConfigError(f"{where}: a mixer needs {key!r}")
    heads = whole(m["heads"], where + ".heads", 1)
    kv = whole(m.get("kv_heads", heads), where + ".kv_heads", 1)
    if heads % kv:
        raise ConfigError(f"{where}: {heads} heads not divisible by {kv} kv heads")
    return heads, kv


@dataclass(frozen=True)
class BiasedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int                          # size of a query or key head
    vdim: int                         # size of a value head
    scale: float                      # factor on q . k
    window: Optional[int]             # a query sees itself and the window - 1 tokens before it; None: all
    temper_coef: Optional[float]      # q *= 1 + coef * ln(floor((p + 1) / every) + 1); None: no temperature
    temper_every: int = 1

    @classmethod
    def read(cls, m: dict, where: str) -> "BiasedAttentionSizes":
        heads, kv = _heads(m, where)
        if "scale" not in m:
            raise ConfigError(f"{where}: an attention mixer needs 'scale'")
        dim = whole(m["dim"], where + ".dim", 1)
        window = None
        if m.get("mask") is not None and _section(m, "mask", where).get("size") is not None:
            window = whole(m["mask"]["size"], where + ".mask.size", 1)
        coef, every = None, 1
        if m.get("q_temp") is not None:
            qt = _section(m, "q_temp", where)
            coef, every = f32(qt.get("coef"), where + ".q_temp.coef"), whole(qt.get("every"), where + ".q_temp.every", 1)
        return cls(heads, kv, dim, whole(m.get("vdim", dim), where + ".vdim", 1), f32(m["scale"], where + ".scale"),
                   window, coef, every)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.temper_coef is not None:
            out["q_temp"] = {"coef": self.temper_coef, "every": self.temper_every}
        return out


@dataclass(frozen=True)
class DeltaSizes:
    heads: int                        # value heads, each with a state of dim x vdim
    kv_heads: int                     # query/key heads, shared by heads / kv_heads value heads each
    dim: int
    vdim: int
    conv: int                         # taps of the short convolutions over q, k and v

    @classmethod
    def read(cls, m: dict, where: str) -> "DeltaSizes":
        heads, kv = _heads(m, where)
        if "conv" not in m:
            raise ConfigError(f"{where}: a delta mixer needs 'conv'")
        dim = whole(m["dim"], where + ".dim", 1)
        return cls(heads, kv, dim, whole(m.get("vdim", dim), where + ".vdim", 1), whole(m["conv"], where + ".conv", 1))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertsSizes:
    experts: int
    top: int
    ff: int                           # width of one expert
    limit: float                      # the experts' gate is capped at limit, their up branch clamped to +-limit

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top}}


def _read_mlp(entry: dict, where: str):
    if entry.get("mlp") is None:
        return None
    mlp = _section(entry, "mlp", where)
    kind = mlp.get("kind")
    if kind == "dense":
        return DenseSizes(whole(mlp.get("ff"), where + ".mlp.ff", 1))
    if kind == "moe":
        expert, router = _section(mlp, "expert", where + ".mlp"), _section(mlp, "router", where + ".mlp")
        experts = whole(router.get("experts"), where + ".mlp.router.experts", 1)
        top = whole(router.get("top"), where + ".mlp.router.top", 1)
        if top > experts:
            raise ConfigError(f"{where}.mlp: the {top} best of {experts} experts")
        limit = f32(expert.get("limit"), where + ".mlp.expert.limit")
        if not limit > 0.0:
            raise ConfigError(f"{where}.mlp.expert.limit {limit} must be positive")
        return ExpertsSizes(experts, top, whole(expert.get("ff"), where + ".mlp.expert.ff", 1), limit)
    raise UnsupportedError(f"{where}: feed-forward kind {kind!r} is neither 'dense' nor 'moe'")


@dataclass(frozen=True)
class PisulornLayer:
    type: str                                     # one of MIXER_KINDS
    mixer: object                                 # BiasedAttentionSizes or DeltaSizes
    mlp: object = None                            # DenseSizes, ExpertsSizes or None: the layer has no feed-forward

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class PisulornConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: tuple = ()
    norm_eps: float = 1e-5
    residual_mult: float = 1.0                    # every sublayer's output enters the residual times this
    streams: Optional[int] = None                 # None: one plain residual; n: hyper-connections over n streams
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    max_positions: int = DEFAULT_MAX_POSITIONS

    ARCHITECTURE: ClassVar[str] = "Pisulorn"
    MODEL_TYPE: ClassVar[str] = "pisulorn"
    REQUIRED: ClassVar[tuple[str, ...]] = ("vocab", "width", "layers", "norm")

    @classmethod
    def from_dict(cls, raw: dict) -> "PisulornConfig":
        cls.require(raw)
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config key 'layers' must be a list of at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXER_KINDS:
                kind = entry.get("type") if isinstance(entry, dict) else entry
                raise UnsupportedError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_KINDS)}")
            sizes = (BiasedAttentionSizes if entry["type"] == "attention" else DeltaSizes).read(
                _section(entry, "mixer", where), where + ".mixer")
            layers.append(PisulornLayer(entry["type"], sizes, _read_mlp(entry, where)))
        start = stop = 0
        times = 1
        if raw.get("loop") is not None:
            loop = _section(raw, "loop", "config.json")
            start, stop = whole(loop.get("start"), "loop.start"), whole(loop.get("stop"), "loop.stop")
            times = whole(loop.get("times", 1), "loop.times", 1)
        streams = raw.get("streams")
        cfg = cls(vocab=whole(raw["vocab"], "vocab", 1), width=whole(raw["width"], "width", 1), layers=tuple(layers),
                  norm_eps=f32(_section(raw, "norm", "config.json").get("eps"), "norm.eps"),
                  residual_mult=f32(raw.get("residual_mult", 1.0), "residual_mult"),
                  streams=None if streams is None else whole(streams, "streams", 1),
                  loop_start=start, loop_stop=stop, loop_times=times,
                  max_positions=whole(raw.get("max_positions", DEFAULT_MAX_POSITIONS), "max_positions", 1))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"norm.eps {self.norm_eps} must not be negative")
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers):
            raise ConfigError(f"loop {self.loop_start}..{self.loop_stop} does not lie inside the {len(self.layers)} layers")

    def order(self) -> list[int]:
        """The layers in the order they run: the looped stretch ``times`` times in a row, then the rest."""
        n, a, b = len(self.layers), self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))

    def to_dict(self) -> dict:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.loop_times != 1 or self.loop_stop > self.loop_start:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out
