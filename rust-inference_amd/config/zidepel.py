"""Configuration of the Zidepel decoder, from its config.json.

A Zidepel model is a list of layers, each with a mixer of its own kind and sizes (softmax attention with a
score cap and a query temperature, or gated linear attention) and an optional dense feed-forward; a stretch of
the layers may run several times in a row with the same weights; the residual may be kept in several streams.
config.json names the design in ``"architecture"`` and gives every size and constant:

    vocab, width, max_positions, norm: {eps}, streams (absent: one plain residual),
    loop: {start, stop, times} (absent: every layer once),
    layers: [{type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, softcap, q_temp: {coef, every}},
              mlp: {kind: "dense", ff} or null},
             {type: "gla", mixer: {heads, dim, vdim, tau}, mlp: ...}, ...]

The width of a gla mixer's two-step decay product is given by its tensors' shapes alone; a configuration that is
to be filled with random weights names it as ``rank`` in the mixer's sizes.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar, Optional

from ..errors import ConfigError, UnsupportedError
from .base import ModelConfig, f32, whole

MIXER_KINDS = ("attention", "gla")


def _section(raw, key: str, where: str) -> dict:
    v = raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: {key!r} must be an object, got {v!r}")
    return v


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int                          # size of a query or key head
    vdim: int                         # size of a value head
    scale: float                      # factor on q . k
    softcap: Optional[float]          # scores become softcap * tanh(score / softcap); None: no cap
    temper_coef: Optional[float]      # q *= 1 + coef * ln(floor((p + 1) / every) + 1); None: no temperature
    temper_every: int = 1

    @classmethod
    def read(cls, m: dict, where: str) -> "AttentionSizes":
        for key in ("heads", "kv_heads", "dim", "scale"):
            if key not in m:
                raise ConfigError(f"{where}: an attention mixer needs {key!r}")
        heads, kv = whole(m["heads"], where + ".heads", 1), whole(m["kv_heads"], where + ".kv_heads", 1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads not divisible by {kv} kv heads")
        dim = whole(m["dim"], where + ".dim", 1)
        cap = m.get("softcap")
        if cap is not None and not f32(cap, where + ".softcap") > 0.0:
            raise ConfigError(f"{where}: softcap {cap!r} must be positive")
        qt = m.get("q_temp")
        coef, every = None, 1
        if qt is not None:
            qt = _section(m, "q_temp", where)
            coef, every = f32(qt.get("coef"), where + ".q_temp.coef"), whole(qt.get("every"), where + ".q_temp.every", 1)
        return cls(heads, kv, dim, whole(m.get("vdim", dim), where + ".vdim", 1), f32(m["scale"], where + ".scale"),
                   None if cap is None else f32(cap, where + ".softcap"), coef, every)

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "softcap": self.softcap,
                "q_temp": None if self.temper_coef is None else {"coef": self.temper_coef, "every": self.temper_every}}


@dataclass(frozen=True)
class GlaSizes:
    heads: int
    dim: int                          # key channels of a head
    vdim: int                         # value channels of a head
    tau: float                        # decay = sigmoid(z)^(1 / tau)
    rank: Optional[int] = None        # width of the decay's two-step product; None: the checkpoint's tensors give it

    @classmethod
    def read(cls, m: dict, where: str) -> "GlaSizes":
        for key in ("heads", "dim", "tau"):
            if key not in m:
                raise ConfigError(f"{where}: a gla mixer needs {key!r}")
        dim = whole(m["dim"], where + ".dim", 1)
        tau = f32(m["tau"], where + ".tau")
        if not tau > 0.0:
            raise ConfigError(f"{where}: tau {tau} must be positive")
        rank = m.get("rank")
        return cls(whole(m["heads"], where + ".heads", 1), dim, whole(m.get("vdim", dim), where + ".vdim", 1), tau,
                   None if rank is None else whole(rank, where + ".rank", 1))

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class ZidepelLayer:
    type: str                                     # one of MIXER_KINDS
    mixer: object                                 # AttentionSizes or GlaSizes
    ff: Optional[int] = None                      # width of the dense feed-forward; None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class ZidepelConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: tuple = ()
    max_positions: int = 0
    norm_eps: float = 1e-5
    streams: Optional[int] = None                 # None: one plain residual; n: hyper-connections over n streams
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    ARCHITECTURE: ClassVar[str] = "Zidepel"
    MODEL_TYPE: ClassVar[str] = "zidepel"
    REQUIRED: ClassVar[tuple[str, ...]] = ("vocab", "width", "layers", "max_positions", "norm")

    @classmethod
    def from_dict(cls, raw: dict) -> "ZidepelConfig":
        cls.require(raw)
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config key 'layers' must be a list of at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXER_KINDS:
                kind = entry.get("type") if isinstance(entry, dict) else entry
                raise UnsupportedError(f"{where}: mixer type {kind!r} is not one of {', '.join(MIXER_KINDS)}")
            sizes = (AttentionSizes if entry["type"] == "attention" else GlaSizes).read(_section(entry, "mixer", where),
                                                                                       where + ".mixer")
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                mlp = _section(entry, "mlp", where)
                if mlp.get("kind") != "dense":
                    raise UnsupportedError(f"{where}: feed-forward kind {mlp.get('kind')!r} is not 'dense'")
                ff = whole(mlp.get("ff"), where + ".mlp.ff", 1)
            layers.append(ZidepelLayer(entry["type"], sizes, ff))
        loop = raw.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            loop = _section(raw, "loop", "config.json")
            start, stop = whole(loop.get("start"), "loop.start"), whole(loop.get("stop"), "loop.stop")
            times = whole(loop.get("times"), "loop.times", 1)
        streams = raw.get("streams")
        cfg = cls(vocab=whole(raw["vocab"], "vocab", 1), width=whole(raw["width"], "width", 1), layers=tuple(layers),
                  max_positions=whole(raw["max_positions"], "max_positions", 1),
                  norm_eps=f32(_section(raw, "norm", "config.json").get("eps"), "norm.eps"),
                  streams=None if streams is None else whole(streams, "streams", 1),
                  loop_start=start, loop_stop=stop, loop_times=times)
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
               "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.loop_times != 1 or self.loop_stop > self.loop_start:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return out
