"""A residual kept in several streams (hyper-connections), and the coefficients that connect a sublayer to them.

Instead of one ``x`` a model keeps ``x_1 .. x_S``, all equal to the embedding's output at the start.  A
sublayer with coefficients ``in [S]``, ``mix [S, S]`` (indexed ``[from, to]``) and ``out [S]`` reads
``u = sum_s in[s] x_s``, computes ``y = sublayer(norm(u))`` and writes every stream at once from the old ones,
``x_t <- sum_s mix[s, t] x_s + out[t] y``.  What leaves the model is the sum of the streams.

As with the plain ``ResidualStream`` the write waits for the next read and is done by it: one kernel
(``ops.streams_read_norm``) applies the waiting write, stores the new streams, forms ``u`` with the reading
sublayer's coefficients and norms it.  Streams and all their sums are float32 in both compute dtypes.
"""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import GAIN, MIXING, TensorSpec
from .base import Part
from .block import ResidualStream
from .registry import register_part

register_part("stream", "residual", ResidualStream)


@register_part("connection", "hyper")
class HyperConnection(Part):
    """The coefficients of one sublayer: tensors ``<prefix>in``, ``<prefix>mix`` and ``<prefix>out``.
    ``out_scale``: a constant of the model on every sublayer's output, ``x_t <- sum_s mix[s, t] x_s + out_scale *
    out[t] * y``; it is multiplied into ``out`` (in float32) when the weights are bound."""

    def __init__(self, streams: int, prefix: str, out_scale: float = 1.0):
        if not 1 <= streams <= ops.MAX_STREAMS:
            raise ConfigError(f"{streams} residual streams: the kernel takes 1 to {ops.MAX_STREAMS}")
        self.streams, self.prefix, self.out_scale = streams, prefix, float(out_scale)

    def tensors(self):
        n, p = self.streams, self.prefix
        return {p + "in": TensorSpec((n,), GAIN), p + "out": TensorSpec((n,), GAIN), p + "mix": TensorSpec((n, n), MIXING)}

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        self.read, self.write, self.mix = (rt.place_gain(weights[p + k]) for k in ("in", "out", "mix"))
        if self.out_scale != 1.0:
            self.write = (self.write * torch.tensor(self.out_scale, dtype=torch.float32, device=self.write.device)).contiguous()


@register_part("connection", "scaled_add")
class ScaledAdd(Part):
    """The connection of a sublayer to one plain residual, ``x <- x + scale * y``, in the terms of the streams'
    kernel: one stream that is read and kept as it is.  It has no tensors."""

    def __init__(self, scale: float = 1.0):
        self.streams, self.scale = 1, float(scale)

    def bind(self, weights, rt):
        self.rt = rt
        self.read = self.mix = None                                   # taken as 1 by the kernel
        self.write = torch.tensor([self.scale], dtype=torch.float32, device=rt.device)


@register_part("stream", "hyper")
class HyperStream:
    """``streams`` copies of the residual, ``[T, streams, hidden]`` float32, with at most one write waiting."""

    def __init__(self, hidden: torch.Tensor, streams: int):
        self.fresh = hidden                  # [T, hidden]: what every stream starts from, until the first read spreads it
        self.n = streams
        self.x = torch.empty((hidden.shape[0], streams, hidden.shape[1]), dtype=torch.float32, device=hidden.device)
        self.waiting = None                  # (y, HyperConnection) of the sublayer that ran last
        self.next_entry_norm = None          # (set by the model for streams that leave norms to products; unused here)
        self.next_entry_tiled = False
        self.links_ok = False

    @property
    def rows(self) -> int:
        return self.x.shape[0]

    def _go(self, reader, norm, out_dtype, rows):
        y, conn = self.waiting if self.waiting is not None else (None, None)
        with profiler.section(profiler.NORM):
            out = ops.streams_read_norm(
                self.x, y, conn.mix if conn else None, conn.write if conn else None, reader,
                getattr(norm, "gain", None), getattr(norm, "bias", None), getattr(norm, "eps", 0.0),
                norm.kind if norm is not None else ops.NORM_NONE, out_dtype, rows, fresh=self.fresh)
        if rows is None:
            self.waiting, self.fresh = None, None
        return out

    def read(self, connection: HyperConnection, norm, out_dtype):
        """``norm(sum_s in[s] x_s)`` for the sublayer with these coefficients, after the write that waits."""
        return self._go(connection.read, norm, out_dtype, None)

    def write(self, y, connection: HyperConnection) -> None:
        """``y`` is the sublayer's output ``[T, hidden]`` (or ``[parts, T, hidden]`` float32, added in order)."""
        if self.waiting is not None:
            self._go(None, None, torch.float32, None)        # two writes in a row: the first is applied by itself
        self.waiting = (y, connection)

    def normed(self, norm, out_dtype, rows=None, **_):
        """What leaves the model: the norm of the sum of the streams (of the given rows only)."""
        return self._go(None, norm, out_dtype, rows)

    def link(self, *_, **__):
        return None

    def push(self, branch) -> None:
        raise ConfigError("a residual in several streams is written through a layer's connections, not by a plain add")

    def flush(self) -> None:
        if self.waiting is not None:
            self._go(None, None, torch.float32, None)
