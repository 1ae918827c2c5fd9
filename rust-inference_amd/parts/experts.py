"""A mixture of experts as a feed-forward part."""
from __future__ import annotations

import torch

from .. import profiler
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, MATRIX, TensorSpec
from .base import FeedForward
from .registry import register_part


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """``experts`` small feed-forward layers of which every token uses ``top``.

    Router: logits ``z = W_router h`` in float32, scores ``s = sigmoid(z)``; the ``top`` experts with the largest
    ``s + correction`` are chosen, and their weights are their scores ``s`` (without the correction) divided by the
    sum of the chosen scores (+ 1e-20).  Expert: ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, -limit, limit)``,
    output ``W_down (g sigmoid(1.702 g) (u + 1))``; no biases.  The part's output is the weighted sum of the chosen
    experts' outputs.

    The experts are two products: every expert's gate and up rows side by side (``[experts, 2, ff]`` rows), and every
    expert's down matrix side by side along K; between them the activation kernel writes zeros for the experts a
    token did not choose and the router's weight times the activation for those it did, so that the second product's
    sum over K is the weighted sum.

    Tensors: ``<prefix>router [experts, hidden]``, ``<prefix>correction [experts]``, ``<prefix>e<i>.gate`` / ``.up``
    ``[ff, hidden]``, ``<prefix>e<i>.down [hidden, ff]``.
    """

    def __init__(self, hidden: int, inter: int, experts: int, top: int, limit: float, prefix: str):
        if not 1 <= top <= experts <= ops.EXPERTS_MAX:
            raise ConfigError(f"the {top} best of {experts} experts: the router takes up to {ops.EXPERTS_MAX} experts")
        if not limit > 0:
            raise ConfigError(f"the experts' limit {limit} must be positive")
        self.hidden, self.inter, self.experts, self.top, self.limit, self.prefix = hidden, inter, experts, top, float(limit), prefix

    def tensors(self):
        p, t = self.prefix, {}
        t[p + "router"] = TensorSpec((self.experts, self.hidden), MATRIX)
        t[p + "correction"] = TensorSpec((self.experts,), BIAS)
        for e in range(self.experts):
            t[f"{p}e{e}.gate"] = TensorSpec((self.inter, self.hidden), MATRIX)
            t[f"{p}e{e}.up"] = TensorSpec((self.inter, self.hidden), MATRIX)
            t[f"{p}e{e}.down"] = TensorSpec((self.hidden, self.inter), MATRIX)
        return t

    def bind(self, weights, rt):
        self.rt = rt
        p = self.prefix
        self.w_router = rt.pack(rt.place_matrix(weights[p + "router"]))
        self.correction = rt.place_gain(weights[p + "correction"])
        rows = []
        for e in range(self.experts):
            rows += [weights[f"{p}e{e}.gate"], weights[f"{p}e{e}.up"]]
        self.w_gate_up = rt.pack(rt.place_matrix(torch.cat(rows, 0)), always=True)
        down = torch.cat([weights[f"{p}e{e}.down"] for e in range(self.experts)], 1)
        self.w_down = rt.pack(rt.place_matrix(down), parts_ok=True)

    def forward(self, x, ctx):
        rt = self.rt
        with profiler.section(profiler.MLP):
            z = rt.linear_packed(x, self.w_router, out_dtype=torch.float32)
            _, _, dense = ops.experts_route(z, self.correction, self.top)
            gu = ops.as_rows(rt.linear_packed(x, self.w_gate_up))
            a = ops.experts_activate(gu, dense, self.inter, self.limit)
            # float32 into the residual (or in parts that the stream's next read adds)
            return rt.linear_packed(a, self.w_down, out_dtype=torch.float32, parts_ok=True)
