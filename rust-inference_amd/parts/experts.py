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

    The experts' matrices lie as two: every expert's gate and up rows side by side (``[experts, 2, ff]`` rows), and
    every expert's down matrix side by side along K.  A step of a few tokens reads only the rows of the experts
    chosen; a prompt sorts its tokens by expert and runs two products an expert; in between (and in float32) the two
    matrices are two products over all tokens, between which the activation kernel writes zeros for the experts a
    token did not choose and the router's weight times the activation for those it did, so that the second product's
    sum over K is the weighted sum.  The three differ by rounding alone.

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

    # A step with fewer assignments (tokens x top) than experts reads only the rows of the experts its tokens chose
    # (one wavefront an output row: every assignment streams its expert's matrices once, so with as many assignments
    # as experts it would read what all experts hold); from SORTED_MIN_TOKENS tokens on a prompt's assignments are
    # sorted by expert and every expert is two library products over its own rows; between them, and in float32, all
    # experts are computed for all tokens as two products, with zeros where a token did not choose.
    SORTED_MIN_TOKENS = 256

    def forward(self, x, ctx):
        rt = self.rt
        with profiler.section(profiler.MLP):
            z = rt.linear_packed(x, self.w_router, out_dtype=torch.float32)
            ids, weights, dense = ops.experts_route(z, self.correction, self.top)
            tokens = z.shape[0]
            routed = (rt.dtype == torch.bfloat16 and not rt.invariant and self.top < self.experts
                      and self.hidden % 8 == 0 and self.inter % 8 == 0)
            if routed and tokens * self.top < self.experts:
                return ops.experts_few_tokens(rt.normed_now(x), self.w_gate_up.w, self.w_down.w, ids, weights, self.inter,
                                              self.limit)
            if (routed and tokens >= self.SORTED_MIN_TOKENS and not ctx.is_decode
                    and not torch.cuda.is_current_stream_capturing()):
                return self.forward_sorted(rt.normed_now(x), ids, weights)
            gu = ops.as_rows(rt.linear_packed(x, self.w_gate_up))
            a = ops.experts_activate(gu, dense, self.inter, self.limit)
            # float32 into the residual (or in parts that the stream's next read adds)
            return rt.linear_packed(a, self.w_down, out_dtype=torch.float32, parts_ok=True)

    def forward_sorted(self, x, ids, weights):
        """A prompt: every expert's tokens as rows side by side, two library products an expert, the weighted sum in
        float32.  The host reads how many rows every expert has (one wait a layer), which a captured step could not."""
        ff = self.inter
        dest, offsets = ops.experts_sort(ids, self.experts)
        rows = ops.experts_gather(x, dest, self.top)
        y = torch.empty_like(rows)
        starts = offsets.tolist()
        for e in range(self.experts):
            a, b = starts[e], starts[e + 1]
            if b > a:
                gu = torch.mm(rows[a:b], self.w_gate_up.w[e * 2 * ff:(e + 1) * 2 * ff].t())
                act = ops.experts_activate(gu, None, ff, self.limit)
                torch.mm(act, self.w_down.w[:, e * ff:(e + 1) * ff].t(), out=y[a:b])
        return ops.experts_combine(y, dest, weights)
