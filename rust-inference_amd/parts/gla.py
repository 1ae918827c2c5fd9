"""Gated linear attention: a mixer that keeps a state of fixed size per sequence instead of keys and values."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import StateNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "gla")
class GatedLinearAttention(Mixer):
    """Per head, with ``q = W_q h / sqrt(dim)``, ``k = W_k h`` (``heads x dim``), ``v = W_v h`` (``heads x vdim``)
    and one decay per key channel, ``alpha = sigmoid(z)^(1 / tau)``, ``z = W_a2 (W_a1 h) + b`` (a product through a
    narrow middle whose width the checkpoint alone gives, unless ``decay_rank`` names it):

        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T q_t.

    Each head's ``o`` goes through an RMS norm over ``vdim`` (one gain for all heads), the heads side by side are
    multiplied by ``silu(W_g h)`` and projected by ``W_o``.  The state ``[heads, dim, vdim]`` starts at zero and
    is float32, as are the decay, its logarithm and the recurrence's sums; it lives in the cache's state arena
    at the sequence's slot, so a sequence goes on from it in any later step.

    ``names``: checkpoint names of ``q, k, v, g, o, norm, a1, a2, a2_bias`` where they are not ``<prefix>q``
    and so on.  q, k, v and g are one product with the row-concatenated weight.
    """

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, tau: float, prefix: str, eps: float = 1e-5,
                 decay_rank: int | None = None, names: dict | None = None):
        if heads < 1 or not 1 <= dim <= ops.GLA_MAX_DIM or vdim < 1 or vdim > 512:
            raise ConfigError(f"gated linear attention with {heads} heads of {dim} x {vdim}: the kernels take key heads "
                              f"of 1 to {ops.GLA_MAX_DIM} and value heads of 1 to 512")
        if not tau > 0:
            raise ConfigError(f"tau {tau} must be positive")
        self.hidden, self.heads, self.dim, self.vdim, self.tau = hidden, heads, dim, vdim, float(tau)
        self.prefix, self.eps, self.decay_rank = prefix, eps, decay_rank
        p = prefix
        self.names = {"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "o": p + "o", "norm": p + "norm",
                      "a1": p + "a1", "a2": p + "a2", "a2_bias": p + "a2.b"}
        self.names.update(names or {})

    def tensors(self):
        n, d, hk, hv = self.names, self.hidden, self.heads * self.dim, self.heads * self.vdim
        return {
            n["q"]: TensorSpec((hk, d), MATRIX), n["k"]: TensorSpec((hk, d), MATRIX),
            n["v"]: TensorSpec((hv, d), MATRIX), n["g"]: TensorSpec((hv, d), MATRIX),
            n["o"]: TensorSpec((d, hv), MATRIX), n["norm"]: TensorSpec((self.vdim,), GAIN),
            n["a1"]: TensorSpec((self.decay_rank, d), MATRIX), n["a2"]: TensorSpec((hk, self.decay_rank), MATRIX),
            n["a2_bias"]: TensorSpec((hk,), BIAS),
        }

    def bind(self, weights, rt):
        self.rt = rt
        n = self.names
        if weights[n["a1"]].shape[0] != weights[n["a2"]].shape[1]:
            raise ConfigError(f"{n['a1']} has {weights[n['a1']].shape[0]} rows, {n['a2']} {weights[n['a2']].shape[1]} columns")
        fused = torch.cat([weights[n["q"]], weights[n["k"]], weights[n["v"]], weights[n["g"]]], 0)
        self.w_qkvg = rt.pack(rt.place_matrix(fused), always=True)      # four projections in one: always worth its packed copy
        self.w_a1 = rt.pack(rt.place_matrix(weights[n["a1"]]))
        self.w_a2 = rt.pack(rt.place_matrix(weights[n["a2"]]))
        self.z_bias = rt.place_gain(weights[n["a2_bias"]])
        self.gain = rt.place_gain(weights[n["norm"]])
        self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)

    def cache_need(self):
        return StateNeed((self.heads, self.dim, self.vdim), torch.float32)

    def forward(self, x, ctx, store, page_table):
        rt, hk, hv = self.rt, self.heads * self.dim, self.heads * self.vdim
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_qkvg))          # [T, q | k | v | g]
            z = rt.linear_packed(ops.as_rows(rt.linear_packed(x, self.w_a1)), self.w_a2, out_dtype=torch.float32)
        if ctx.is_decode and ops.gla_step_fits(self.dim, self.vdim):
            # one token a sequence: the step on the state, the norm and the gate are one kernel
            with profiler.section(profiler.ATTENTION):
                y = ops.gla_step(proj, 0, hk, 2 * hk, 2 * hk + hv, z, self.z_bias, self.tau, self.dim ** -0.5, store,
                                 ctx.slots, self.gain, self.eps, self.heads, self.dim, self.vdim)
            with profiler.section(profiler.OUT_PROJECTION):
                return rt.linear_packed(y, self.w_o, out_dtype=torch.float32, parts_ok=True)
        with profiler.section(profiler.ATTENTION):
            o = ops.gla_scan(proj, 0, hk, 2 * hk, z, self.z_bias, self.tau, self.dim ** -0.5, store, ctx.cu_seqlens,
                             ctx.slots, self.heads, self.dim, self.vdim)
            y = ops.gla_norm_gate(o, proj, 2 * hk + hv, self.gain, self.eps, self.heads, self.vdim)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(y, self.w_o, out_dtype=torch.float32, parts_ok=True)
