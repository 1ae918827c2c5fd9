"""The gated delta rule: a mixer that keeps a float32 state per head and the tails of three short convolutions."""
from __future__ import annotations

import torch

from .. import profiler
from ..cache import StateNeed
from ..errors import ConfigError
from ..kernels import ops
from ..weights.loader import BIAS, GAIN, MATRIX, TensorSpec
from .base import Mixer
from .registry import register_part


@register_part("mixer", "delta")
class GatedDeltaRule(Mixer):
    """With ``q = W_q h`` and ``k = W_k h`` (``kv_heads x dim``, shared by ``heads / kv_heads`` value heads each) and
    ``v = W_v h`` (``heads x vdim``): each of q, k and v goes through a causal convolution over time per channel
    (``taps`` taps, the last one the current token's, zeros before a sequence's start) and silu; q and k become unit
    vectors per head, ``x / sqrt(sum x^2 + 1e-6)``, q also times ``dim^(-1/2)``; ``beta = sigmoid(W_b h)`` and
    ``g = exp(-exp(A_log) softplus(W_a h + dt_bias))`` per value head.  Per head and token

        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q,

    so that the read-out sees the token's own write.  Each head's ``o`` goes through an RMS norm over ``vdim`` (one
    gain for all heads), the heads side by side are multiplied by ``silu(W_g h)`` and projected by ``W_o``.

    Per sequence the mixer keeps two things, in this order: the state ``[heads, dim, vdim]`` and the last ``taps - 1``
    inputs of the convolutions ``[taps - 1, channels]``, both float32 and zero when the sequence starts; a run of a
    layer with this mixer names two cache entries.  Everything after the projections is float32.

    ``names``: checkpoint names of ``q, k, v, g, o, a, b, norm, A_log, dt_bias`` where they are not ``<prefix>q`` and
    so on; the taps of q, k and v are ``<name>.conv``.  q, k, v and g are one product with the row-concatenated
    weight, a and b another whose result is float32.
    """

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, prefix: str,
                 eps: float = 1e-5, names: dict | None = None):
        if heads < 1 or kv_heads < 1 or heads % kv_heads:
            raise ConfigError(f"{heads} delta-rule heads not divisible by {kv_heads} query/key heads")
        if not 1 <= dim <= ops.DELTA_MAX_DIM or vdim < 1:
            raise ConfigError(f"a delta rule with heads of {dim} x {vdim}: the kernels take key heads of 1 to {ops.DELTA_MAX_DIM}")
        if not 1 <= taps <= ops.DELTA_MAX_TAPS:
            raise ConfigError(f"short convolutions of {taps} taps: the kernels take 1 to {ops.DELTA_MAX_TAPS}")
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim, self.taps = hidden, heads, kv_heads, dim, vdim, taps
        self.prefix, self.eps = prefix, eps
        p = prefix
        self.names = {n: p + n for n in ("q", "k", "v", "g", "o", "a", "b", "norm", "A_log", "dt_bias")}
        self.names.update(names or {})
        self.channels = 2 * kv_heads * dim + heads * vdim

    def tensors(self):
        n, d, hk, hv, h = self.names, self.hidden, self.kv_heads * self.dim, self.heads * self.vdim, self.heads
        return {
            n["q"]: TensorSpec((hk, d), MATRIX), n["k"]: TensorSpec((hk, d), MATRIX), n["v"]: TensorSpec((hv, d), MATRIX),
            n["q"] + ".conv": TensorSpec((hk, self.taps), MATRIX), n["k"] + ".conv": TensorSpec((hk, self.taps), MATRIX),
            n["v"] + ".conv": TensorSpec((hv, self.taps), MATRIX),
            n["g"]: TensorSpec((hv, d), MATRIX), n["o"]: TensorSpec((d, hv), MATRIX),
            n["a"]: TensorSpec((h, d), MATRIX), n["b"]: TensorSpec((h, d), MATRIX),
            n["A_log"]: TensorSpec((h,), BIAS), n["dt_bias"]: TensorSpec((h,), BIAS),
            n["norm"]: TensorSpec((self.vdim,), GAIN),
        }

    def bind(self, weights, rt):
        self.rt = rt
        n = self.names
        fused = torch.cat([weights[n["q"]], weights[n["k"]], weights[n["v"]], weights[n["g"]]], 0)
        self.w_qkvg = rt.pack(rt.place_matrix(fused), always=True)      # four projections in one
        self.w_ab = rt.pack(rt.place_matrix(torch.cat([weights[n["a"]], weights[n["b"]]], 0)))
        self.conv_taps = rt.place_gain(torch.cat([weights[n[x] + ".conv"] for x in "qkv"], 0))
        self.a_log, self.dt_bias = rt.place_gain(weights[n["A_log"]]), rt.place_gain(weights[n["dt_bias"]])
        self.gain = rt.place_gain(weights[n["norm"]])
        self.w_o = rt.pack(rt.place_matrix(weights[n["o"]]), parts_ok=True)

    def cache_need(self):
        return (StateNeed((self.heads, self.dim, self.vdim), torch.float32),
                StateNeed((self.taps - 1, self.channels), torch.float32))

    def forward(self, x, ctx, store, page_table):
        rt = self.rt
        state, tails = store
        with profiler.section(profiler.QKV_PROJECTION):
            proj = ops.as_rows(rt.linear_packed(x, self.w_qkvg))          # [T, q | k | v | g]
            ab = rt.linear_packed(x, self.w_ab, out_dtype=torch.float32)
        # float32 and the invariant mode run one form of every kernel whatever the step looks like
        one_form = rt.dtype == torch.float32 or rt.invariant
        if ctx.is_decode and not one_form and ops.delta_step_fits(self.dim, self.vdim):
            # one token a sequence: convolutions, unit norms, gates, the step on the state, norm and gate are one kernel
            with profiler.section(profiler.ATTENTION):
                y = ops.delta_step(proj, 0, self.channels, self.conv_taps, tails, ab, self.a_log, self.dt_bias, state,
                                   ctx.cu_seqlens, ctx.slots, self.gain, self.eps, self.heads, self.kv_heads, self.dim,
                                   self.vdim)
            with profiler.section(profiler.OUT_PROJECTION):
                return rt.linear_packed(y, self.w_o, out_dtype=torch.float32, parts_ok=True)
        with profiler.section(profiler.ATTENTION):
            qkv, gates = ops.delta_prepare(proj, 0, self.conv_taps, tails, ab, self.a_log, self.dt_bias, ctx.tok_seq,
                                           ctx.cu_seqlens, ctx.slots, self.heads, self.kv_heads, self.dim, self.vdim)
            o = ops.delta_scan(qkv, gates, state, ctx.cu_seqlens, ctx.slots, self.heads, self.kv_heads, self.dim,
                               self.vdim, slices=4 if one_form else 0)
            y = ops.gla_norm_gate(o, proj, self.channels, self.gain, self.eps, self.heads, self.vdim)
        with profiler.section(profiler.OUT_PROJECTION):
            return rt.linear_packed(y, self.w_o, out_dtype=torch.float32, parts_ok=True)
