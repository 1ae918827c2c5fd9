"""Pisulorn as a list of parts.

Embedding: the token's row.  Every layer is pre-norm with RMS norms: a mixer of the layer's own kind and sizes,
softmax attention without rotation (per-head q/k RMS norm, a query temperature by position, a scaled score minus
a per-head slope times the distance, an optional sliding window) or the gated delta rule (short convolutions over
q, k and v, unit q and k, a float32 state per head), and an optional feed-forward, dense with the tanh form of GELU
or a mixture of experts with a sigmoid router.  Every sublayer's output enters the residual times
``residual_mult``.  A stretch of the layers may run several times in a row with the same weights, every pass with
cache entries of its own.  With ``streams`` the residual is kept in that many copies joined by each sublayer's
hyper-connection.  Final RMS norm, output matrix.

Checkpoint names: ``embed``, ``l<i>.norm1`` / ``norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.hc1.*`` / ``hc2.*``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config import PisulornConfig, register_architecture
from ..config.pisulorn import DenseSizes
from .spec import LayerSpec, ModelSpec, PartSpec, Run


def distance_slopes(heads: int) -> tuple:
    """The design's slope of query head ``h``: 2^(-8 (h + 1) / heads)."""
    return tuple(2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads))


def _norm(cfg: PisulornConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.norm_eps, "name": name})


def _mixer(cfg: PisulornConfig, layer, p: str) -> PartSpec:
    m = layer.mixer
    if layer.type == "attention":
        return PartSpec("attention", {
            "hidden": cfg.width, "heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim, "v_dim": m.vdim,
            "prefix": p, "qk_norm": True, "eps": cfg.norm_eps, "window": m.window, "scale": m.scale,
            "q_temper": None if m.temper_coef is None else (m.temper_coef, m.temper_every),
            "distance_slopes": distance_slopes(m.heads),
            "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "q_norm": p + "q.norm", "k_norm": p + "k.norm"},
        })
    return PartSpec("delta", {"hidden": cfg.width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                              "taps": m.conv, "prefix": p, "eps": cfg.norm_eps})


def _feed_forward(cfg: PisulornConfig, mlp, p: str) -> PartSpec:
    if isinstance(mlp, DenseSizes):
        return PartSpec("dense", {"hidden": cfg.width, "inter": mlp.ff, "prefix": p, "activation": "gelu_tanh",
                                  "names": {"up": p + "up", "down": p + "down"}})
    return PartSpec("routed_experts", {"hidden": cfg.width, "inter": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                                       "limit": mlp.limit, "prefix": p})


def _connection(cfg: PisulornConfig, prefix: str) -> PartSpec:
    if cfg.streams is None:           # one residual: x <- x + m y, as a connection with fixed coefficients
        return PartSpec("scaled_add", {"scale": cfg.residual_mult})
    return PartSpec("hyper", {"streams": cfg.streams, "prefix": prefix, "out_scale": cfg.residual_mult})


def pisulorn_spec(cfg: PisulornConfig) -> ModelSpec:
    layers, entries_of = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer_norm": _norm(cfg, p + "norm1"), "mixer": _mixer(cfg, layer, p + "mix."),
                 "mixer_connection": _connection(cfg, p + "hc1.")}
        if layer.mlp is not None:
            parts["feed_forward_norm"] = _norm(cfg, p + "norm2")
            parts["feed_forward"] = _feed_forward(cfg, layer.mlp, p + "mlp.")
            parts["feed_forward_connection"] = _connection(cfg, p + "hc2.")
        layers.append(LayerSpec("hyper_prenorm", parts))
        entries_of.append(1 if layer.type == "attention" else 2)      # keys and values; or the state and the convolutions' tails
    # every run of a layer, a looped one's every pass too, keeps its own keys and values or state
    schedule, at = [], 0
    for i in cfg.order():
        n = entries_of[i]
        schedule.append(Run(layer=i, cache=at if n == 1 else tuple(range(at, at + n))))
        at += n
    return ModelSpec(
        architecture=cfg.ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("table", {"vocab": cfg.vocab, "dim": cfg.width, "name": "embed"}),
        layers=tuple(layers),
        schedule=tuple(schedule),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab": cfg.vocab, "dim": cfg.width, "name": "head", "tied": False}),
        max_positions=cfg.max_positions,
        stream=PartSpec("hyper", {"streams": cfg.streams or 1}),
    )


register_architecture("Pisulorn", PisulornConfig, pisulorn_spec, model_types=("pisulorn",))
