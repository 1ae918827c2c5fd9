"""Zidepel as a list of parts.

Embedding: token row plus learned position row, then a layer norm.  Every layer is pre-norm with layer norms
(gain and bias): a mixer of the layer's own kind and sizes, softmax attention without rotation (per-head q/k RMS
norm, a query temperature by position, a scaled and capped score) or gated linear attention, and an optional
dense feed-forward with a squared ReLU.  A stretch of the layers may run several times in a row with the same
weights, every pass with a cache entry of its own.  With ``streams`` the residual is kept in that many copies
joined by each sublayer's hyper-connection.  Final layer norm, output matrix.

Checkpoint names: ``embed``, ``pos``, ``embed.norm`` (+ ``.b``), ``l<i>.norm1`` / ``norm2`` (+ ``.b``),
``l<i>.mix.*``, ``l<i>.mlp.up`` / ``down``, ``l<i>.hc1.*`` / ``hc2.*``, ``final.norm`` (+ ``.b``), ``head``.
"""
from __future__ import annotations

from ..config import ZidepelConfig, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, Run


def _norm(cfg: ZidepelConfig, name: str) -> PartSpec:
    return PartSpec("layernorm", {"dim": cfg.width, "eps": cfg.norm_eps, "name": name, "bias_name": name + ".b"})


def _mixer(cfg: ZidepelConfig, layer, p: str) -> PartSpec:
    m = layer.mixer
    if layer.type == "attention":
        return PartSpec("attention", {
            "hidden": cfg.width, "heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim, "v_dim": m.vdim,
            "prefix": p, "qk_norm": True, "eps": cfg.norm_eps, "window": None, "scale": m.scale, "softcap": m.softcap,
            "q_temper": None if m.temper_coef is None else (m.temper_coef, m.temper_every),
            "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "q_norm": p + "q.norm", "k_norm": p + "k.norm"},
        })
    return PartSpec("gla", {"hidden": cfg.width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau,
                            "prefix": p, "eps": cfg.norm_eps, "decay_rank": getattr(m, "rank", None)})


def zidepel_spec(cfg: ZidepelConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer_norm": _norm(cfg, p + "norm1"), "mixer": _mixer(cfg, layer, p + "mix.")}
        if layer.ff is not None:
            parts["feed_forward_norm"] = _norm(cfg, p + "norm2")
            parts["feed_forward"] = PartSpec("relu2", {"hidden": cfg.width, "inter": layer.ff, "prefix": p + "mlp.",
                                                       "names": {"up": p + "mlp.up", "down": p + "mlp.down"}})
        if cfg.streams is not None:
            parts["mixer_connection"] = PartSpec("hyper", {"streams": cfg.streams, "prefix": p + "hc1."})
            if layer.ff is not None:
                parts["feed_forward_connection"] = PartSpec("hyper", {"streams": cfg.streams, "prefix": p + "hc2."})
        layers.append(LayerSpec("prenorm" if cfg.streams is None else "hyper_prenorm", parts))
    return ModelSpec(
        architecture=cfg.ARCHITECTURE,
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("table_positions", {"vocab": cfg.vocab, "dim": cfg.width, "max_positions": cfg.max_positions,
                                               "name": "embed", "positions_name": "pos", "norm": _norm(cfg, "embed.norm")}),
        layers=tuple(layers),
        # every run of a layer, a looped one's every pass too, keeps its own keys and values or state
        schedule=tuple(Run(layer=i, cache=run) for run, i in enumerate(cfg.order())),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab": cfg.vocab, "dim": cfg.width, "name": "head", "tied": False}),
        max_positions=cfg.max_positions,
        stream=PartSpec("residual") if cfg.streams is None else PartSpec("hyper", {"streams": cfg.streams}),
    )


register_architecture("Zidepel", ZidepelConfig, zidepel_spec, model_types=("zidepel",))
