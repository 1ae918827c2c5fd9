"""The Pisulorn decoder, plain and slow: numpy in float64, one function per mechanism, written from the design's
equations and sharing nothing with the library under test.

A model is ``(cfg, w)``: the parsed config.json and ``{tensor name: float64 array}``.  Everything works on one
sequence; ``Decoder`` carries keys, values, states and convolution tails so that the same functions serve
token-by-token decoding.

Notation.  ``h`` is a sublayer's input ``[T, width]``.  Linear weights are ``[out, in]``: ``y = h W^T``.
``i`` is a query's position, ``j`` a key's.
"""
import math

import numpy as np


# ---------------------------------------------------------------- small functions
def rms_norm(x, gain, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * gain


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ---------------------------------------------------------------- softmax attention
def query_temperature(p, q_temp):
    """The factor on the query at position ``p``: 1 + c ln(floor((p + 1) / n) + 1)."""
    if not q_temp:
        return np.ones_like(np.asarray(p, dtype=np.float64))
    return 1.0 + q_temp["coef"] * np.log(np.floor((np.asarray(p) + 1) / q_temp["every"]) + 1.0)


def distance_slopes(heads):
    """One slope per query head: 2^(-8 (h + 1) / H)."""
    return np.array([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)])


def attention_qkv(m, w, pre, h, positions, eps):
    """Normed and tempered queries ``[T, H, dim]``, normed keys ``[T, G, dim]``, values ``[T, G, vdim]``."""
    T = h.shape[0]
    q = (h @ w[pre + "q"].T).reshape(T, m["heads"], m["dim"])
    k = (h @ w[pre + "k"].T).reshape(T, m["kv_heads"], m["dim"])
    v = (h @ w[pre + "v"].T).reshape(T, m["kv_heads"], m.get("vdim", m["dim"]))
    q = rms_norm(q, w[pre + "q.norm"], eps)
    k = rms_norm(k, w[pre + "k.norm"], eps)
    q = q * query_temperature(positions, m.get("q_temp"))[:, None, None]
    return q, k, v


def visible(m, q_positions, key_positions):
    """``[T_q, T_k]`` booleans: 0 <= i - j, and i - j < window where there is one."""
    d = np.asarray(q_positions)[:, None] - np.asarray(key_positions)[None, :]
    ok = d >= 0
    mask = m.get("mask")
    if mask and mask.get("size"):
        ok &= d < mask["size"]
    return ok


def attention_core(m, q, k, v, q_positions):
    """Causal softmax attention with the distance bias.  ``k``, ``v`` hold all keys from position 0."""
    T = q.shape[0]
    rep = m["heads"] // m["kv_heads"]
    out = np.zeros((T, m["heads"], v.shape[-1]))
    key_pos = np.arange(k.shape[0])
    dist = np.asarray(q_positions)[:, None] - key_pos[None, :]
    see = visible(m, q_positions, key_pos)
    slopes = distance_slopes(m["heads"])
    for head in range(m["heads"]):
        g = head // rep
        s = (q[:, head] @ k[:, g].T) * m["scale"] - slopes[head] * dist
        s = np.where(see, s, -np.inf)
        s = s - s.max(-1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(-1, keepdims=True)
        out[:, head] = p @ v[:, g]
    return out


def attention_mixer(m, w, pre, h, eps, cache, first_pos):
    """``cache`` is a dict that keeps this run's keys and values between calls."""
    T = h.shape[0]
    positions = np.arange(first_pos, first_pos + T)
    q, k, v = attention_qkv(m, w, pre, h, positions, eps)
    if "k" in cache:
        k, v = np.concatenate([cache["k"], k]), np.concatenate([cache["v"], v])
    cache["k"], cache["v"] = k, v
    o = attention_core(m, q, k, v, positions)
    return o.reshape(T, -1) @ w[pre + "o"].T


# ---------------------------------------------------------------- gated delta rule
def short_convolution(x, taps, tail):
    """``x [T, C]``, ``taps [C, K]`` (last column: the current token's), ``tail [K - 1, C]``: the inputs before
    ``x`` (zeros at a sequence's start).  Returns silu of the convolution and the new tail."""
    K = taps.shape[1]
    full = np.concatenate([tail, x], 0)
    y = np.zeros_like(x)
    for t in range(x.shape[0]):
        y[t] = (full[t:t + K] * taps.T).sum(0)
    return silu(y), full[full.shape[0] - (K - 1):]


def unit(x):
    return x / np.sqrt((x * x).sum(-1, keepdims=True) + 1e-6)


def delta_recurrence(q, k, v, beta, g, state):
    """One head.  ``state [dim, vdim]`` is changed in place: S <- g S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q."""
    out = np.zeros((q.shape[0], v.shape[1]))
    for t in range(q.shape[0]):
        state *= g[t]
        u = beta[t] * (v[t] - state.T @ k[t])
        state += np.outer(k[t], u)
        out[t] = state.T @ q[t]
    return out


def delta_mixer(m, w, pre, h, eps, cache, first_pos):
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    dv = m.get("vdim", dk)
    if "state" not in cache:
        cache["state"] = np.zeros((H, dk, dv))
        for n in "qkv":
            taps = w[pre + n + ".conv"]
            cache["tail_" + n] = np.zeros((taps.shape[1] - 1, taps.shape[0]))
    proj = {}
    for n in "qkv":
        proj[n], cache["tail_" + n] = short_convolution(h @ w[pre + n].T, w[pre + n + ".conv"], cache["tail_" + n])
    q = unit(proj["q"].reshape(T, G, dk)) * dk ** -0.5
    k = unit(proj["k"].reshape(T, G, dk))
    v = proj["v"].reshape(T, H, dv)
    beta = sigmoid(h @ w[pre + "b"].T)                                                        # [T, H]
    g = np.exp(-np.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))   # [T, H]
    rep = H // G
    o = np.stack([delta_recurrence(q[:, i // rep], k[:, i // rep], v[:, i], beta[:, i], g[:, i], cache["state"][i])
                  for i in range(H)], 1)
    o = rms_norm(o, w[pre + "norm"], eps).reshape(T, H * dv)
    return (o * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


MIXERS = {"attention": attention_mixer, "delta": delta_mixer}


# ---------------------------------------------------------------- feed-forward
def dense_ff(mlp, w, pre, h):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


ROUTE_MARGINS = None      # a list: route() then notes, per call, every token's gap between the last expert chosen and the best one left out


def route(mlp, w, pre, h):
    """Chosen experts ``[T, top]`` and their weights ``[T, top]``: sigmoid scores, the choice by score plus
    correction, the weights from the scores alone, normalised."""
    s = sigmoid(h @ w[pre + "router"].T)
    choice = s + w[pre + "correction"]
    top = mlp["router"]["top"]
    if ROUTE_MARGINS is not None and top < choice.shape[-1]:
        ranked = -np.sort(-choice, axis=-1)
        ROUTE_MARGINS.append(ranked[:, top - 1] - ranked[:, top])
    chosen = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, -1)
    return chosen, picked / (picked.sum(-1, keepdims=True) + 1e-20)


def expert(mlp, w, pre, h):
    limit = mlp["expert"]["limit"]
    g = np.minimum(h @ w[pre + "gate"].T, limit)
    u = np.clip(h @ w[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def moe_ff(mlp, w, pre, h):
    chosen, weights = route(mlp, w, pre, h)
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            out[t] += a * expert(mlp, w, f"{pre}e{e}.", h[t:t + 1])[0]
    return out


def feed_forward(mlp, w, pre, h):
    return {"dense": dense_ff, "moe": moe_ff}[mlp["kind"]](mlp, w, pre, h)


# ---------------------------------------------------------------- residual
def hyper_sublayer(streams, w, pre, branch, m):
    """``streams [S, T, width]``; ``branch(u)`` is norm and sublayer together.  Returns the new streams:
    x_t' = sum_s mix[s, t] x_s + m out[t] y with y = branch(sum_s in[s] x_s)."""
    u = np.tensordot(w[pre + "in"], streams, axes=(0, 0))
    y = branch(u)
    mixed = np.tensordot(w[pre + "mix"].T, streams, axes=(1, 0))        # [to, T, width]
    return mixed + m * w[pre + "out"][:, None, None] * y[None]


def schedule(cfg):
    """Layer indices in the order the layers run: the looped stretch several times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop.get("times", 1) + list(range(b, n))


class Decoder:
    """One sequence fed in pieces of any size."""

    def __init__(self, cfg, w):
        self.cfg, self.w = cfg, w
        self.order = schedule(cfg)
        self.caches = [dict() for _ in self.order]
        self.length = 0

    def feed(self, tokens, layers_out=None):
        """Logits ``[len(tokens), vocab]``; ``layers_out``, a list, gets the residual after every layer run."""
        cfg, w = self.cfg, self.w
        eps = cfg["norm"]["eps"]
        m = cfg.get("residual_mult", 1.0)
        x = w["embed"][np.asarray(tokens)]
        hyper = bool(cfg.get("streams"))
        xs = np.repeat(x[None], cfg["streams"], 0) if hyper else None
        for run, li in enumerate(self.order):
            layer = cfg["layers"][li]
            p = f"l{li}."
            mix = lambda u: MIXERS[layer["type"]](layer["mixer"], w, p + "mix.", rms_norm(u, w[p + "norm1"], eps), eps,
                                                  self.caches[run], self.length)
            ff = lambda u: feed_forward(layer["mlp"], w, p + "mlp.", rms_norm(u, w[p + "norm2"], eps))
            if hyper:
                xs = hyper_sublayer(xs, w, p + "hc1.", mix, m)
                if layer.get("mlp"):
                    xs = hyper_sublayer(xs, w, p + "hc2.", ff, m)
                x = xs.sum(0)
            else:
                x = x + m * mix(x)
                if layer.get("mlp"):
                    x = x + m * ff(x)
            if layers_out is not None:
                layers_out.append(x.copy())
        self.length += len(tokens)
        return rms_norm(x, w["final.norm"], eps) @ w["head"].T


def logits(cfg, w, tokens):
    return Decoder(cfg, w).feed(tokens)


def greedy(cfg, w, prompt, n):
    """``n`` greedy tokens after ``prompt`` and the logits rows they were picked from."""
    d = Decoder(cfg, w)
    row = d.feed(prompt)[-1]
    toks, rows = [], []
    for _ in range(n):
        rows.append(row)
        toks.append(int(np.argmax(row)))
        if len(toks) < n:
            row = d.feed([toks[-1]])[-1]
    return toks, rows
