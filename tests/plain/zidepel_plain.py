"""The Zidepel decoder, plain and slow: numpy in float64, one function per mechanism, written from the
design's equations and sharing nothing with the library under test.

A model is ``(cfg, w)``: the parsed config.json and ``{tensor name: float64 array}``.  Everything works on one
sequence, positions 0..T-1; ``Decoder`` below carries caches and states so that the same functions serve
token-by-token decoding.

Notation.  ``h`` is a mixer's input ``[T, width]``.  Linear weights are ``[out, in]``: ``y = h W^T``.
"""
import math

import numpy as np


# ---------------------------------------------------------------- small functions
def layer_norm(x, gain, bias, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * gain + bias


def rms_norm(x, gain, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * gain


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


# ---------------------------------------------------------------- embedding
def embed(cfg, w, tokens, first_pos=0):
    """Table row plus learned position row, then the model's norm."""
    pos = np.arange(first_pos, first_pos + len(tokens))
    x = w["embed"][np.asarray(tokens)] + w["pos"][pos]
    return layer_norm(x, w["embed.norm"], w["embed.norm.b"], cfg["norm"]["eps"])


# ---------------------------------------------------------------- softmax attention
def query_temperature(p, q_temp):
    """The factor on the query at position ``p``: 1 + c ln(floor((p + 1) / n) + 1)."""
    if not q_temp:
        return np.ones_like(np.asarray(p, dtype=np.float64))
    return 1.0 + q_temp["coef"] * np.log(np.floor((np.asarray(p) + 1) / q_temp["every"]) + 1.0)


def attention_qkv(m, w, pre, h, positions, eps):
    """Normed and tempered queries ``[T, H, dim]``, normed keys ``[T, G, dim]``, values ``[T, G, vdim]``."""
    T = h.shape[0]
    q = (h @ w[pre + "q"].T).reshape(T, m["heads"], m["dim"])
    k = (h @ w[pre + "k"].T).reshape(T, m["kv_heads"], m["dim"])
    v = (h @ w[pre + "v"].T).reshape(T, m["kv_heads"], m["vdim"])
    q = rms_norm(q, w[pre + "q.norm"], eps)
    k = rms_norm(k, w[pre + "k.norm"], eps)
    q = q * query_temperature(positions, m.get("q_temp"))[:, None, None]
    return q, k, v


def attention_scores(q, k, m):
    """``[T_q, T_k]`` scores of one head after scale and cap."""
    s = (q @ k.T) * m["scale"]
    cap = m.get("softcap")
    return cap * np.tanh(s / cap) if cap else s


def attention_core(m, q, k, v, q_positions):
    """Causal softmax attention: query at position p sees keys 0..p.  ``k``, ``v`` hold all keys from 0."""
    T = q.shape[0]
    rep = m["heads"] // m["kv_heads"]
    out = np.zeros((T, m["heads"], m["vdim"]))
    key_pos = np.arange(k.shape[0])
    for head in range(m["heads"]):
        g = head // rep
        s = attention_scores(q[:, head], k[:, g], m)
        s = np.where(key_pos[None, :] <= np.asarray(q_positions)[:, None], s, -np.inf)
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


# ---------------------------------------------------------------- gated linear attention
def gla_decay(m, w, pre, h):
    """``alpha [T, heads, dim]``: sigmoid(z)^(1/tau), z from the two-step projection and its bias."""
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    return (sigmoid(z) ** (1.0 / m["tau"])).reshape(h.shape[0], m["heads"], m["dim"])


def gla_recurrence(q, k, v, alpha, state):
    """One head.  ``state [dim, vdim]`` is changed in place: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t."""
    out = np.zeros((q.shape[0], v.shape[1]))
    for t in range(q.shape[0]):
        state *= alpha[t][:, None]
        state += np.outer(k[t], v[t])
        out[t] = state.T @ q[t]
    return out


def gla_mixer(m, w, pre, h, eps, cache, first_pos):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, dk)
    v = (h @ w[pre + "v"].T).reshape(T, H, dv)
    alpha = gla_decay(m, w, pre, h)
    if "state" not in cache:
        cache["state"] = np.zeros((H, dk, dv))
    o = np.stack([gla_recurrence(q[:, i], k[:, i], v[:, i], alpha[:, i], cache["state"][i]) for i in range(H)], 1)
    o = rms_norm(o, w[pre + "norm"], eps).reshape(T, H * dv)
    return (o * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


MIXERS = {"attention": attention_mixer, "gla": gla_mixer}


# ---------------------------------------------------------------- feed-forward
def feed_forward(mlp, w, pre, h):
    if mlp["kind"] != "dense":
        raise ValueError(mlp["kind"])
    return relu_squared(h @ w[pre + "up"].T) @ w[pre + "down"].T


# ---------------------------------------------------------------- streams
def hyper_sublayer(streams, w, pre, branch):
    """``streams [S, T, width]``; ``branch(u)`` is norm and sublayer together.  Returns the new streams:
    x_t' = sum_s mix[s, t] x_s + out[t] y with y = branch(sum_s in[s] x_s)."""
    u = np.tensordot(w[pre + "in"], streams, axes=(0, 0))
    y = branch(u)
    mixed = np.tensordot(w[pre + "mix"].T, streams, axes=(1, 0))        # [to, T, width]
    return mixed + w[pre + "out"][:, None, None] * y[None]


def schedule(cfg):
    """(layer index, run index) in the order the layers run: the looped stretch several times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop.get("times", 1) == 1:
        order = list(range(n))
    else:
        a, b = loop["start"], loop["stop"]
        order = list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, n))
    return order


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
        x = embed(cfg, w, tokens, self.length)
        hyper = "streams" in cfg and cfg["streams"]
        xs = np.repeat(x[None], cfg["streams"], 0) if hyper else None
        for run, li in enumerate(self.order):
            layer = cfg["layers"][li]
            p = f"l{li}."
            mix = lambda u: MIXERS[layer["type"]](layer["mixer"], w, p + "mix.", layer_norm(u, w[p + "norm1"], w[p + "norm1.b"], eps),
                                                  eps, self.caches[run], self.length)
            ff = lambda u: feed_forward(layer["mlp"], w, p + "mlp.", layer_norm(u, w[p + "norm2"], w[p + "norm2.b"], eps))
            if hyper:
                xs = hyper_sublayer(xs, w, p + "hc1.", mix)
                if layer.get("mlp"):
                    xs = hyper_sublayer(xs, w, p + "hc2.", ff)
                x = xs.sum(0)
            else:
                x = x + mix(x)
                if layer.get("mlp"):
                    x = x + ff(x)
            if layers_out is not None:
                layers_out.append(x.copy())
        self.length += len(tokens)
        x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
        return x @ w["head"].T


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
