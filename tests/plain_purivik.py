"""Purivik in float64 NumPy: one function a mechanism, whole sequences, no cache.  It shares no code with the package and is
what the engine's logits are compared with.  `cfg` is the config.json dict, `W` maps tensor names to float64 arrays."""
import math

import numpy as np


def rms(x, weight, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * weight


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotary_frequencies(rot):
    """f_i = base^(-2i/dims), then the banded scaling: long waves slowed by `factor`, short waves kept, a blend between."""
    dims = rot["dims"]
    f = np.array([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f
    out = np.empty_like(f)
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < sc["original"] / sc["high"]:
            out[i] = fi
        elif wavelength > sc["original"] / sc["low"]:
            out[i] = fi / sc["factor"]
        else:
            t = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
            out[i] = (1.0 - t) * fi / sc["factor"] + t * fi
    return out


def rotate(x, rot, positions):
    """x [tokens, heads, dim]: lane i turns with lane i + dims/2 by position * f_i; lanes from dims on stay."""
    if not rot or not rot["dims"]:
        return x
    dims = rot["dims"]
    half = dims // 2
    angle = np.asarray(positions, dtype=np.float64)[:, None] * rotary_frequencies(rot)[None, :]
    c, s = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return np.concatenate([a * c - b * s, b * c + a * s, x[..., dims:]], axis=-1)


def visible(n, mask):
    """[row, key]: key <= row, and with a mask both in the same block of mask.size positions counted from 0."""
    row, key = np.arange(n)[:, None], np.arange(n)[None, :]
    see = key <= row
    if mask:
        see = see & (row // mask["size"] == key // mask["size"])
    return see


def attention(W, prefix, m, h):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = np.arange(n)
    q = rotate((h @ W[prefix + "q"].T).reshape(n, H, d), m.get("rot"), positions)
    k = rotate((h @ W[prefix + "k"].T).reshape(n, G, d), m.get("rot"), positions)
    v = (h @ W[prefix + "v"].T).reshape(n, G, dv)
    see = visible(n, m.get("mask"))
    out = np.empty((n, H, dv))
    for head in range(H):
        g = head // (H // G)
        score = np.where(see, (q[:, head] @ k[:, g].T) * m["scale"], -np.inf)
        weight = np.exp(score - score.max(axis=1, keepdims=True))
        out[:, head] = (weight / weight.sum(axis=1, keepdims=True)) @ v[:, g]
    return out.reshape(n, H * dv) @ W[prefix + "o"].T


def dense_ff(W, prefix, mlp, h):
    limit = mlp["limit"]
    g = np.minimum(h @ W[prefix + "gate"].T, limit)
    u = np.clip(h @ W[prefix + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[prefix + "down"].T


def router(W, prefix, mlp, h):
    """(picks [tokens, top], their scores): the largest sigmoid scores, the lower index among equals."""
    score = sigmoid(h @ W[prefix + "router"].T)
    picks = np.argsort(-score, axis=1, kind="stable")[:, :mlp["router"]["top"]]
    return picks, np.take_along_axis(score, picks, axis=1)


def expert(W, prefix, x):
    g, u = x @ W[prefix + "gate"].T, x @ W[prefix + "up"].T
    return (g * sigmoid(g) * u) @ W[prefix + "down"].T


def experts_ff(W, prefix, mlp, h):
    picks, scores = router(W, prefix, mlp, h)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(picks[t], scores[t]):
            out[t] += expert(W, f"{prefix}e{e}.", s * h[t])      # the score scales what goes INTO the expert
    return out


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg, W, tokens, stream_after_every_run=None):
    """Logits [tokens, vocab]."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    first = W["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    x = first.copy()
    for i, add_first in run_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        if add_first:
            x = x + first
        y = attention(W, p + "mix.", layer["mixer"], rms(x, W[p + "norm1"], eps))
        x = x + mult * (W[p + "ls1"] * rms(y, W[p + "norm1b"], eps))
        mlp = layer.get("mlp")
        if mlp:
            h = rms(x, W[p + "norm2"], eps)
            y = dense_ff(W, p + "mlp.", mlp, h) if mlp["kind"] == "dense" else experts_ff(W, p + "mlp.", mlp, h)
            x = x + mult * (W[p + "ls2"] * rms(y, W[p + "norm2b"], eps))
        if stream_after_every_run is not None:
            stream_after_every_run.append(x.copy())
    return rms(x, W["final.norm"], eps) @ W["embed"].T


def greedy(cfg, W, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(np.argmax(forward(cfg, W, tokens)[-1])))
    return tokens[len(prompt):]
