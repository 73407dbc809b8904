"""A plain, slow Menitar: whole sequences, no cache, float64, one function per mechanism.

It shares no code with `fllm_amd`.  Weights come in as a dict of float64 NumPy arrays under the checkpoint's tensor
names, the configuration as the config.json dict.

The design in this file's notation (n = tokens, W = width):
  x0 = E[tokens] * embedding.scale
  the layers loop.start .. loop.stop - 1 run loop.times times in a row; before pass t > 0 x += x0, before every pass
  x += loop.step[t]; the other layers run once, in order
  a layer:  x += mixer(rms(x; norm1)) + ff(rms(x; norm2))            (both branches read the same x)
  logits = E rms(x; final.norm) * logit_scale
"""
import math

import numpy as np


def rms(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * np.asarray(weight, dtype=np.float64)


def rotate_half_layout(x, positions, dims, base):
    """x [n, heads, dim]: lane i < dims/2 of every head is paired with lane i + dims/2; the pair (u, v) at position p
    becomes (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2 i / dims).  Lanes from `dims` on stay."""
    if not dims:
        return x
    out = np.array(x, dtype=np.float64)
    half = dims // 2
    freq = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    a = np.asarray(positions, dtype=np.float64)[:, None, None] * freq[None, None, :]
    u, v = out[..., :half].copy(), out[..., half:dims].copy()
    out[..., :half] = u * np.cos(a) - v * np.sin(a)
    out[..., half:dims] = v * np.cos(a) + u * np.sin(a)
    return out


def visible(n, chunk):
    """[n, n] booleans: i sees j <= i of its own chunk of `chunk` positions (None: every j <= i)."""
    i = np.arange(n)[:, None]
    j = np.arange(n)[None, :]
    see = j <= i
    if chunk:
        see &= (i // chunk) == (j // chunk)
    return see


def mixed_scores(q, k, scale, temp, talk, group):
    """[heads, n, n]: (q_h . k_{h / group}) * scale * temp[h], then head h gets sum_g talk[h, g] * score_g."""
    heads = q.shape[1]
    raw = np.stack([q[:, h, :] @ k[:, h // group, :].T * scale * temp[h] for h in range(heads)])
    return np.einsum("hg,gij->hij", talk, raw)


def softmax_rows(s, see):
    s = np.where(see, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def attention_mixer(h, w, prefix, m, eps, positions=None):
    """The mixer of one layer over a whole sequence h [n, W]; `m` is the layer's `mixer` dict."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = np.arange(n) if positions is None else positions
    t = lambda name: np.asarray(w[prefix + name], dtype=np.float64)
    q = rms(h @ t("q").T, t("q.norm"), eps).reshape(n, H, d)          # one norm over all rows of the projection
    k = rms(h @ t("k").T, t("k.norm"), eps).reshape(n, G, d)
    v = (h @ t("v").T).reshape(n, G, dv)
    rot = m.get("rot") or {}
    q = rotate_half_layout(q, positions, rot.get("dims", 0), rot.get("base", 1.0))
    k = rotate_half_layout(k, positions, rot.get("dims", 0), rot.get("base", 1.0))
    s = mixed_scores(q, k, m["scale"], t("temp"), t("talk"), H // G)
    p = softmax_rows(s, visible(n, (m.get("mask") or {}).get("size")))
    out = np.stack([p[hh] @ v[:, hh // (H // G), :] for hh in range(H)], axis=1)      # [n, H, dv]
    gate = 1.0 / (1.0 + np.exp(-(h @ t("g").T)))                                      # [n, H]
    out = out * gate[:, :, None]
    return out.reshape(n, H * dv) @ t("o").T


def dense_ff(h, w, prefix, mlp):
    """g = min(gate h, limit), u = clamp(up h, -limit, limit); down (g sigmoid(1.702 g) (u + 1))."""
    t = lambda name: np.asarray(w[prefix + name], dtype=np.float64)
    limit = mlp["limit"]
    g = np.minimum(h @ t("gate").T, limit)
    u = np.clip(h @ t("up").T, -limit, limit)
    y = g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)
    return y @ t("down").T


def layer(x, w, i, spec, eps):
    p = f"l{i}."
    out = attention_mixer(rms(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps)
    if spec.get("mlp") is not None:
        out = out + dense_ff(rms(x, w[p + "norm2"], eps), w, p + "mlp.", spec["mlp"])
    return x + out


def run_order(cfg):
    """[(layer, pass number or None)]: None for layers outside the loop."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(start)]
    for t in range(times):
        order += [(i, t) for i in range(start, stop)]
    return order + [(i, None) for i in range(stop, n)]


def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] of a whole sequence.  `layers_out`: a list that receives x after every layer run."""
    eps = cfg["norm"]["eps"]
    table = np.asarray(w["embed"], dtype=np.float64)
    x0 = table[np.asarray(tokens)] * cfg["embedding"]["scale"]
    x = x0.copy()
    loop = cfg.get("loop")
    for i, t in run_order(cfg):
        if t is not None and i == loop["start"]:
            if t > 0:
                x = x + x0
            x = x + np.asarray(w["loop.step"], dtype=np.float64)[t]
        x = layer(x, w, i, cfg["layers"][i], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms(x, w["final.norm"], eps) @ table.T * cfg["logit_scale"]


def greedy(cfg, w, tokens, count):
    """`count` tokens after `tokens`, each the first index of the largest logit, the whole sequence run again each time."""
    tokens = list(tokens)
    out = []
    for _ in range(count):
        out.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
        tokens.append(out[-1])
    return out
