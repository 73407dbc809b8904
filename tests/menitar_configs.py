"""Tiny Menitar configurations and weights for tests.  The weights are drawn here, larger than a checkpoint's random
init, so that scores differ between keys and heads (with weights of deviation 0.02 every softmax is nearly flat and a
wrong key, a missing gate or an unmixed score would hide in the rounding)."""
import json
import os

import numpy as np
import torch


def layer(heads, kv_heads, dim, vdim, chunk=None, rot=None, ff=None, limit=2.0, scale=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
    mlp = None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config(width, vocab, layers, loop=None, eps=1e-5, embedding_scale=3.0, logit_scale=0.5):
    cfg = {"architecture": "Menitar", "width": width, "vocab": vocab, "embedding": {"scale": embedding_scale},
           "logit_scale": logit_scale, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# P: looped first two layers (three passes), a layer without feed-forward, keys wider than values, partial rotary
P = config(64, 96, [layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0), ff=80),
                    layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0)),
                    layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0), ff=80, limit=0.75)], loop=(0, 2, 3))
# Q: as many key/value heads as heads, every lane rotated, no loop, chunks that are no multiple of the page
Q = config(96, 120, [layer(3, 3, 32, 32, chunk=40, rot=(32, 500.0), ff=112),
                     layer(3, 3, 32, 32, chunk=40, rot=(32, 500.0), ff=112)], logit_scale=1.5, eps=1e-6)
# R: one key/value head, head sizes that no matrix-core kernel takes (keys stored lane by lane), no rotation, no mask
# (every earlier key is seen), a loop of one pass over the last layer
R = config(48, 80, [layer(2, 1, 20, 12, ff=64), layer(2, 1, 20, 12, ff=64, limit=3.0)], loop=(1, 2, 1), embedding_scale=1.0)
# S: layers of different geometry (two cache groups), sizes the matrix-core kernel takes, a loop in the middle
S = config(128, 160, [layer(8, 2, 64, 32, chunk=80, rot=(32, 25000.0), ff=192),
                      layer(2, 1, 32, 64, chunk=16, rot=(8, 100.0), ff=192),
                      layer(8, 2, 64, 32, chunk=80, rot=(32, 25000.0), ff=192)], loop=(1, 3, 2))
# T: twelve heads (the wider instance of the matrix-core kernel), a chunk of one page
T = config(64, 72, [layer(12, 4, 32, 16, chunk=16, rot=(32, 3000.0), ff=96)])
# U: sizes that are multiples of nothing (width, vocabulary, feed-forward), heads of 24 lanes with values of 20, three heads
# on one key/value head, a chunk of 7 positions, a loop over every layer
U = config(68, 77, [layer(3, 1, 24, 20, chunk=7, rot=(10, 77.0), ff=50, limit=0.9),
                    layer(3, 1, 24, 20, chunk=7, rot=(10, 77.0), ff=50, limit=0.9)], loop=(0, 2, 2), embedding_scale=2.0, logit_scale=3.0)
# V: twenty heads on four key/value heads (more heads than the row-tile kernel holds: prompts run the plain kernel, decode
# steps the matrix-core one), values wider than keys
V = config(80, 90, [layer(20, 4, 32, 48, chunk=48, rot=(32, 1000.0), ff=120)])
CONFIGS = {"P": P, "Q": Q, "R": R, "S": S, "T": T, "U": U, "V": V}
PAGE_SIZES = {"P": 8, "Q": 16, "R": 8, "S": 16, "T": 16, "U": 16, "V": 16}


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32)


def weights(cfg, seed):
    """name -> float32 torch tensor whose values are exact in bfloat16 (both precisions load the same numbers)."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {"embed": rng.normal(0, 0.4, (cfg["vocab"], W)), "final.norm": 1 + rng.uniform(-0.3, 0.3, W)}
    if cfg.get("loop"):
        out["loop.step"] = rng.normal(0, 0.5, (cfg["loop"]["times"], W))
    for i, spec in enumerate(cfg["layers"]):
        m = spec["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = f"l{i}."
        out[p + "norm1"] = 1 + rng.uniform(-0.3, 0.3, W)
        out[p + "mix.q"] = rng.normal(0, W ** -0.5, (H * d, W))
        out[p + "mix.k"] = rng.normal(0, W ** -0.5, (G * d, W))
        out[p + "mix.v"] = rng.normal(0, W ** -0.5, (G * dv, W))
        out[p + "mix.o"] = rng.normal(0, (H * dv) ** -0.5, (W, H * dv))
        out[p + "mix.g"] = rng.normal(0, 2 * W ** -0.5, (H, W))
        out[p + "mix.q.norm"] = 1.5 + rng.uniform(-0.5, 0.5, H * d)
        out[p + "mix.k.norm"] = 1.5 + rng.uniform(-0.5, 0.5, G * d)
        out[p + "mix.talk"] = np.eye(H) + rng.normal(0, 0.4, (H, H))
        out[p + "mix.temp"] = rng.uniform(0.5, 2.5, H)
        if spec["mlp"] is not None:
            ff = spec["mlp"]["ff"]
            out[p + "norm2"] = 1 + rng.uniform(-0.3, 0.3, W)
            out[p + "mlp.gate"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[p + "mlp.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[p + "mlp.down"] = rng.normal(0, ff ** -0.5, (W, ff))
    return {n: bf16_round(a) for n, a in out.items()}


def to_float64(tensors):
    return {n: t.to(torch.float64).numpy() for n, t in tensors.items()}


def write_model(folder, cfg, tensors, dtype=torch.bfloat16):
    from fllm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), {n: t.to(dtype) for n, t in tensors.items()})
    return folder


def random_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()
