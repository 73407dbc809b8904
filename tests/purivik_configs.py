"""Tiny Purivik configurations and weights for tests.  The weights are drawn here, larger than a checkpoint's random init,
so that scores differ between keys and experts (with weights of deviation 0.02 every softmax is nearly flat and every
router score is one half: a wrong key, a wrong pick or a score left out would hide in the rounding)."""
import json
import os

import numpy as np
import torch


def layer(heads, kv_heads, dim, vdim, chunk=None, rot=None, scaling=None, mlp=None, scale=None):
    """`rot`: (dims, base); `scaling`: (factor, low, high, original); `mlp`: None, ("dense", ff, limit) or ("moe", ff, experts, top)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
        if scaling is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if mlp is None:
        ff = None
    elif mlp[0] == "dense":
        ff = {"kind": "dense", "ff": mlp[1], "limit": mlp[2]}
    else:
        ff = {"kind": "moe", "expert": {"ff": mlp[1]}, "router": {"experts": mlp[2], "top": mlp[3]}}
    return {"type": "attention", "mixer": mixer, "mlp": ff}


def config(width, vocab, layers, loop=None, eps=1e-5, embedding_scale=3.0, residual_mult=0.6):
    cfg = {"architecture": "Purivik", "width": width, "vocab": vocab, "embedding": {"scale": embedding_scale},
           "residual_mult": residual_mult, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# A: the last two layers looped three times, a layer without feed-forward, two picks of five experts, keys wider than
# values, partial rotary with scaled frequencies (the bands lie inside the frequencies of 16 lanes at base 10,000: some lanes
# are kept, some slowed, some blended)
A = config(64, 96, [layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0), scaling=(4.0, 1.0, 4.0, 64), mlp=("dense", 80, 0.75)),
                    layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0), scaling=(4.0, 1.0, 4.0, 64), mlp=("moe", 24, 5, 2)),
                    layer(4, 2, 32, 16, chunk=24, rot=(16, 10000.0), scaling=(4.0, 1.0, 4.0, 64))], loop=(1, 3, 3))
# B: as many key/value heads as heads, every lane rotated, unscaled frequencies, no loop, chunks that are no multiple of the
# page, one pick of three experts, sums added as they are (residual_mult 1), an embedding that is not scaled, a score scale
# that is not the head size's inverse root
B = config(96, 120, [layer(3, 3, 32, 32, chunk=40, rot=(32, 500.0), mlp=("moe", 40, 3, 1), scale=0.11),
                     layer(3, 3, 32, 32, chunk=40, rot=(32, 500.0), mlp=("dense", 112, 2.0), scale=0.11)], eps=1e-6, embedding_scale=1.0,
           residual_mult=1.0)
# C: one key/value head, head sizes that are no multiple of 8 (keys stored lane by lane), no rotation, no mask (every earlier
# key is seen), a loop of one pass over the last layer, every expert picked (top = experts)
C = config(48, 80, [layer(2, 1, 20, 12, mlp=("moe", 16, 3, 3)), layer(2, 1, 20, 12, mlp=("dense", 64, 3.0))], loop=(1, 2, 1),
           residual_mult=0.9)
# D: layers of different geometry (two cache groups), keys and values of 64 lanes (sizes the matrix-core attention takes)
# beside values half as wide, a loop in the middle, sixteen experts
D = config(128, 160, [layer(8, 2, 64, 64, chunk=80, rot=(32, 25000.0), scaling=(8.0, 1.0, 4.0, 256), mlp=("dense", 192, 1.0)),
                      layer(4, 1, 64, 32, chunk=16, rot=(8, 100.0), mlp=("moe", 48, 16, 2)),
                      layer(8, 2, 64, 64, chunk=80, rot=(32, 25000.0), scaling=(8.0, 1.0, 4.0, 256), mlp=("moe", 48, 16, 4))],
           loop=(1, 3, 2), residual_mult=0.5)
# E: sizes that are multiples of nothing (width, vocabulary, feed-forward, experts), heads of 24 lanes with values of 40
# (wider than the keys), three heads on one key/value head, a chunk of 7 positions, a loop over every layer
E = config(68, 77, [layer(3, 1, 24, 40, chunk=7, rot=(10, 77.0), scaling=(2.5, 0.5, 3.0, 30), mlp=("moe", 18, 7, 2), scale=0.3),
                    layer(3, 1, 24, 40, chunk=7, rot=(10, 77.0), mlp=("dense", 50, 0.9), scale=0.3)], loop=(0, 2, 2), embedding_scale=2.0,
           residual_mult=0.8)
# F: heads wider than any matrix-core kernel takes (keys of 160 lanes, values of 136: the plain attention in both precisions),
# a single expert (always picked, its score still scales its input), the first layer looped
F = config(96, 100, [layer(4, 2, 160, 136, chunk=50, rot=(40, 1000000.0), scaling=(8.0, 1.0, 4.0, 128), mlp=("moe", 32, 1, 1)),
                     layer(4, 2, 160, 136, chunk=50, rot=(40, 1000000.0), scaling=(8.0, 1.0, 4.0, 128), mlp=("dense", 72, 1.5))],
           loop=(0, 1, 2), residual_mult=0.7)
# G: keys of 80 and values of 96 lanes (widened to 128 in bfloat16), chunks of 150 positions (no multiple of a page or of a
# key tile) under requests of several hundred tokens, one pick of six experts
G = config(128, 200, [layer(8, 4, 80, 96, chunk=150, rot=(20, 50000.0), mlp=("moe", 40, 6, 1)),
                      layer(8, 4, 80, 96, chunk=150, rot=(20, 50000.0), mlp=("dense", 160, 1.0))], embedding_scale=6.0, residual_mult=0.7)
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F, "G": G}
PAGE_SIZES = {"A": 8, "B": 16, "C": 8, "D": 16, "E": 16, "F": 16, "G": 16}


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32)


def weights(cfg, seed, decided_router=False):
    """name -> float32 torch tensor whose values are exact in bfloat16 (both precisions load the same numbers).

    `decided_router`: for comparisons in bfloat16, where a random router has close calls (two experts whose scores differ
    by less than the rounding of the stream, one in fifty decisions) and a flipped pick is a large error that says nothing
    about the kernels.  The first two lanes of the stream then carry a direction that depends on the token alone (the layer
    scales are zero there, so no layer changes it, and the norm before a router weighs both lanes alike), every router row
    looks at those two lanes only, row e along the angle 2 pi e / E, and the tokens' angles lie halfway between the angles at
    which two experts tie: every pick has a margin far above the rounding, and tokens differ in their picks and scores."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {"embed": rng.normal(0, 0.4, (cfg["vocab"], W)), "final.norm": 1 + rng.uniform(-0.3, 0.3, W)}
    counts = {spec["mlp"]["router"]["experts"] for spec in cfg["layers"] if spec["mlp"] and spec["mlp"]["kind"] == "moe"}
    if decided_router:
        assert len(counts) == 1, "one number of experts a configuration"
        E = counts.pop()
        angle = (np.arange(cfg["vocab"]) % (2 * E) + 0.5) * np.pi / E
        out["embed"][:, 0], out["embed"][:, 1] = 1.2 * np.cos(angle), 1.2 * np.sin(angle)
    for i, spec in enumerate(cfg["layers"]):
        m = spec["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = f"l{i}."
        for name in ("norm1", "norm1b"):
            out[p + name] = 1 + rng.uniform(-0.3, 0.3, W)
        out[p + "ls1"] = rng.uniform(0.5, 1.5, W)
        if decided_router:
            out[p + "ls1"][:2] = 0.0
        out[p + "mix.q"] = rng.normal(0, 2 * W ** -0.5, (H * d, W))
        out[p + "mix.k"] = rng.normal(0, 2 * W ** -0.5, (G * d, W))
        out[p + "mix.v"] = rng.normal(0, W ** -0.5, (G * dv, W))
        out[p + "mix.o"] = rng.normal(0, (H * dv) ** -0.5, (W, H * dv))
        mlp = spec["mlp"]
        if mlp is None:
            continue
        for name in ("norm2", "norm2b"):
            out[p + name] = 1 + rng.uniform(-0.3, 0.3, W)
        out[p + "ls2"] = rng.uniform(0.5, 1.5, W)
        if decided_router:
            out[p + "ls2"][:2] = 0.0
            out[p + "norm2"][:2] = 1.0
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            out[p + "mlp.gate"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[p + "mlp.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[p + "mlp.down"] = rng.normal(0, ff ** -0.5, (W, ff))
        else:
            ff = mlp["expert"]["ff"]
            out[p + "mlp.router"] = rng.normal(0, 1.5 * W ** -0.5, (mlp["router"]["experts"], W))
            if decided_router:
                at = 2 * np.pi * np.arange(mlp["router"]["experts"]) / mlp["router"]["experts"]
                out[p + "mlp.router"][:] = 0.0
                out[p + "mlp.router"][:, 0], out[p + "mlp.router"][:, 1] = 5.0 * np.cos(at), 5.0 * np.sin(at)
            for e in range(mlp["router"]["experts"]):
                out[f"{p}mlp.e{e}.gate"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
                out[f"{p}mlp.e{e}.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
                out[f"{p}mlp.e{e}.down"] = rng.normal(0, ff ** -0.5, (W, ff))
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
