"""Menitar: the description of the architecture in terms of parts.

x = E[token] * embedding.scale; a layer adds both of its branches, each behind an RMSNorm of its own of the same
stream: x += mixer(norm1 x) + ff(norm2 x).  The mixer is attention with one RMSNorm over the whole query projection
and one over the whole key projection, rotary on the first lanes of every head, scores with a temperature a head that
are mixed across heads before the softmax, keys visible inside the row's own chunk of positions, and a sigmoid gate a
head on the output (`parts/talking_attention.py`).  The feed-forward is gated with clamped operands
(`parts/mlp.py: ClampedGLU`).  The layers loop.start .. loop.stop - 1 run loop.times times in a row with the same
weights and a cache of their own each pass (the run order names them again); before every pass a learned vector of
that pass is added to the stream, and before every pass but the first the embedding of the tokens as well
(`parts/stream.py`).  logits = E rms(x) * logit_scale with the embedding table itself.

Tensor names: `embed`, `loop.step`, `final.norm`, and per layer `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.{q,k,v,o,g,
q.norm,k.norm,talk,temp}`, `l<i>.mlp.{gate,up,down}`.
"""
from __future__ import annotations

from ..config.menitar import MenitarConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import Architecture, register_architecture


def build_spec(cfg: MenitarConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        norm = lambda name: PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": f"{p}.{name}"})
        position = None
        if m.rot_dims:
            position = {"kind": "rotary", "dims": m.rot_dims, "theta": m.rot_base, "pairing": "half", "scaling": "none",
                        "max_position": cfg.max_position}
        mixer = PartSpec(
            "talking_attention",
            {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
             "value_head_dim": m.vdim, "scale": m.scale, "chunk": m.chunk, "qk_norm_eps": cfg.eps, "position": position},
            {"q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "o": f"{p}.mix.o", "gate": f"{p}.mix.g",
             "q_norm": f"{p}.mix.q.norm", "k_norm": f"{p}.mix.k.norm", "talk": f"{p}.mix.talk", "temp": f"{p}.mix.temp"},
        )
        ffn = None
        norms = {"mixer": norm("norm1")}
        if layer.mlp is not None:
            ffn = PartSpec("clamped_glu",
                           {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "limit": layer.mlp.limit,
                            "alpha": 1.702, "up_offset": 1.0},
                           {"gate": f"{p}.mlp.gate", "up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
            norms["feed_forward"] = norm("norm2")
        layers.append(LayerSpec(block=PartSpec("parallel"), mixer=mixer, feed_forward=ffn, norms=norms))
    ignorable = [f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.mlp is None]
    n = len(cfg.layers)
    if cfg.loop is None:
        order = [RunEntry(layer=i) for i in range(n)]
        ignorable.append("loop.step")
    else:
        start, stop, times = cfg.loop
        order = [RunEntry(layer=i) for i in range(start)]
        for t in range(times):
            enter = PartSpec("pass_input", {"row": t, "rows": times, "size": cfg.width, "add_embedding": t > 0},
                             {"steps": "loop.step"})
            order += [RunEntry(layer=i, before=enter if i == start else None) for i in range(start, stop)]
        order += [RunEntry(layer=i) for i in range(stop, n)]
    table = {"weight": "embed"}
    return ModelSpec(
        architecture="menitar",
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_position,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": cfg.embedding_scale}, table),
        layers=tuple(layers),
        run_order=tuple(order),
        final_norm=PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": cfg.logit_scale}, table),
        ignorable_tensors=tuple(ignorable),
    )


register_architecture(Architecture(
    model_type="menitar",
    hf_architectures=(),
    parse_config=MenitarConfig.from_dict,
    build_spec=build_spec,
))
