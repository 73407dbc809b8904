"""Purivik: the description of the architecture in terms of parts.

x = E[token] * embedding.scale.  A layer norms each part's input AND its output, scales the output lane by lane with a
learned vector and adds it times a constant: x += m * s1 * rms_1b(mixer(rms_1(x))), then x += m * s2 * rms_2b(ff(rms_2(x)))
(`parts/block.py: SandwichBlock`).  The mixer is grouped-query attention with values of a width of their own, rotary on
the first lanes of every head (lane i paired with lane i + dims / 2; frequencies scaled by wavelength bands, the "llama3"
rule of `parts/rope.py`), a score scale from the file, and keys visible inside the row's own chunk of positions
(`parts/attention.py`).  The feed-forward is either dense and gated with clamped operands (`parts/mlp.py: ClampedGLU`) or
a set of small SwiGLU experts of which a token uses its `top` best by sigmoid score, the score multiplying the expert's
input (`parts/experts.py`).  The layers loop.start .. loop.stop - 1 run loop.times times in a row with the same weights
and a cache of their own each pass (the run order names them again); before every pass but the first the embedding of
the tokens is added to the stream (`parts/stream.py`).  logits = E rms(x) with the embedding table itself.

Tensor names: `embed`, `final.norm`, and per layer `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`, `l<i>.norm2b`, `l<i>.ls1`,
`l<i>.ls2`, `l<i>.mix.{q,k,v,o}`, and `l<i>.mlp.{gate,up,down}` or `l<i>.mlp.router` with `l<i>.mlp.e<j>.{gate,up,down}`.
"""
from __future__ import annotations

from ..config.purivik import PurivikConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import Architecture, register_architecture


def build_spec(cfg: PurivikConfig) -> ModelSpec:
    layers = []
    ignorable = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        norm = lambda name: PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": f"{p}.{name}"})
        position = None
        if m.rot_dims:
            position = {"kind": "rotary", "dims": m.rot_dims, "theta": m.rot_base, "pairing": "half", "scaling": "none",
                        "max_position": cfg.max_position}
            if m.rot_scaling is not None:
                s = m.rot_scaling
                position.update(scaling="llama3", factor=s.factor, low_freq_factor=s.low, high_freq_factor=s.high,
                                original_max_position=s.original)
        mixer = PartSpec(
            "attention",
            {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
             "value_head_dim": m.vdim, "scale": m.scale, "chunk": m.chunk, "position": position, "widen_heads": True},
            {"q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "o": f"{p}.mix.o"},
        )
        ffn = None
        norms = {"mixer": norm("norm1"), "mixer_out": norm("norm1b")}
        scales = {"mixer_scale": f"{p}.ls1"}
        if layer.mlp is None:
            ignorable += [f"{p}.norm2", f"{p}.norm2b", f"{p}.ls2"]
        else:
            norms.update(feed_forward=norm("norm2"), feed_forward_out=norm("norm2b"))
            scales["feed_forward_scale"] = f"{p}.ls2"
            if layer.mlp.kind == "dense":
                ffn = PartSpec("clamped_glu",
                               {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "limit": layer.mlp.limit,
                                "alpha": 1.702, "up_offset": 1.0},
                               {"gate": f"{p}.mlp.gate", "up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
            else:
                names = {"router": f"{p}.mlp.router"}
                for e in range(layer.mlp.experts):
                    names.update({f"gate_{e}": f"{p}.mlp.e{e}.gate", f"up_{e}": f"{p}.mlp.e{e}.up", f"down_{e}": f"{p}.mlp.e{e}.down"})
                ffn = PartSpec("routed_experts",
                               {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "experts": layer.mlp.experts,
                                "top": layer.mlp.top, "score": "sigmoid"}, names)
        block = PartSpec("sandwich", {"size": cfg.width, "residual_mult": cfg.residual_mult}, scales)
        layers.append(LayerSpec(block=block, mixer=mixer, feed_forward=ffn, norms=norms))
    n = len(cfg.layers)
    if cfg.loop is None:
        order = [RunEntry(layer=i) for i in range(n)]
    else:
        start, stop, times = cfg.loop
        order = [RunEntry(layer=i) for i in range(start)]
        for t in range(times):
            # every pass but the first begins with the embedding of the tokens added to the stream
            enter = PartSpec("pass_input", {"size": cfg.width, "add_embedding": True}) if t > 0 else None
            order += [RunEntry(layer=i, before=enter if i == start else None) for i in range(start, stop)]
        order += [RunEntry(layer=i) for i in range(stop, n)]
    table = {"weight": "embed"}
    return ModelSpec(
        architecture="purivik",
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_position,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": cfg.embedding_scale}, table),
        layers=tuple(layers),
        run_order=tuple(order),
        final_norm=PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}, table),
        ignorable_tensors=tuple(ignorable),
    )


register_architecture(Architecture(
    model_type="purivik",
    hf_architectures=(),
    parse_config=PurivikConfig.from_dict,
    build_spec=build_spec,
))
