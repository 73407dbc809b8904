"""Typed configuration of the Purivik architecture, read from a checkpoint's config.json.

The file names the design under `architecture`; sizes and constants are nested by what they belong to: `width`, `vocab`,
`embedding.scale`, `norm.eps`, `residual_mult`, `loop` (start, stop, times; absent: no layer runs twice) and `layers`, a
list whose entries give the mixer's `type`, its sizes under `mixer` (heads, kv_heads, dim, vdim, scale, `rot` {base, dims,
`scaling` {factor, low, high, original}}, `mask` {size}) and the feed-forward under `mlp`: null for none, `kind` "dense"
with ff and limit, or `kind` "moe" with `expert.ff` and `router` {experts, top}.  Everything is checked here, before any
weight is read.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .menitar import DEFAULT_MAX_POSITION, _need, _positive
from .spec import ConfigError


@dataclass(frozen=True)
class FrequencyScaling:
    """Rotary frequencies divided by `factor` where the wavelength is longer than original / low, kept where it is shorter
    than original / high, and a straight line between the two in original / wavelength."""
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class PurivikMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int                  # 0: no rotation
    rot_base: float
    rot_scaling: Optional[FrequencyScaling]
    chunk: Optional[int]           # positions see their own chunk of this many positions; None: all before them


@dataclass(frozen=True)
class PurivikMLP:
    kind: str                      # "dense" or "moe"
    ff: int                        # lanes of the dense layer, or of one expert
    limit: float = 0.0             # dense: what gate and up are clamped to
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class PurivikLayer:
    mixer: PurivikMixer
    mlp: Optional[PurivikMLP]


@dataclass(frozen=True)
class PurivikConfig:
    width: int
    vocab: int
    embedding_scale: float
    residual_mult: float
    eps: float
    layers: Tuple[PurivikLayer, ...]
    loop: Optional[Tuple[int, int, int]]      # (start, stop, times)
    max_position: int

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @staticmethod
    def from_dict(cfg: Dict[str, Any]) -> "PurivikConfig":
        width = _positive(cfg, "width", "")
        vocab = _positive(cfg, "vocab", "")
        eps = _need(_need(cfg, "norm", dict, ""), "eps", float, "norm.")
        if not eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, is {eps}")
        raw_layers = _need(cfg, "layers", list, "")
        if not raw_layers:
            raise ConfigError("layers must list at least one layer")
        layers = tuple(_layer(raw, f"layers[{i}].") for i, raw in enumerate(raw_layers))
        loop = None
        if cfg.get("loop") is not None:
            raw = cfg["loop"]
            start, stop, times = _need(raw, "start", int, "loop."), _need(raw, "stop", int, "loop."), _positive(raw, "times", "loop.")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop.start {start} and loop.stop {stop} must name a run of the {len(layers)} layers")
            loop = (start, stop, times)
        max_position = cfg.get("max_position", DEFAULT_MAX_POSITION)
        if isinstance(max_position, bool) or not isinstance(max_position, int) or max_position <= 0:
            raise ConfigError(f"max_position must be a positive integer, is {max_position!r}")
        return PurivikConfig(width, vocab, _need(_need(cfg, "embedding", dict, ""), "scale", float, "embedding."),
                             _need(cfg, "residual_mult", float, ""), eps, layers, loop, max_position)


def _layer(raw, where: str) -> PurivikLayer:
    kind = _need(raw, "type", str, where)
    if kind != "attention":
        raise ConfigError(f"{where}type {kind!r} is no mixer of this design (known: 'attention')")
    m = _need(raw, "mixer", dict, where)
    mw = where + "mixer."
    heads, kv_heads = _positive(m, "heads", mw), _positive(m, "kv_heads", mw)
    if heads % kv_heads != 0:
        raise ConfigError(f"{mw}heads {heads} is not a multiple of kv_heads {kv_heads}")
    dim, vdim = _positive(m, "dim", mw), _positive(m, "vdim", mw)
    rot = m.get("rot")
    rot_dims, rot_base, rot_scaling = 0, 1.0, None
    if rot is not None:
        rw = mw + "rot."
        rot_dims, rot_base = _need(rot, "dims", int, rw), _need(rot, "base", float, rw)
        if rot_dims < 0 or rot_dims % 2 != 0 or rot_dims > dim:
            raise ConfigError(f"{rw}dims must be even and at most dim {dim}, is {rot_dims}")
        if rot_dims and not rot_base > 0.0:
            raise ConfigError(f"{rw}base must be positive, is {rot_base}")
        if rot.get("scaling") is not None:
            sw = rw + "scaling."
            sc = rot["scaling"]
            rot_scaling = FrequencyScaling(_need(sc, "factor", float, sw), _need(sc, "low", float, sw),
                                           _need(sc, "high", float, sw), _need(sc, "original", float, sw))
            if not (rot_scaling.factor > 0.0 and rot_scaling.original > 0.0 and 0.0 < rot_scaling.low < rot_scaling.high):
                raise ConfigError(f"{sw}factor and original must be positive and 0 < low < high, is {sc!r}")
    mask = m.get("mask")
    chunk = None if mask is None else _positive(mask, "size", mw + "mask.")
    mixer = PurivikMixer(heads, kv_heads, dim, vdim, _need(m, "scale", float, mw), rot_dims, rot_base, rot_scaling, chunk)
    raw_mlp = raw.get("mlp")
    mlp = None
    if raw_mlp is not None:
        pw = where + "mlp."
        mlp_kind = _need(raw_mlp, "kind", str, pw)
        if mlp_kind == "dense":
            limit = _need(raw_mlp, "limit", float, pw)
            if not limit > 0.0:
                raise ConfigError(f"{pw}limit must be positive, is {limit}")
            mlp = PurivikMLP("dense", _positive(raw_mlp, "ff", pw), limit=limit)
        elif mlp_kind == "moe":
            router = _need(raw_mlp, "router", dict, pw)
            experts, top = _positive(router, "experts", pw + "router."), _positive(router, "top", pw + "router.")
            if top > experts:
                raise ConfigError(f"{pw}router.top {top} is more than router.experts {experts}")
            mlp = PurivikMLP("moe", _positive(_need(raw_mlp, "expert", dict, pw), "ff", pw + "expert."), experts=experts, top=top)
        else:
            raise ConfigError(f"{pw}kind {mlp_kind!r} is no feed-forward of this design (known: 'dense', 'moe')")
    return PurivikLayer(mixer, mlp)
