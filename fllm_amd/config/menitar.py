"""Typed configuration of the Menitar architecture, read from a checkpoint's config.json.

The file names the design under `architecture`; sizes and constants are nested by what they belong to:
`width`, `vocab`, `embedding.scale`, `logit_scale`, `norm.eps`, `loop` (start, stop, times; absent: no layer runs
twice) and `layers`, a list whose entries give the mixer's `type`, its sizes under `mixer` (heads, kv_heads, dim,
vdim, scale, `rot` {base, dims}, `mask` {size}) and the feed-forward under `mlp` (kind, ff, limit; null: none).
Everything is checked here, before any weight is read.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .spec import ConfigError

DEFAULT_MAX_POSITION = 131072      # the file names no context length: rotary positions are not bounded by the design


def _need(d: Dict[str, Any], key: str, kind, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json requires {where}{key}")
    v = d[key]
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}{key} must be a number, is {v!r}")
        return float(v)
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}{key} must be an integer, is {v!r}")
        return v
    if not isinstance(v, kind):
        raise ConfigError(f"{where}{key} must be {kind.__name__}, is {v!r}")
    return v


def _positive(d, key, where) -> int:
    v = _need(d, key, int, where)
    if v <= 0:
        raise ConfigError(f"{where}{key} must be positive, is {v}")
    return v


@dataclass(frozen=True)
class MenitarMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int                  # 0: no rotation
    rot_base: float
    chunk: Optional[int]           # positions see their own chunk of this many positions; None: all before them


@dataclass(frozen=True)
class MenitarMLP:
    ff: int
    limit: float


@dataclass(frozen=True)
class MenitarLayer:
    mixer: MenitarMixer
    mlp: Optional[MenitarMLP]


@dataclass(frozen=True)
class MenitarConfig:
    width: int
    vocab: int
    embedding_scale: float
    logit_scale: float
    eps: float
    layers: Tuple[MenitarLayer, ...]
    loop: Optional[Tuple[int, int, int]]      # (start, stop, times)
    max_position: int

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @staticmethod
    def from_dict(cfg: Dict[str, Any]) -> "MenitarConfig":
        width = _positive(cfg, "width", "")
        vocab = _positive(cfg, "vocab", "")
        eps = _need(_need(cfg, "norm", dict, ""), "eps", float, "norm.")
        if not eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, is {eps}")
        raw_layers = _need(cfg, "layers", list, "")
        if not raw_layers:
            raise ConfigError("layers must list at least one layer")
        layers = []
        for i, raw in enumerate(raw_layers):
            where = f"layers[{i}]."
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
            rot_dims, rot_base = 0, 1.0
            if rot is not None:
                rot_dims, rot_base = _need(rot, "dims", int, mw + "rot."), _need(rot, "base", float, mw + "rot.")
                if rot_dims < 0 or rot_dims % 2 != 0 or rot_dims > dim:
                    raise ConfigError(f"{mw}rot.dims must be even and at most dim {dim}, is {rot_dims}")
                if rot_dims and not rot_base > 0.0:
                    raise ConfigError(f"{mw}rot.base must be positive, is {rot_base}")
            mask = m.get("mask")
            chunk = None if mask is None else _positive(mask, "size", mw + "mask.")
            mixer = MenitarMixer(heads, kv_heads, dim, vdim, _need(m, "scale", float, mw), rot_dims, rot_base, chunk)
            raw_mlp = raw.get("mlp")
            mlp = None
            if raw_mlp is not None:
                pw = where + "mlp."
                mlp_kind = _need(raw_mlp, "kind", str, pw)
                if mlp_kind != "dense":
                    raise ConfigError(f"{pw}kind {mlp_kind!r} is no feed-forward of this design (known: 'dense')")
                limit = _need(raw_mlp, "limit", float, pw)
                if not limit > 0.0:
                    raise ConfigError(f"{pw}limit must be positive, is {limit}")
                mlp = MenitarMLP(_positive(raw_mlp, "ff", pw), limit)
            layers.append(MenitarLayer(mixer, mlp))
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
        return MenitarConfig(width, vocab, _need(_need(cfg, "embedding", dict, ""), "scale", float, "embedding."),
                             _need(cfg, "logit_scale", float, ""), eps, tuple(layers), loop, max_position)
