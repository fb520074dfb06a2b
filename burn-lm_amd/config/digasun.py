"""Typed configuration of the Digasun design, read from the keys of its ``config.json``.

Top level: ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``, ``canon.taps`` (taps of the convolution in front
of the sublayers), ``token_side.dim`` (columns per layer of the side table) and ``layers``: a list of
``{type, mixer, mlp}`` with ``type`` one of ``attention`` and ``gla``, ``mixer`` that type's sizes and constants,
and ``mlp`` ``null`` (none), ``{kind: dense, ff, limit}`` or ``{kind: moe, router: {experts, top}, expert: {ff},
shared: {ff}}`` (``shared`` may be missing).  An attention layer with ``kv_from: j`` has no key and value
projections and reads layer j's.  Every size is a required key.  One size is in a tensor's shape only (the inner
width of the decay projections of a ``gla`` mixer); for a fresh random checkpoint it may be given as ``decay_rank``."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError

MAX_POSITIONS = 1 << 20     # the design has no limit of its own; the cache's size decides
DEFAULT_DECAY_RANK = 16


def _get(d, key, kind, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing in {where}")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
            raise ConfigError(f"config.json: '{key}' in {where} must be a positive integer, got {v!r}")
        return v
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' in {where} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int           # 0: every earlier key
    rot_dims: int         # 0: no rotation
    rot_base: float
    kv_from: Optional[int]
    type: str = "attention"


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int]
    type: str = "gla"


@dataclass(frozen=True)
class DenseConfig:
    ff: int
    limit: float
    kind: str = "dense"


@dataclass(frozen=True)
class MoeConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int        # 0: no shared expert
    kind: str = "moe"


@dataclass(frozen=True)
class LayerConfig:
    mixer: object
    mlp: object           # DenseConfig, MoeConfig or None


@dataclass(frozen=True)
class DigasunConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    taps: int
    side_dim: int
    layers: Tuple[LayerConfig, ...]

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def max_positions(self):
        return MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "DigasunConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        out = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            m = entry.get("mixer") if isinstance(entry, dict) else None
            mw = where + ".mixer"
            if kind == "attention":
                heads, kv_heads = _get(m, "heads", int, mw), _get(m, "kv_heads", int, mw)
                if heads % kv_heads:
                    raise ConfigError(f"config.json: {mw}.heads must be a multiple of kv_heads")
                dim = _get(m, "dim", int, mw)
                rot = m.get("rot")
                rot_dims = _get(rot, "dims", int, mw + ".rot") if rot is not None else 0
                if rot_dims % 2 or rot_dims > dim:
                    raise ConfigError(f"config.json: {mw}.rot.dims must be even and at most dim")
                kv_from = m.get("kv_from")
                if kv_from is not None:
                    src = out[kv_from].mixer if isinstance(kv_from, int) and not isinstance(kv_from, bool) and 0 <= kv_from < i else None
                    if src is None or src.type != "attention" or src.kv_from is not None:
                        raise ConfigError(f"config.json: {mw}.kv_from must name an earlier attention layer with "
                                          f"key and value projections of its own, got {kv_from!r}")
                mixer = AttentionConfig(heads=heads, kv_heads=kv_heads, dim=dim, vdim=_get(m, "vdim", int, mw),
                                        scale=_get(m, "scale", float, mw),
                                        window=_get(m["mask"], "size", int, mw + ".mask") if m.get("mask") is not None else 0,
                                        rot_dims=rot_dims,
                                        rot_base=_get(rot, "base", float, mw + ".rot") if rot is not None else 0.0,
                                        kv_from=kv_from)
                if kv_from is not None:
                    src = out[kv_from].mixer
                    if (src.kv_heads, src.dim, src.vdim) != (kv_heads, dim, mixer.vdim):
                        raise ConfigError(f"config.json: {mw} reads the keys and values of layer {kv_from}, whose "
                                          f"key-value head count or head sizes differ")
            elif kind == "gla":
                rank = m.get("decay_rank") if isinstance(m, dict) else None
                mixer = GlaConfig(heads=_get(m, "heads", int, mw), dim=_get(m, "dim", int, mw), vdim=_get(m, "vdim", int, mw),
                                  tau=_get(m, "tau", float, mw),
                                  decay_rank=_get(m, "decay_rank", int, mw) if rank is not None else None)
                if mixer.tau <= 0:
                    raise ConfigError(f"config.json: {mw}.tau must be positive")
            else:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: attention, gla")
            mlp = entry.get("mlp")
            lw = where + ".mlp"
            if mlp is None:
                ff = None
            elif mlp.get("kind") == "dense":
                ff = DenseConfig(ff=_get(mlp, "ff", int, lw), limit=_get(mlp, "limit", float, lw))
                if ff.limit <= 0:
                    raise ConfigError(f"config.json: {lw}.limit must be positive")
            elif mlp.get("kind") == "moe":
                router = mlp.get("router")
                ff = MoeConfig(experts=_get(router, "experts", int, lw + ".router"), top=_get(router, "top", int, lw + ".router"),
                               ff=_get(mlp.get("expert"), "ff", int, lw + ".expert"),
                               shared_ff=_get(mlp["shared"], "ff", int, lw + ".shared") if mlp.get("shared") is not None else 0)
                if ff.top > ff.experts:
                    raise ConfigError(f"config.json: {lw}.router.top is larger than the number of experts")
            else:
                raise ConfigError(f"config.json: {lw}.kind is {mlp.get('kind')!r}; known: dense, moe")
            out.append(LayerConfig(mixer, ff))
        top = "the top level"
        return cls(vocab=_get(d, "vocab", int, top), width=_get(d, "width", int, top),
                   embedding_scale=_get(d.get("embedding"), "scale", float, "embedding"),
                   eps=_get(d.get("norm"), "eps", float, "norm"), taps=_get(d.get("canon"), "taps", int, "canon"),
                   side_dim=_get(d.get("token_side"), "dim", int, "token_side"), layers=tuple(out))
