"""Typed configuration of the Fuvirax design, read from the keys of its ``config.json``.

Top level: ``vocab``, ``width``, ``streams``, ``logit_scale``, ``norm.eps``, ``layers`` (a list of
``{type, mixer, mlp}``) and ``loop`` (``start``, ``stop``, ``times``: layers start .. stop-1 run that many times
in a row, each pass with a cache of its own).  Every size is a required key; what a mixer type needs is checked
by type.  Two sizes are not in config.json but in tensor shapes (the inner widths of the delta mixer's two
low-rank projections); for a fresh random checkpoint they may be given as ``decay_rank`` and ``gate_rank``."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError

MIXER_KEYS = {
    "latent_attention": dict(dim=int, heads=int, kv_rank=int, rot_dim=int, vdim=int, scale=float),
    "hgrn2": dict(dim=int, heads=int, vdim=int),
    "channel_delta": dict(conv=int, dim=int, heads=int, kv_heads=int, vdim=int),
}
DEFAULT_LOW_RANK = 16
MAX_POSITIONS = 1 << 20     # the design has no limit of its own; the cache's size decides


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
class MixerConfig:
    type: str
    sizes: dict          # the integer and float keys of MIXER_KEYS[type]
    rot_base: float = 0.0
    rot_dims: int = 0
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None

    def __getattr__(self, key):
        try:
            return self.__dict__["sizes"][key]
        except KeyError:
            raise AttributeError(key) from None


@dataclass(frozen=True)
class LayerConfig:
    mixer: MixerConfig
    ff: Optional[int]     # inner width of the dense feed-forward, None: the layer has none


@dataclass(frozen=True)
class FuviraxConfig:
    vocab: int
    width: int
    streams: int
    logit_scale: float
    eps: float
    layers: Tuple[LayerConfig, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def max_positions(self):
        return MAX_POSITIONS

    def order(self):
        """Indices of the layers in the order they run."""
        n = len(self.layers)
        body = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + body * self.loop_times + list(range(self.loop_stop, n))

    @classmethod
    def from_dict(cls, d: dict) -> "FuviraxConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        out = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {', '.join(sorted(MIXER_KEYS))}")
            m = entry.get("mixer")
            sizes = {k: _get(m, k, t, where + ".mixer") for k, t in MIXER_KEYS[kind].items()}
            extra = {}
            if kind == "latent_attention":
                rot = m.get("rot")
                extra = dict(rot_base=_get(rot, "base", float, where + ".mixer.rot"),
                             rot_dims=_get(rot, "dims", int, where + ".mixer.rot"))
                if extra["rot_dims"] % 2 or extra["rot_dims"] > sizes["rot_dim"]:
                    raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even and at most rot_dim")
            if kind == "channel_delta":
                if sizes["heads"] % sizes["kv_heads"]:
                    raise ConfigError(f"config.json: {where}.mixer.heads must be a multiple of kv_heads")
                extra = {k: _get(m, k, int, where + ".mixer") for k in ("decay_rank", "gate_rank") if m.get(k) is not None}
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; known: dense")
                ff = _get(mlp, "ff", int, where + ".mlp")
            out.append(LayerConfig(MixerConfig(kind, sizes, **extra), ff))
        loop = d.get("loop")
        ls = dict(loop_start=0, loop_stop=0, loop_times=1)
        if loop is not None:
            for k in ("start", "stop", "times"):
                v = loop.get(k) if isinstance(loop, dict) else None
                if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                    raise ConfigError(f"config.json: loop.{k} must be a non-negative integer, got {v!r}")
            ls = dict(loop_start=loop["start"], loop_stop=loop["stop"], loop_times=loop["times"])
            if not ls["loop_start"] <= ls["loop_stop"] <= len(out) or ls["loop_times"] < 1:
                raise ConfigError("config.json: loop must name a range of the layers and run it at least once")
        streams = _get(d, "streams", int, "the top level")
        if streams > 16:
            raise ConfigError(f"config.json: {streams} streams; at most 16 are supported")
        return cls(vocab=_get(d, "vocab", int, "the top level"), width=_get(d, "width", int, "the top level"),
                   streams=streams, logit_scale=_get(d, "logit_scale", float, "the top level"),
                   eps=_get(d.get("norm"), "eps", float, "norm"), layers=tuple(out), **ls)
