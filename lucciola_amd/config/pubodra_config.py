"""Typed configuration of the Pubodra decoder, read from the keys of its config.json.

The file lists the layers one by one (``layers``: each with the ``type`` of its mixer, the
mixer's sizes under ``mixer`` and its feed-forward under ``mlp``, which may be null), the
model's ``width`` and ``vocab``, the norms' ``eps`` under ``norm`` and, optionally, a ``loop``:
the layers ``start`` .. ``stop - 1`` run ``times`` times in a row with the same weights.  Every
size and constant is a field read from the file; nothing is assumed equal between layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError, read_config_json

ARCHITECTURE = "Pubodra"


def _get(data: Dict[str, Any], key: str, where: str):
    if not isinstance(data, dict) or key not in data or data[key] is None:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return data[key]


def _int(data, key, where, least=1) -> int:
    value = _get(data, key, where)
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json: {where}.{key} must be an integer, got {value!r}")
    if value < least:
        raise ConfigError(f"config.json: {where}.{key} must be at least {least}, got {value}")
    return value


@dataclass(frozen=True)
class YarnScaling:
    """How the rotary frequencies are stretched: a frequency whose wavelength is long against
    the ``original`` context is divided by ``factor``, one that turns more than ``fast`` times in
    it is kept, those between ``slow`` and ``fast`` turns are blended."""

    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self) -> Dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[YarnScaling] = None


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # unrotated query/key entries of a head
    rot_dim: int        # rotated query/key entries of a head; the key's are shared by all heads
    vdim: int
    kv_rank: int        # size of the cached latent
    scale: float
    rot: Optional[RotaryConfig]
    window: Optional[int]


@dataclass(frozen=True)
class MlpConfig:
    kind: str           # "dense" or "moe"
    ff: int             # inner size (of one expert, for "moe")
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: LatentAttentionConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class PubodraConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[LayerConfig, ...]
    loop: Optional[LoopConfig] = None
    initializer_range: float = 0.02
    eos_token_ids: Tuple[int, ...] = ()
    raw: Optional[Dict[str, Any]] = None    # the dict it was read from, for writing it out again

    @staticmethod
    def from_dict(data: Dict[str, Any]) -> "PubodraConfig":
        layers = _get(data, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(_read_layer(entry, i) for i, entry in enumerate(layers))
        loop = data.get("loop")
        loop_cfg = None
        if loop:
            loop_cfg = LoopConfig(_int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0),
                                  _int(loop, "times", "loop", 1))
            if not 0 <= loop_cfg.start < loop_cfg.stop <= len(parsed):
                raise ConfigError(f"config.json: loop {loop_cfg.start}..{loop_cfg.stop} does not lie "
                                  f"inside the {len(parsed)} layers")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        eps = float(_get(_get(data, "norm", "the model"), "eps", "norm"))
        if not eps > 0:
            raise ConfigError("config.json: norm.eps must be positive")
        return PubodraConfig(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                             norm_eps=eps, layers=parsed, loop=loop_cfg,
                             initializer_range=float(data.get("initializer_range", 0.02)),
                             eos_token_ids=eos_ids, raw=dict(data))

    @staticmethod
    def from_folder(folder: str) -> "PubodraConfig":
        return PubodraConfig.from_dict(read_config_json(folder))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw) if self.raw is not None else {}


def _read_layer(entry: Dict[str, Any], i: int) -> LayerConfig:
    where = f"layers[{i}]"
    kind = str(_get(entry, "type", where))
    if kind != "latent_attention":
        raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design "
                          f"(latent_attention)")
    m = _get(entry, "mixer", where)
    mw = where + ".mixer"
    rot = m.get("rot")
    rot_dim = _int(m, "rot_dim", mw, 0)
    rot_cfg = None
    if rot and rot_dim:
        scaling = rot.get("scaling")
        yarn = None
        if scaling:
            yarn = YarnScaling(float(_get(scaling, "factor", mw + ".rot.scaling")),
                               float(_get(scaling, "original", mw + ".rot.scaling")),
                               float(_get(scaling, "fast", mw + ".rot.scaling")),
                               float(_get(scaling, "slow", mw + ".rot.scaling")))
            if yarn.factor <= 0 or yarn.original <= 0 or yarn.fast <= 0 or yarn.slow <= 0:
                raise ConfigError(f"config.json: {mw}.rot.scaling needs positive numbers")
        rot_cfg = RotaryConfig(float(_get(rot, "base", mw + ".rot")), _int(rot, "dims", mw + ".rot", 2), yarn)
        if rot_cfg.dims % 2 or rot_cfg.dims > rot_dim:
            raise ConfigError(f"config.json: {mw}.rot.dims ({rot_cfg.dims}) must be even and at most "
                              f"rot_dim ({rot_dim})")
        if not rot_cfg.base > 1:
            raise ConfigError(f"config.json: {mw}.rot.base must be above 1")
    mask = m.get("mask")
    window = None
    if mask and mask.get("size") is not None:
        window = _int(mask, "size", mw + ".mask")
    mixer = LatentAttentionConfig(heads=_int(m, "heads", mw), dim=_int(m, "dim", mw, 0), rot_dim=rot_dim,
                                  vdim=_int(m, "vdim", mw), kv_rank=_int(m, "kv_rank", mw),
                                  scale=float(_get(m, "scale", mw)), rot=rot_cfg, window=window)
    if mixer.dim + mixer.rot_dim <= 0:
        raise ConfigError(f"config.json: {mw}: a head needs query/key entries (dim + rot_dim > 0)")
    mlp = entry.get("mlp")
    mlp_cfg = None
    if mlp:
        lw = where + ".mlp"
        mkind = str(_get(mlp, "kind", lw))
        if mkind == "dense":
            mlp_cfg = MlpConfig("dense", _int(mlp, "ff", lw))
        elif mkind == "moe":
            router = _get(mlp, "router", lw)
            mlp_cfg = MlpConfig("moe", _int(_get(mlp, "expert", lw), "ff", lw + ".expert"),
                                _int(router, "experts", lw + ".router"), _int(router, "top", lw + ".router"))
            if mlp_cfg.top > mlp_cfg.experts:
                raise ConfigError(f"config.json: {lw}.router.top ({mlp_cfg.top}) exceeds its "
                                  f"{mlp_cfg.experts} experts")
        else:
            raise ConfigError(f"config.json: {lw}.kind '{mkind}' is neither 'dense' nor 'moe'")
    return LayerConfig(kind, mixer, mlp_cfg)
