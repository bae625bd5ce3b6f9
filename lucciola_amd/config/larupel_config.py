"""Typed configuration of the Larupel decoder, read from the keys of its config.json.

The file lists the layers one by one (``layers``: each with the ``type`` of its mixer, the
mixer's sizes under ``mixer`` and its feed-forward under ``mlp``, which may be null), the
model's ``width`` and ``vocab`` and the norms' ``eps`` under ``norm``.  A layer's mixer is one of
``attention`` (softmax attention over cached keys and values; ``kv_from`` names an earlier
attention layer whose keys and values it reads instead of making its own), ``delta`` (the gated
delta rule behind short convolutions) and ``general_delta`` (the generalized delta rule with a
decay and a removal rate per key channel).  Every size and constant is a field read from the
file; nothing is assumed equal between layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError, read_config_json

ARCHITECTURE = "Larupel"
MIXER_TYPES = ("attention", "delta", "general_delta")


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
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int                # query/key entries of a head
    vdim: int               # value entries of a head
    scale: float
    kv_from: Optional[int]  # the layer whose keys and values this one reads; None: its own


@dataclass(frozen=True)
class DeltaConfig:
    """The gated delta rule: ``kv_heads`` query/key heads of ``dim`` serve ``heads`` value heads
    of ``vdim``; ``conv`` taps of the short convolutions."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class GeneralDeltaConfig:
    heads: int
    dim: int


@dataclass(frozen=True)
class SharedExpertConfig:
    ff: int


@dataclass(frozen=True)
class MlpConfig:
    kind: str           # "dense" or "moe"
    ff: int             # inner size (of one expert, for "moe")
    experts: int = 0
    top: int = 0
    shared: Optional[SharedExpertConfig] = None


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any          # AttentionConfig, DeltaConfig or GeneralDeltaConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class LarupelConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[LayerConfig, ...]
    initializer_range: float = 0.02
    eos_token_ids: Tuple[int, ...] = ()
    raw: Optional[Dict[str, Any]] = None    # the dict it was read from, for writing it out again

    @staticmethod
    def from_dict(data: Dict[str, Any]) -> "LarupelConfig":
        layers = _get(data, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(_read_layer(entry, i) for i, entry in enumerate(layers))
        for i, layer in enumerate(parsed):
            _check_kv_from(parsed, i)
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        eps = float(_get(_get(data, "norm", "the model"), "eps", "norm"))
        if not eps > 0:
            raise ConfigError("config.json: norm.eps must be positive")
        return LarupelConfig(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                             norm_eps=eps, layers=parsed,
                             initializer_range=float(data.get("initializer_range", 0.02)),
                             eos_token_ids=eos_ids, raw=dict(data))

    @staticmethod
    def from_folder(folder: str) -> "LarupelConfig":
        return LarupelConfig.from_dict(read_config_json(folder))

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw) if self.raw is not None else {}


def _check_kv_from(layers: Tuple[LayerConfig, ...], i: int) -> None:
    m = layers[i].mixer
    if not isinstance(m, AttentionConfig) or m.kv_from is None:
        return
    where = f"layers[{i}].mixer.kv_from"
    if not 0 <= m.kv_from < i:
        raise ConfigError(f"config.json: {where} = {m.kv_from} must name an earlier layer")
    other = layers[m.kv_from].mixer
    if not isinstance(other, AttentionConfig) or other.kv_from is not None:
        raise ConfigError(f"config.json: {where} = {m.kv_from} must name an attention layer with keys "
                          f"and values of its own")
    if (other.kv_heads, other.dim, other.vdim) != (m.kv_heads, m.dim, m.vdim):
        raise ConfigError(f"config.json: {where}: layer {m.kv_from} keeps {other.kv_heads} heads of "
                          f"{other.dim}/{other.vdim}, this layer reads {m.kv_heads} of {m.dim}/{m.vdim}")


def _read_mixer(kind: str, m: Dict[str, Any], mw: str):
    if kind == "attention":
        heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {mw}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        kv_from = m.get("kv_from")
        if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int)):
            raise ConfigError(f"config.json: {mw}.kv_from must be a layer's number, got {kv_from!r}")
        return AttentionConfig(heads, kv_heads, _int(m, "dim", mw), _int(m, "vdim", mw),
                               float(_get(m, "scale", mw)), kv_from)
    if kind == "delta":
        heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {mw}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        return DeltaConfig(heads, kv_heads, _int(m, "dim", mw), _int(m, "vdim", mw), _int(m, "conv", mw))
    return GeneralDeltaConfig(_int(m, "heads", mw), _int(m, "dim", mw))


def _read_layer(entry: Dict[str, Any], i: int) -> LayerConfig:
    where = f"layers[{i}]"
    kind = str(_get(entry, "type", where))
    if kind not in MIXER_TYPES:
        raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design "
                          f"({', '.join(MIXER_TYPES)})")
    mixer = _read_mixer(kind, _get(entry, "mixer", where), where + ".mixer")
    mlp = entry.get("mlp")
    mlp_cfg = None
    if mlp:
        lw = where + ".mlp"
        mkind = str(_get(mlp, "kind", lw))
        if mkind == "dense":
            mlp_cfg = MlpConfig("dense", _int(mlp, "ff", lw))
        elif mkind == "moe":
            router = _get(mlp, "router", lw)
            shared = mlp.get("shared")
            mlp_cfg = MlpConfig("moe", _int(_get(mlp, "expert", lw), "ff", lw + ".expert"),
                                _int(router, "experts", lw + ".router"), _int(router, "top", lw + ".router"),
                                SharedExpertConfig(_int(shared, "ff", lw + ".shared")) if shared else None)
            if mlp_cfg.top > mlp_cfg.experts:
                raise ConfigError(f"config.json: {lw}.router.top ({mlp_cfg.top}) exceeds its "
                                  f"{mlp_cfg.experts} experts")
        else:
            raise ConfigError(f"config.json: {lw}.kind '{mkind}' is neither 'dense' nor 'moe'")
    return LayerConfig(kind, mixer, mlp_cfg)
