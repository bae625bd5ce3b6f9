"""The Larupel decoder as data: how its configuration becomes a :class:`ModelSpec`.

The token embedding gets a sinusoidal position vector; nothing else in the model knows a
position.  Every layer wraps each of its two branches in a layer norm before and after:
``x += norm1b(mixer(norm1(x)))``, ``x += norm2b(ff(norm2(x)))``.  The mixer is softmax attention
(q/k RMS norm, a learned temperature per head, no rotation; a layer may read an earlier
layer's keys and values instead of making its own), the gated delta rule behind short causal
convolutions, or the generalized delta rule; the last two keep a matrix of state per head and
request instead of keys and values.  The feed-forward is a gated tanh-GELU layer, a mixture of
gated SiLU experts (router with a bias, softmax over the chosen logits, a gated shared expert)
or absent.  Final layer norm, then an untied head.

Tensor names: ``embed``, ``head``, ``final.norm``(``.b``) and, for layer i,
``l<i>.norm1|norm1b|norm2|norm2b``(``.b``), ``l<i>.mix.*`` and ``l<i>.mlp.*`` as the functions
below list them.
"""
from __future__ import annotations

from typing import Dict

from ..config.larupel_config import (ARCHITECTURE, AttentionConfig, DeltaConfig, GeneralDeltaConfig,
                                     LarupelConfig, LayerConfig)
from ..config.registry import ARCHITECTURES, Architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry

SINUSOID_BASE = 10000.0     # the position vector's frequencies are base^(-2i/width)
UNIT_KEY_EPS = 1e-6         # inside the root of a key's (or query's) length
DECAY_SCALE = 0.6065306597126334    # exp(-1/2): the generalized delta rule's decay is exp(-this * sigmoid(.))


def _norm_names(slot: str, name: str) -> Dict[str, str]:
    return {f"{slot}.weight": name, f"{slot}.bias": name + ".b"}


def _attention(cfg: LarupelConfig, m: AttentionConfig, p: str):
    mixer = PartSpec("attention", {
        "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
        "value_dim": m.vdim, "scale": m.scale, "qk_norm": PartSpec("rms", {"size": m.dim, "eps": cfg.norm_eps}),
        "position": None, "window": None, "head_temperature": True, "shared_kv": m.kv_from is not None})
    names = {"mixer.q_proj": p + "q", "mixer.o_proj": p + "o", "mixer.q_norm.weight": p + "q.norm",
             "mixer.head_temperature": p + "temp"}
    if m.kv_from is None:
        names.update({"mixer.k_proj": p + "k", "mixer.v_proj": p + "v", "mixer.k_norm.weight": p + "k.norm"})
    return mixer, names


def _delta(cfg: LarupelConfig, m: DeltaConfig, p: str):
    mixer = PartSpec("gated_delta", {
        "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
        "value_dim": m.vdim, "conv_taps": m.conv, "norm_eps": cfg.norm_eps, "unit_eps": UNIT_KEY_EPS})
    names = {"mixer." + logical: p + stored for logical, stored in (
        ("q", "q"), ("q_conv", "q.conv"), ("k", "k"), ("k_conv", "k.conv"), ("v", "v"), ("v_conv", "v.conv"),
        ("beta", "b"), ("rate", "a"), ("rate_log", "A_log"), ("rate_bias", "dt_bias"), ("norm", "norm"),
        ("gate", "g"), ("o", "o"))}
    return mixer, names


def _general_delta(cfg: LarupelConfig, m: GeneralDeltaConfig, p: str):
    mixer = PartSpec("general_delta", {
        "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "norm_eps": cfg.norm_eps,
        "unit_eps": UNIT_KEY_EPS, "decay_scale": DECAY_SCALE})
    names = {"mixer." + logical: p + stored for logical, stored in (
        ("r", "r"), ("k", "k"), ("v", "v"), ("gate", "g"), ("removal", "a"), ("removal_bias", "a.b"),
        ("decay_in", "w1"), ("decay_out", "w2"), ("decay_bias", "w0"), ("norm", "norm"), ("o", "o"))}
    return mixer, names


def _feed_forward(cfg: LarupelConfig, layer: LayerConfig, p: str):
    mlp = layer.mlp
    if mlp.kind == "dense":
        part = PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": mlp.ff,
                                      "activation": "gelu_tanh"})
        return part, {"feed_forward.gate_proj": p + "gate", "feed_forward.up_proj": p + "up",
                      "feed_forward.down_proj": p + "down"}
    part = PartSpec("routed_gated_mlp", {
        "hidden_size": cfg.width, "intermediate_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "activation": "silu", "router_bias": True,
        "shared_size": mlp.shared.ff if mlp.shared is not None else 0})
    names = {"feed_forward.router": p + "router", "feed_forward.router_bias": p + "router.b"}
    for k in range(mlp.experts):
        for which in ("gate", "up", "down"):
            names[f"feed_forward.experts.{k}.{which}"] = p + f"e{k}.{which}"
    if mlp.shared is not None:
        for which in ("gate", "up", "down"):
            names[f"feed_forward.shared.{which}"] = p + f"shared.{which}"
        names["feed_forward.shared_gate"] = p + "shared.sg"
    return part, names


def larupel_layer(cfg: LarupelConfig, i: int, layer: LayerConfig) -> LayerSpec:
    p = f"l{i}."
    norm = PartSpec("layer_norm", {"size": cfg.width, "eps": cfg.norm_eps})
    build = {AttentionConfig: _attention, DeltaConfig: _delta, GeneralDeltaConfig: _general_delta}
    mixer, names = build[type(layer.mixer)](cfg, layer.mixer, p + "mix.")
    names.update(_norm_names("mixer_norm", p + "norm1"))
    names.update(_norm_names("mixer_post_norm", p + "norm1b"))
    parts = {"mixer": mixer, "mixer_norm": norm, "mixer_post_norm": norm}
    if layer.mlp is None:
        return LayerSpec("sandwich_mixer", parts, names)
    feed_forward, ff_names = _feed_forward(cfg, layer, p + "mlp.")
    names.update(ff_names)
    names.update(_norm_names("feed_forward_norm", p + "norm2"))
    names.update(_norm_names("feed_forward_post_norm", p + "norm2b"))
    parts.update({"feed_forward": feed_forward, "feed_forward_norm": norm, "feed_forward_post_norm": norm})
    return LayerSpec("sandwich_residual", parts, names)


def larupel_run_order(cfg: LarupelConfig):
    """Each layer runs once; a layer that reads another layer's keys and values is a site without
    a cache of its own."""
    return [RunEntry(i, cache_of=getattr(layer.mixer, "kv_from", None)) for i, layer in enumerate(cfg.layers)]


def larupel_model_spec(cfg: LarupelConfig) -> ModelSpec:
    layers = [larupel_layer(cfg, i, layer) for i, layer in enumerate(cfg.layers)]
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embedding_name="embed", layers=layers,
        run_order=larupel_run_order(cfg),
        final_norm=PartSpec("layer_norm", {"size": cfg.width, "eps": cfg.norm_eps}),
        final_norm_names={"weight": "final.norm", "bias": "final.norm.b"},
        head_name="head", init_std=cfg.initializer_range, max_positions=0,
        embedding=PartSpec("sinusoid_token_embedding", dict(sizes, base=SINUSOID_BASE)))


ARCHITECTURES.register(ARCHITECTURE, Architecture(
    name=ARCHITECTURE, read_config=LarupelConfig.from_dict, model_spec=larupel_model_spec))
