"""The Pubodra decoder as data: how its configuration becomes a :class:`ModelSpec`.

Every layer is a pre-norm residual block whose norms are Dynamic Tanh, whose mixer is latent
attention (a small cached latent per token, a rotated key part shared by all heads, a window,
an output gate) and whose feed-forward is dense (tanh-GELU), routed (softmax router, squared
ReLU experts) or absent.  A stretch of the layers may run several times in a row with the same
weights: each run of a layer is a site of the run order with a cache of its own, and a learned
vector per pass is added to the stream right before the pass's first layer.  The head shares
the embedding table.

Tensor names: ``embed``, ``loop.step``, ``final.norm``(``.b``, ``.alpha``) and, for layer i,
``l<i>.norm1|norm2``(``.b``, ``.alpha``), ``l<i>.mix.{q,dkv,dkv.norm,uk,uv,g,o}``,
``l<i>.mlp.{up,down}`` or ``l<i>.mlp.router`` with ``l<i>.mlp.e<k>.{up,down}``.
"""
from __future__ import annotations

from typing import Dict

from ..config.pubodra_config import ARCHITECTURE, LayerConfig, PubodraConfig
from ..config.registry import ARCHITECTURES, Architecture
from ..config.specs import ModelSpec, PartSpec, RunEntry, mixer_only_layer, prenorm_layer


def _norm_names(slot: str, name: str) -> Dict[str, str]:
    return {f"{slot}.weight": name, f"{slot}.bias": name + ".b", f"{slot}.alpha": name + ".alpha"}


def pubodra_layer(cfg: PubodraConfig, i: int, layer: LayerConfig):
    p = f"l{i}."
    m = layer.mixer
    norm = PartSpec("dynamic_tanh", {"size": cfg.width})
    position = None
    if m.rot is not None:
        position = PartSpec("rotary", {
            "rotary_dim": m.rot.dims, "theta": m.rot.base, "pairing": "interleaved",
            "scaling": m.rot.scaling.to_dict() if m.rot.scaling is not None else None})
    mixer = PartSpec("latent_attention", {
        "hidden_size": cfg.width, "num_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
        "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps,
        "position": position, "window": m.window, "gate": True})
    names = {"mixer.q": p + "mix.q", "mixer.dkv": p + "mix.dkv", "mixer.dkv_norm": p + "mix.dkv.norm",
             "mixer.uk": p + "mix.uk", "mixer.uv": p + "mix.uv", "mixer.g": p + "mix.g",
             "mixer.o": p + "mix.o"}
    names.update(_norm_names("mixer_norm", p + "norm1"))
    if layer.mlp is None:
        return mixer_only_layer(mixer, norm, names)
    names.update(_norm_names("feed_forward_norm", p + "norm2"))
    if layer.mlp.kind == "dense":
        feed_forward = PartSpec("mlp", {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff,
                                        "activation": "gelu_tanh"})
        names.update({"feed_forward.up": p + "mlp.up", "feed_forward.down": p + "mlp.down"})
    else:
        feed_forward = PartSpec("routed_mlp", {
            "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "experts": layer.mlp.experts,
            "top": layer.mlp.top, "activation": "relu_squared", "scores": "softmax",
            "renormalise": True, "renormalise_eps": 1e-20})
        names["feed_forward.router"] = p + "mlp.router"
        for k in range(layer.mlp.experts):
            names[f"feed_forward.experts.{k}.up"] = p + f"mlp.e{k}.up"
            names[f"feed_forward.experts.{k}.down"] = p + f"mlp.e{k}.down"
    return prenorm_layer(mixer, feed_forward, norm, norm, names)


def pubodra_run_order(cfg: PubodraConfig):
    n = len(cfg.layers)
    if cfg.loop is None:
        return [RunEntry(i) for i in range(n)]
    loop = cfg.loop
    order = [RunEntry(i) for i in range(loop.start)]
    for turn in range(loop.times):
        for i in range(loop.start, loop.stop):
            if i == loop.start:
                step = PartSpec("row_offset", {"size": cfg.width, "rows": loop.times, "row": turn})
                order.append(RunEntry(i, before=step, before_names={"table": "loop.step"}))
            else:
                order.append(RunEntry(i))
    return order + [RunEntry(i) for i in range(loop.stop, n)]


def pubodra_model_spec(cfg: PubodraConfig) -> ModelSpec:
    layers = [pubodra_layer(cfg, i, layer) for i, layer in enumerate(cfg.layers)]
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embedding_name="embed", layers=layers,
        run_order=pubodra_run_order(cfg),
        final_norm=PartSpec("dynamic_tanh", {"size": cfg.width}),
        final_norm_names={"weight": "final.norm", "bias": "final.norm.b", "alpha": "final.norm.alpha"},
        head_name=None, init_std=cfg.initializer_range, max_positions=0)


ARCHITECTURES.register(ARCHITECTURE, Architecture(
    name=ARCHITECTURE, read_config=PubodraConfig.from_dict, model_spec=pubodra_model_spec))
