"""The Pamolix decoder as a ``ModelSpec``: a scaled token embedding, pre-norm blocks over
several residual streams that hyper-connections mix (or over one plain stream when the model
names none), RMS norms whose weights are stored around zero, a final norm of the same kind and
a head tied to the embedding table (without its scale).  A block's mixer is one of two kinds of
softmax attention: the first with biased projections, a norm over every query and key head, a
factor on the queries that grows with the position, all earlier keys and a learned sink in the
softmax (it may read the keys and values of an earlier layer instead of making its own); the
second with a rotation of a part of every head under stretched positions, capped scores, a
sliding window that also keeps the sequence's first keys, and a gate per head on its output.
Its feed-forward, when it has one, is dense (erf form of GELU) or a mixture of squared-ReLU
units behind a biased router.  Every part is one of the package's registered kinds with this
model's sizes and constants as parameters; tensor names are the checkpoint's (``embed``,
``l<i>.norm1``, ``l<i>.mix. ...``, ``l<i>.mlp. ...``, ``l<i>.hc1. ...``, ``final.norm``)."""
from __future__ import annotations

from typing import List, Optional

from ..config.pamolix import ARCHITECTURE, PamolixConfig, PamolixLayer, PamolixMixer
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, RunEntry


def _kept_by_cache(cfg: PamolixConfig, index: int) -> Optional[dict]:
    """What the pages of layer ``index`` (or of the layer whose pages it reads) must keep: the
    widest of the masks of all layers that read them; None when the layer's own mask says it."""
    owner = cfg.layers[index].mixer.kv_from
    owner = index if owner is None else owner
    readers = [l.mixer for i, l in enumerate(cfg.layers) if i == owner or l.mixer.kv_from == owner]
    if len(readers) == 1:
        return None
    if any(m.window is None for m in readers):
        return {"window": None, "keep_first": 0}
    return {"window": max(m.window for m in readers),
            "keep_first": max(m.keep_first for m in readers)}


def _mixer(cfg: PamolixConfig, m: PamolixMixer, index: int) -> PartSpec:
    params = {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
              "head_dim": m.dim, "value_dim": m.vdim, "scale": m.scale,
              "names": {"q": "q", "k": "k", "v": "v", "o": "o"},
              "cache_like": _kept_by_cache(cfg, index)}
    if m.kind == "attention":
        params.update({
            "window": None, "position": PartSpec("none"), "bias": ".b",
            "qk_norm": {"q": "q.norm", "k": "k.norm", "eps": cfg.norm_eps}, "sinks": "sink",
            "shared_kv": m.kv_from is not None})
        if m.temp_every:
            params["query_temperature"] = {"coef": m.temp_coef, "every": m.temp_every}
        return PartSpec("attention", params)
    position = PartSpec("none")
    if m.rot_dims:
        scaling = None if m.rot_factor == 1.0 else {"rope_type": "linear", "factor": m.rot_factor}
        position = PartSpec("rope", {"rot_dim": m.rot_dims, "theta": m.rot_base,
                                     "scaling": scaling, "precise": True})
    params.update({"window": m.window, "keep_first": m.keep_first if m.window else 0,
                   "position": position, "softcap": m.softcap or None, "gate": "g",
                   "shared_kv": m.kv_from is not None})
    return PartSpec("attention", params)


def _feed_forward(cfg: PamolixConfig, layer: PamolixLayer) -> Optional[PartSpec]:
    mlp = layer.mlp
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return PartSpec("mlp", {"hidden_size": cfg.width, "intermediate_size": mlp.ff,
                                "activation": "gelu_erf", "names": {"up": "up", "down": "down"}})
    return PartSpec("routed_mlp", {"hidden_size": cfg.width, "expert_size": mlp.ff,
                                   "experts": mlp.experts, "top": mlp.top, "activation": "relu2",
                                   "router_bias": ".b"})


def pamolix_spec(cfg: PamolixConfig) -> ModelSpec:
    W = cfg.width
    norm = PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "weight_offset": 1.0,
                                "weight_name": ""})
    layers: List[LayerSpec] = []
    runs: List[RunEntry] = []
    for i, layer in enumerate(cfg.layers):
        params = {"mixer": _mixer(cfg, layer.mixer, i), "feed_forward": _feed_forward(cfg, layer),
                  "mixer_norm": norm, "ffn_norm": norm,
                  "names": {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2",
                            "feed_forward": "mlp"}}
        if cfg.streams:
            params.update({"streams": cfg.streams, "connections": ("hc1", "hc2")})
        layers.append(LayerSpec(PartSpec("hyper" if cfg.streams else "prenorm", params), f"l{i}"))
        # (every layer runs once, so a layer's index is its run's)
        runs.append(RunEntry(i, cache_of=layer.mixer.kv_from))
    return ModelSpec(
        hidden_size=W,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W, "weight_name": "",
                                     "scale": cfg.embedding_scale}),
        embedding_prefix="embed",
        layers=layers,
        run_order=runs,
        final_norm=norm,
        final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": "embed"}),
        head_prefix="head",
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    parse_config=PamolixConfig.from_dict,
    build_spec=pamolix_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
))
