"""The Lagedra decoder as a ``ModelSpec``: a token embedding plus a learned vector per position,
parallel blocks with a norm each in front of mixer and feed-forward (RMS norms whose weight is
one number), behind every block a learned mix of the embedding output and of all layers' results
so far as the next layer's input, a final norm of the same kind and an untied head.  A block's
mixer is linear attention with a fixed decay per head or windowed softmax attention behind short
convolutions; its feed-forward, when it has one, is dense (tanh form of GELU) or a mixture of
bounded gated units.  Every part is one of the package's registered kinds with this model's
sizes and constants as parameters; tensor names are the checkpoint's (``embed``, ``pos``,
``l<i>.norm1``, ``l<i>.mix. ...``, ``l<i>.mlp. ...``, ``l<i>.dwa``, ``final.norm``, ``head``)."""
from __future__ import annotations

from typing import Optional

from ..config.lagedra import ARCHITECTURE, AttentionMixer, LagedraConfig, LagedraLayer
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec

GLU_ALPHA = 1.702       # the design fixes the sigmoid's slope in its experts
VALUE_MIX_KEY = "first_values"


def _position(m: AttentionMixer) -> PartSpec:
    if not m.rot_dims:
        return PartSpec("none")
    scaling = None
    if m.rot_scaling is not None:
        s = m.rot_scaling
        scaling = {"rope_type": "yarn", "factor": s.factor, "original": s.original,
                   "fast": s.fast, "slow": s.slow}
    return PartSpec("rope", {"rot_dim": m.rot_dims, "theta": m.rot_base, "scaling": scaling,
                             "precise": scaling is None})


def _mixer(cfg: LagedraConfig, layer: LagedraLayer, index: int, first_mixer: Optional[int]
           ) -> PartSpec:
    W, m = cfg.width, layer.mixer
    if layer.type == "lightning":
        return PartSpec("decay_attention", {
            "hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
            "decay": list(m.decay), "eps": cfg.norm_eps})
    params = {
        "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
        "value_dim": m.vdim, "scale": m.scale, "window": m.window, "position": _position(m),
        "names": {"q": "q", "k": "k", "v": "v", "o": "o"}, "conv": m.conv or None,
        "head_scales": "temp", "softcap": m.softcap or None}
    if m.v_mix:
        params["value_mix"] = {"name": "vmix", "key": VALUE_MIX_KEY,
                               "source": index == first_mixer}
    return PartSpec("attention", params)


def _feed_forward(cfg: LagedraConfig, layer: LagedraLayer) -> Optional[PartSpec]:
    mlp = layer.mlp
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return PartSpec("mlp", {"hidden_size": cfg.width, "intermediate_size": mlp.ff,
                                "activation": "gelu_tanh", "names": {"up": "up", "down": "down"}})
    return PartSpec("routed_swiglu", {
        "hidden_size": cfg.width, "expert_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "groups": mlp.groups, "keep": mlp.keep, "scale": 1.0, "shared_size": None,
        "scores": "softmax", "group_score": "max", "renormalise": True, "correction": False,
        "limit": mlp.limit, "alpha": GLU_ALPHA})


def lagedra_spec(cfg: LagedraConfig) -> ModelSpec:
    W, L = cfg.width, len(cfg.layers)
    norm = PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "scalar": True,
                                "weight_name": ""})
    first_mixer = cfg.first_value_mixer()
    layers, optional = [], []
    for i, layer in enumerate(cfg.layers):
        ff = _feed_forward(cfg, layer)
        block = PartSpec("parallel", {
            "mixer": _mixer(cfg, layer, i, first_mixer), "feed_forward": ff, "norm": norm,
            "ffn_norm": norm if ff is not None else None,
            "depth_mix": {"weight_name": "dwa", "sources": i + 2, "slots": L + 1},
            "names": {"norm": "norm1", "mixer": "mix", "ffn_norm": "norm2",
                      "feed_forward": "mlp"}})
        layers.append(LayerSpec(block, f"l{i}"))
        if ff is None:
            optional.append(f"l{i}.norm2")
        if layer.type == "attention" and not layer.mixer.v_mix:
            optional.append(f"l{i}.mix.vmix")       # may be stored, is not read
    return ModelSpec(
        hidden_size=W,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W, "weight_name": "",
                                     "learned_positions": {"name": "pos",
                                                           "rows": cfg.max_positions}}),
        embedding_prefix="embed",
        layers=layers,
        final_norm=norm,
        final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "tied_to": None,
                                 "weight_name": ""}),
        head_prefix="head",
        optional_tensors=tuple(optional),
    )


register_architecture(Architecture(
    name=ARCHITECTURE,
    parse_config=LagedraConfig.from_dict,
    build_spec=lagedra_spec,
    config_to_dict=lambda cfg: cfg.to_dict(),
))
