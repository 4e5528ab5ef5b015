"""Typed configuration of the Pamolix decoder, read from its ``config.json``.

The file names the design under ``architecture`` and gives every size and every constant that
may differ between two models of it: vocabulary, width, the factor on the embedding rows, the
norms' epsilon, the number of residual streams that the layers' hyper-connections mix
(``streams``; absent: one plain residual stream) and a list of layers.  A layer's ``type``
names its mixer: ``attention`` (biased projections, a norm over every query and key head, a
factor on the queries that grows with the position, all earlier keys, a learned sink in the
softmax's denominator, optionally the keys and values of an earlier layer, ``kv_from``) or
``attention_2`` (rotation of a part of every head with linearly stretched positions, capped
scores, a sliding window that also keeps the sequence's first keys, a gate per head on the
output).  Its ``mlp`` is null, ``dense`` (two projections around the erf form of GELU) or
``moe`` (a mixture of two-projection units around a squared ReLU behind a biased router whose
chosen logits are soft-maxed among themselves).

The parser refuses what the engine would compute wrongly, with the key's name."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .gipotar import _obj, _positive
from .llama import _need, _typed

ARCHITECTURE = "Pamolix"
MIXERS = ("attention", "attention_2")


@dataclass(frozen=True)
class PamolixMixer:
    kind: str                           # "attention" or "attention_2"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    # "attention"
    temp_coef: float = 0.0              # queries times 1 + coef ln(floor((p + 1) / every) + 1)
    temp_every: int = 0                 # 0: no such factor
    # either kind
    kv_from: Optional[int] = None       # layer whose keys and values this one reads
    # "attention_2"
    window: Optional[int] = None        # positions a query sees, itself included
    keep_first: int = 0                 # first keys of the sequence that stay visible
    softcap: float = 0.0                # 0: no cap
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_factor: float = 1.0             # positions are divided by it

    @classmethod
    def from_dict(cls, kind: str, d: Dict[str, Any], where: str) -> "PamolixMixer":
        kw: Dict[str, Any] = dict(
            kind=kind,
            heads=_positive(_need(d, "heads", int, where), "heads", where),
            kv_heads=_positive(_need(d, "kv_heads", int, where), "kv_heads", where),
            dim=_positive(_need(d, "dim", int, where), "dim", where),
            vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
            scale=_need(d, "scale", float, where))
        if kind == "attention":
            if d.get("q_temp") is not None:
                temp = _obj(d, "q_temp", where)
                kw["temp_coef"] = _need(temp, "coef", float, where + " q_temp")
                kw["temp_every"] = _positive(_need(temp, "every", int, where + " q_temp"),
                                             "every", where + " q_temp")
        else:
            if d.get("mask") is not None:
                mask = _obj(d, "mask", where)
                kw["window"] = _positive(_need(mask, "size", int, where + " mask"), "size",
                                         where + " mask")
                if mask.get("keep_first") is not None:
                    kw["keep_first"] = _typed(mask["keep_first"], "keep_first", int,
                                              where + " mask")
                    if kw["keep_first"] < 0:
                        raise ConfigError(f"{where} mask: 'keep_first' must not be negative")
            if d.get("softcap") is not None:
                kw["softcap"] = _typed(d["softcap"], "softcap", float, where)
                if kw["softcap"] < 0:
                    raise ConfigError(f"{where}: 'softcap' must be positive")
            if d.get("rot") is not None:
                rot = _obj(d, "rot", where)
                kw["rot_dims"] = _need(rot, "dims", int, where + " rot")
                kw["rot_base"] = _need(rot, "base", float, where + " rot")
                if rot.get("scaling") is not None:
                    kw["rot_factor"] = _need(_obj(rot, "scaling", where + " rot"), "factor",
                                             float, where + " rot scaling")
        if d.get("kv_from") is not None:
            kw["kv_from"] = _typed(d["kv_from"], "kv_from", int, where)
        out = cls(**kw)
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: 'heads' {out.heads} is not a multiple of 'kv_heads' "
                              f"{out.kv_heads}")
        if out.rot_dims < 0 or out.rot_dims % 2 or out.rot_dims > out.dim:
            raise ConfigError(f"{where} rot: 'dims' {out.rot_dims} must be even and at most "
                              f"'dim' {out.dim}")
        if out.rot_dims and not (out.rot_base > 1 and out.rot_factor > 0):
            raise ConfigError(f"{where} rot: 'base' must be above 1 and the scaling's 'factor' "
                              "positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                             "scale": self.scale, "vdim": self.vdim}
        if self.kind == "attention":
            if self.temp_every:
                d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
            if self.kv_from is not None:
                d["kv_from"] = self.kv_from
            return d
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        if self.window is not None:
            d["mask"] = {"keep_first": self.keep_first, "size": self.window}
        if self.softcap:
            d["softcap"] = self.softcap
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims,
                        "scaling": {"factor": self.rot_factor}}
        return d


@dataclass(frozen=True)
class PamolixMlp:
    kind: str                           # "dense" or "moe"
    ff: int                             # inner width (of one expert for "moe")
    experts: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "PamolixMlp":
        kind = _need(d, "kind", str, where)
        if kind == "dense":
            return cls("dense", _positive(_need(d, "ff", int, where), "ff", where))
        if kind != "moe":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (known: 'dense', 'moe')")
        expert, router = _obj(d, "expert", where), _obj(d, "router", where)
        out = cls("moe", _positive(_need(expert, "ff", int, where + " expert"), "ff", where),
                  experts=_positive(_need(router, "experts", int, where + " router"), "experts",
                                    where),
                  top=_positive(_need(router, "top", int, where + " router"), "top", where))
        if out.top > out.experts:
            raise ConfigError(f"{where} router: {out.top} chosen of {out.experts} experts")
        return out

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        return {"expert": {"ff": self.ff}, "kind": "moe",
                "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class PamolixLayer:
    type: str
    mixer: PamolixMixer
    mlp: Optional[PamolixMlp]

    @classmethod
    def from_dict(cls, d: Any, index: int) -> "PamolixLayer":
        where = f"config.json layers[{index}]"
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: must be an object")
        kind = _need(d, "type", str, where)
        if kind not in MIXERS:
            raise ConfigError(f"{where}: type '{kind}' is not supported (known: "
                              f"{', '.join(repr(m) for m in MIXERS)})")
        mixer = PamolixMixer.from_dict(kind, _obj(d, "mixer", where), where + " mixer")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: 'mlp' must be an object or null")
        return cls(kind, mixer, None if mlp is None else PamolixMlp.from_dict(mlp, where + " mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class PamolixConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    streams: int                        # 0: one plain residual stream, no hyper-connections
    layers: Tuple[PamolixLayer, ...]
    architecture: str = ARCHITECTURE

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_position_embeddings(self) -> int:
        """No table bounds the positions: the engine's own limit holds."""
        return 1 << 20

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PamolixConfig":
        where = "config.json"
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        scale = 1.0
        if d.get("embedding") is not None:
            scale = _need(_obj(d, "embedding", where), "scale", float, where + " embedding")
        streams = 0
        if d.get("streams") is not None:
            streams = _positive(_typed(d["streams"], "streams", int, where), "streams", where)
        out = cls(vocab=_positive(_need(d, "vocab", int), "vocab", where),
                  width=_positive(_need(d, "width", int), "width", where),
                  embedding_scale=scale,
                  norm_eps=_need(_obj(d, "norm", where), "eps", float, where + " norm"),
                  streams=streams,
                  layers=tuple(PamolixLayer.from_dict(l, i) for i, l in enumerate(layers)))
        if not out.norm_eps > 0:
            raise ConfigError(f"{where} norm: 'eps' must be positive")
        if out.streams > 16:
            raise ConfigError(f"{where}: 'streams' {out.streams} is above the kernels' 16")
        for i, layer in enumerate(out.layers):
            m = layer.mixer
            if m.kv_from is None:
                continue
            at = f"{where} layers[{i}] mixer"
            if not 0 <= m.kv_from < i:
                raise ConfigError(f"{at}: 'kv_from' {m.kv_from} must name an earlier layer")
            src = out.layers[m.kv_from]
            if src.type != layer.type or src.mixer.kv_from is not None:
                raise ConfigError(f"{at}: 'kv_from' {m.kv_from} must name a layer of the same "
                                  "type with keys and values of its own")
            s = src.mixer
            if (s.heads, s.kv_heads, s.dim, s.vdim) != (m.heads, m.kv_heads, m.dim, m.vdim):
                raise ConfigError(f"{at}: heads and head sizes differ from those of layers"
                                  f"[{m.kv_from}], whose keys and values it reads")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture,
                             "embedding": {"scale": self.embedding_scale},
                             "layers": [l.to_dict() for l in self.layers],
                             "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                             "width": self.width}
        if self.streams:
            d["streams"] = self.streams
        return d
