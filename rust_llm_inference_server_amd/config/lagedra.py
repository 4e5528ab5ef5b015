"""Typed configuration of the Lagedra decoder, read from its ``config.json``.

The file names the design under ``architecture`` and gives every size and every constant that
may differ between two models of it: vocabulary, width, the number of learned position vectors,
the norms' epsilon, and a list of layers.  A layer's ``type`` names its mixer: ``lightning``
(linear attention with a fixed decay per head) or ``attention`` (softmax attention behind short
convolutions, with a sliding window, a cap on the scores, a number per head on top of the score
scale, rotation with stretched frequencies, and optionally values mixed with those of the first
such layer).  Its ``mlp`` is null, ``dense`` (two projections around the tanh form of GELU) or
``moe`` (a mixture of bounded gated units behind a softmax router with groups).

The parser refuses what the engine would compute wrongly, with the key's name."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .gipotar import _obj, _positive
from .llama import _need, _typed

ARCHITECTURE = "Lagedra"


@dataclass(frozen=True)
class LightningMixer:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LightningMixer":
        decay = d.get("decay")
        if not isinstance(decay, list) or not decay:
            raise ConfigError(f"{where}: key 'decay' must be a list with one number per head")
        out = cls(heads=_positive(_need(d, "heads", int, where), "heads", where),
                  dim=_positive(_need(d, "dim", int, where), "dim", where),
                  vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
                  decay=tuple(_typed(x, "decay", float, where) for x in decay))
        if len(out.decay) != out.heads:
            raise ConfigError(f"{where}: 'decay' has {len(out.decay)} entries for {out.heads} heads")
        if not all(0.0 < x <= 1.0 for x in out.decay):
            raise ConfigError(f"{where}: every 'decay' must lie in (0, 1]")
        if out.dim > 256:
            raise ConfigError(f"{where}: 'dim' {out.dim} is above the kernels' 256")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class RotScaling:
    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "RotScaling":
        out = cls(factor=_need(d, "factor", float, where),
                  original=_need(d, "original", float, where),
                  fast=_need(d, "fast", float, where), slow=_need(d, "slow", float, where))
        for key in ("factor", "original", "fast", "slow"):
            if not getattr(out, key) > 0:
                raise ConfigError(f"{where}: key '{key}' must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        original = int(self.original) if float(self.original).is_integer() else self.original
        return {"factor": self.factor, "fast": self.fast, "original": original, "slow": self.slow}


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0                       # taps of the short convolutions (0: none)
    window: Optional[int] = None        # positions a query sees, itself included
    softcap: float = 0.0                # 0: no cap
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[RotScaling] = None
    v_mix: bool = False

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "AttentionMixer":
        kw: Dict[str, Any] = dict(
            heads=_positive(_need(d, "heads", int, where), "heads", where),
            kv_heads=_positive(_need(d, "kv_heads", int, where), "kv_heads", where),
            dim=_positive(_need(d, "dim", int, where), "dim", where),
            vdim=_positive(_need(d, "vdim", int, where), "vdim", where),
            scale=_need(d, "scale", float, where))
        if d.get("conv") is not None:
            kw["conv"] = _typed(d["conv"], "conv", int, where)
            if not 0 <= kw["conv"] <= 16:
                raise ConfigError(f"{where}: 'conv' {kw['conv']} must be 0 to 16 taps")
        if d.get("mask") is not None:
            mask = _obj(d, "mask", where)
            kw["window"] = _positive(_need(mask, "size", int, where + " mask"), "size",
                                     where + " mask")
        if d.get("softcap") is not None:
            kw["softcap"] = _typed(d["softcap"], "softcap", float, where)
            if kw["softcap"] < 0:
                raise ConfigError(f"{where}: 'softcap' must be positive")
        if d.get("rot") is not None:
            rot = _obj(d, "rot", where)
            kw["rot_dims"] = _need(rot, "dims", int, where + " rot")
            kw["rot_base"] = _need(rot, "base", float, where + " rot")
            if rot.get("scaling") is not None:
                kw["rot_scaling"] = RotScaling.from_dict(_obj(rot, "scaling", where + " rot"),
                                                         where + " rot scaling")
        if d.get("v_mix") is not None:
            kw["v_mix"] = _typed(d["v_mix"], "v_mix", bool, where)
        out = cls(**kw)
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: 'heads' {out.heads} is not a multiple of 'kv_heads' "
                              f"{out.kv_heads}")
        if out.rot_dims < 0 or out.rot_dims % 2 or out.rot_dims > out.dim:
            raise ConfigError(f"{where} rot: 'dims' {out.rot_dims} must be even and at most "
                              f"'dim' {out.dim}")
        if out.rot_dims and not out.rot_base > 1:
            raise ConfigError(f"{where} rot: 'base' must be above 1")
        if out.v_mix and not out.conv:
            raise ConfigError(f"{where}: 'v_mix' needs the convolutions ('conv')")
        return out

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"conv": self.conv, "dim": self.dim, "heads": self.heads,
                             "kv_heads": self.kv_heads, "scale": self.scale,
                             "softcap": self.softcap, "v_mix": self.v_mix, "vdim": self.vdim}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.rot_dims:
            rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                rot["scaling"] = self.rot_scaling.to_dict()
            d["rot"] = rot
        return d


@dataclass(frozen=True)
class LagedraMlp:
    kind: str                           # "dense" or "moe"
    ff: int                             # inner width (of one expert for "moe")
    limit: float = 0.0
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LagedraMlp":
        kind = _need(d, "kind", str, where)
        if kind == "dense":
            return cls("dense", _positive(_need(d, "ff", int, where), "ff", where))
        if kind != "moe":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (known: 'dense', 'moe')")
        expert, router = _obj(d, "expert", where), _obj(d, "router", where)
        groups = router.get("groups")
        count = keep = 1
        if groups is not None:
            groups = _obj(router, "groups", where + " router")
            count = _positive(_need(groups, "count", int, where + " router groups"), "count", where)
            keep = _positive(_need(groups, "keep", int, where + " router groups"), "keep", where)
        out = cls("moe", _positive(_need(expert, "ff", int, where + " expert"), "ff", where),
                  limit=_need(expert, "limit", float, where + " expert"),
                  experts=_positive(_need(router, "experts", int, where + " router"), "experts",
                                    where),
                  top=_positive(_need(router, "top", int, where + " router"), "top", where),
                  groups=count, keep=keep)
        if not out.limit > 0:
            raise ConfigError(f"{where} expert: 'limit' must be positive")
        if out.experts % out.groups or out.keep > out.groups \
                or out.top > out.keep * (out.experts // out.groups):
            raise ConfigError(f"{where} router: {out.experts} experts in {out.groups} groups, "
                              f"{out.keep} kept, {out.top} chosen do not fit")
        return out

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                "router": {"experts": self.experts,
                           "groups": {"count": self.groups, "keep": self.keep}, "top": self.top}}


@dataclass(frozen=True)
class LagedraLayer:
    type: str                           # "lightning" or "attention"
    mixer: Any                          # LightningMixer or AttentionMixer
    mlp: Optional[LagedraMlp]

    @classmethod
    def from_dict(cls, d: Any, index: int) -> "LagedraLayer":
        where = f"config.json layers[{index}]"
        if not isinstance(d, dict):
            raise ConfigError(f"{where}: must be an object")
        kind = _need(d, "type", str, where)
        mixer = _obj(d, "mixer", where)
        if kind == "lightning":
            m: Any = LightningMixer.from_dict(mixer, where + " mixer")
        elif kind == "attention":
            m = AttentionMixer.from_dict(mixer, where + " mixer")
        else:
            raise ConfigError(f"{where}: type '{kind}' is not supported (known: 'lightning', "
                              "'attention')")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}: 'mlp' must be an object or null")
        return cls(kind, m, None if mlp is None else LagedraMlp.from_dict(mlp, where + " mlp"))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class LagedraConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    layers: Tuple[LagedraLayer, ...]
    architecture: str = ARCHITECTURE

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_position_embeddings(self) -> int:
        """The longest sequence the model can place: one learned vector per position."""
        return self.max_positions

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LagedraConfig":
        where = "config.json"
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        out = cls(vocab=_positive(_need(d, "vocab", int), "vocab", where),
                  width=_positive(_need(d, "width", int), "width", where),
                  max_positions=_positive(_need(d, "max_positions", int), "max_positions", where),
                  norm_eps=_need(_obj(d, "norm", where), "eps", float, where + " norm"),
                  layers=tuple(LagedraLayer.from_dict(l, i) for i, l in enumerate(layers)))
        if not out.norm_eps > 0:
            raise ConfigError(f"{where} norm: 'eps' must be positive")
        first = out.first_value_mixer()
        if first is not None:
            a = out.layers[first].mixer
            for i, layer in enumerate(out.layers):
                m = layer.mixer
                if layer.type == "attention" and m.v_mix and (m.kv_heads, m.vdim) != (a.kv_heads, a.vdim):
                    raise ConfigError(
                        f"{where} layers[{i}] mixer: 'v_mix' needs the {a.kv_heads} key/value "
                        f"heads of {a.vdim} that layers[{first}] has, got {m.kv_heads} of {m.vdim}")
        return out

    def first_value_mixer(self) -> Optional[int]:
        """Index of the first layer whose mixer says ``v_mix`` (the one whose values the later
        ones mix into theirs); None when no layer does."""
        for i, layer in enumerate(self.layers):
            if layer.type == "attention" and layer.mixer.v_mix:
                return i
        return None

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers],
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
                "vocab": self.vocab, "width": self.width}
