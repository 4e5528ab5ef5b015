"""Rotary position encoding with optional llama3 frequency scaling.

Inverse frequencies are computed in float32 exactly as the reference does
(crates/model/src/rope.rs:19-49): ``1 / theta^(2j/d)``; under ``llama3`` scaling a frequency
whose wavelength is below ``original / high_freq_factor`` is kept, one above
``original / low_freq_factor`` is divided by ``factor``, and those between are blended.
Angles ``position * inv_freq``, cosines and sines are float32 (rope.rs:61-78) and stay so:
the table is never rounded to the activation dtype.  A second kind of scaling, ``yarn``,
stretches the slow frequencies by ``factor``, keeps the fast ones, blends those between along
a ramp over the pair index, and multiplies cosines and sines by ``0.1 ln(factor) + 1``.  The rotation pairs dim ``j`` with
``j + rot/2`` (rotate-half, rope.rs:111-117) and is applied by the cache-write kernel."""
from __future__ import annotations

import math
from typing import Any, Dict, Optional

import torch

from .base import BuildContext, PositionEncoding, register


def yarn_frequencies(rot_dim: int, theta: float, scaling: Dict[str, Any]) -> torch.Tensor:
    """Frequencies of pair i = 0 .. rot_dim / 2 - 1 in double precision.  With ``turns(n)`` the
    (fractional) pair index whose wave makes n turns over ``original`` positions,
    ``rot_dim ln(original / (2 pi n)) / (2 ln theta)``: pairs up to ``lo = floor(turns(fast))``
    keep ``f_i = theta^(-2 i / rot_dim)``, pairs from ``hi = ceil(turns(slow))`` on get
    ``f_i / factor``, and between the two the share of the stretched frequency rises linearly."""
    factor, original, fast, slow = (float(scaling.get(key) or 0.0)
                                    for key in ("factor", "original", "fast", "slow"))
    if not (factor > 0 and original > 0 and fast > 0 and slow > 0):
        raise ValueError("position encoding 'rope': yarn scaling needs positive 'factor', "
                         "'original', 'fast' and 'slow'")

    def turns(n: float) -> float:
        return rot_dim * math.log(original / (2.0 * math.pi * n)) / (2.0 * math.log(theta))

    lo = max(math.floor(turns(fast)), 0)
    hi = min(math.ceil(turns(slow)), rot_dim - 1)
    i = torch.arange(0, rot_dim // 2, dtype=torch.float64)
    f = float(theta) ** (-2.0 * i / rot_dim)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp)


def inverse_frequencies(rot_dim: int, theta: float, scaling: Optional[Dict[str, Any]]
                        ) -> torch.Tensor:
    f32 = torch.float32
    exponent = torch.arange(0, rot_dim, 2, dtype=f32) / torch.tensor(float(rot_dim), dtype=f32)
    inv = 1.0 / torch.pow(torch.tensor(float(theta), dtype=f32), exponent)
    if not scaling:
        return inv
    kind = scaling.get("rope_type")
    if kind != "llama3":
        raise ValueError(f"position encoding 'rope': unknown scaling '{kind}' (known: 'llama3')")
    factor = torch.tensor(float(scaling["factor"]), dtype=f32)
    low = torch.tensor(float(scaling["low_freq_factor"]), dtype=f32)
    high = torch.tensor(float(scaling["high_freq_factor"]), dtype=f32)
    old_ctx = torch.tensor(float(scaling["original_max_position_embeddings"]), dtype=f32)
    low_wavelen, high_wavelen = old_ctx / low, old_ctx / high
    wavelen = torch.tensor(2.0 * math.pi, dtype=f32) / inv
    smooth = (old_ctx / wavelen - low) / (high - low)
    blended = (1.0 - smooth) * inv / factor + smooth * inv
    return torch.where(wavelen < high_wavelen, inv,
                       torch.where(wavelen > low_wavelen, inv / factor, blended))


@register("position", "rope")
class RotaryEmbedding(PositionEncoding):
    """Parameters: ``rot_dim`` (rotated width, at most the head size), ``theta``, ``scaling``
    (None, the llama3 fields, ``{"rope_type": "yarn", "factor", "original", "fast",
    "slow"}``, or with ``precise`` ``{"rope_type": "linear", "factor"}``: every frequency divided
    by the factor).  Holds ``cos``/``sin`` float32 ``(max_positions, rot/2)``.
    Optional ``precise``: frequencies, angles, cosines and sines are made in double precision
    and rounded once to float32 (without it they are float32 from the start, as the reference
    makes them); yarn scaling is always made that way."""

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        rot = int(params["rot_dim"])
        if rot % 2:
            raise ValueError(f"position encoding 'rope': rot_dim {rot} must be even")
        scaling = params.get("scaling")
        magnitude = 1.0
        if scaling and scaling.get("rope_type") == "yarn":
            inv = yarn_frequencies(rot, float(params["theta"]), scaling)
            magnitude = 0.1 * math.log(float(scaling["factor"])) + 1.0
            pos = torch.arange(ctx.max_positions, dtype=torch.float64).reshape(-1, 1)
        elif params.get("precise"):
            if scaling and scaling.get("rope_type") != "linear":
                raise ValueError("position encoding 'rope': 'precise' has no llama3 scaling")
            f64 = torch.float64
            inv = float(params["theta"]) ** (-torch.arange(0, rot, 2, dtype=f64) / rot)
            if scaling:
                # positions stretched evenly: every frequency divided by the factor
                factor = float(scaling.get("factor") or 0.0)
                if not factor > 0:
                    raise ValueError("position encoding 'rope': linear scaling needs a positive "
                                     "'factor'")
                inv = inv / factor
            pos = torch.arange(ctx.max_positions, dtype=f64).reshape(-1, 1)
        else:
            inv = inverse_frequencies(rot, params["theta"], params.get("scaling"))
            pos = torch.arange(ctx.max_positions, dtype=torch.float32).reshape(-1, 1)
        angles = pos * inv.reshape(1, -1)
        self.rot_dim = rot
        self.inv_freq = inv.to(torch.float32)
        self.cos = (torch.cos(angles) * magnitude).to(torch.float32).to(ctx.device).contiguous()
        self.sin = (torch.sin(angles) * magnitude).to(torch.float32).to(ctx.device).contiguous()
        self.max_positions = ctx.max_positions


@register("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: queries and keys go to the cache as they are."""

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.rot_dim, self.cos, self.sin = 0, None, None
        self.max_positions = ctx.max_positions


def shared_position(spec, ctx: BuildContext) -> PositionEncoding:
    """One table per distinct parameter set, shared by all mixers that name it."""
    from .base import create
    key = ("position", spec.kind, repr(sorted(spec.params.items(), key=lambda kv: kv[0])))
    if key not in ctx.shared:
        ctx.shared[key] = create("position", spec, "", ctx)
    return ctx.shared[key]
