"""Norms over the hidden axis.

RMSNorm: ``y = x * rsqrt(mean(x^2) + eps) * w``; the weight multiplies
directly, not as ``1 + w`` (crates/model/src/layers.rs:103-122, 141-146), unless the model
stores its weights around zero (``weight_offset`` 1: ``y = ... * (1 + w)``).  The input is the
32-bit residual stream; statistics and both multiplies are 32-bit, one rounding at the store.

LayerNorm: ``y = (x - mean) / sqrt(var + eps) * w + b`` with ``var`` the mean squared
deviation from the mean; the same input, the same precision."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import BuildContext, Norm, ResidualStream, TensorSpec, join, register


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    """Parameters: ``size`` (hidden width), ``eps``; optional ``weight_offset`` (a number added
    to the stored weight, in float32, once at build time: 1 for weights stored around zero) and
    ``weight_name`` (the tensor's name under the prefix, "weight" by default; "" when the
    tensor is stored under the prefix itself); ``scalar``: the stored weight is one number that
    multiplies every coordinate (a tensor without axes)."""

    graph_safe = True

    @classmethod
    def _weight_name(cls, params: Dict[str, Any], prefix: str) -> str:
        return join(prefix, params.get("weight_name", "weight"))

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        init = "normal" if float(params.get("weight_offset", 0.0)) else "ones_normal"
        shape = () if params.get("scalar") else (params["size"],)
        return [TensorSpec(cls._weight_name(params, prefix), shape, init=init)]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.eps = float(params["eps"])
        self.weight = ctx.take(self._weight_name(params, prefix))
        if params.get("scalar"):
            # the kernels take one weight per coordinate: the one number, float32, repeated
            self.weight = self.weight.to(torch.float32).reshape(1).expand(
                int(params["size"])).contiguous()
        offset = float(params.get("weight_offset", 0.0))
        if offset:
            self.weight = (self.weight.to(torch.float32) + offset).contiguous()
        self.out_dtype = ctx.act_dtype

    def forward(self, stream: ResidualStream) -> torch.Tensor:
        if stream.lanes is not None:
            return stream.lanes.normed(self.weight, self.eps, self.out_dtype)
        delta, scale = stream.take_delta()
        return ops.add_rmsnorm(stream.x, delta, self.weight, self.eps, self.out_dtype,
                               round_parts=stream.round_parts, delta_scale=scale)

    def forward_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        if stream.lanes is not None:
            return stream.lanes.normed(self.weight, self.eps, self.out_dtype, rows)
        return ops.add_rmsnorm(stream.x, stream.delta(), self.weight, self.eps, self.out_dtype,
                               rows=rows, round_parts=stream.round_parts,
                               delta_scale=stream.pending_scale)

    def fused_linear(self, stream: ResidualStream, w: torch.Tensor, out_dtype: torch.dtype,
                     gated: bool, rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        if self.out_dtype != torch.bfloat16 or stream.lanes is not None:
            return None
        if stream.pending is not None and stream.pending_scale != 1.0:
            if rows is not None:
                return None
            stream.flush()          # the fused forms add a delta as it is
        product = stream.pending
        if isinstance(product, ops.PendingProduct) and rows is None \
                and ops.can_join_norm_linear(product, stream.x, w):
            # The product in front adds itself to the residual and leaves the rows times this
            # norm's weight and their sums of squares; the product behind scales by them.
            xw, ss = ops.linear_join_norm(product, stream.x, self.weight, stream.round_parts)
            stream.pending = None
            return ops.linear_scaled(xw, ss, self.eps, w, out_dtype, gated=gated)
        count = stream.x.shape[0] if rows is None else rows.numel()
        if not ops.can_fuse_norm_linear(stream.x, w, count):
            return None
        y, total = ops.norm_linear(stream.x, stream.delta(), self.weight, self.eps, w, out_dtype,
                                   gated=gated, rows=rows, round_parts=stream.round_parts)
        if rows is None:
            stream.x, stream.pending = total, None
        return y


@register("norm", "layernorm")
class LayerNorm(Norm):
    """Parameters: ``size``, ``eps``; optional ``weight_name`` and ``bias_name`` (the tensors'
    names under the prefix, "weight" and "bias" by default; "" for the prefix itself)."""

    graph_safe = True

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str):
        return (join(prefix, params.get("weight_name", "weight")),
                join(prefix, params.get("bias_name", "bias")))

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        w, b = cls._names(params, prefix)
        return [TensorSpec(w, (params["size"],), init="ones_normal"),
                TensorSpec(b, (params["size"],))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.eps = float(params["eps"])
        w, b = self._names(params, prefix)
        self.weight, self.bias = ctx.take(w), ctx.take(b)
        if self.weight.dtype != self.bias.dtype:
            self.weight, self.bias = (t.to(torch.float32).contiguous()
                                      for t in (self.weight, self.bias))
        self.out_dtype = ctx.act_dtype

    def forward(self, stream: ResidualStream) -> torch.Tensor:
        delta, scale = stream.take_delta()
        return ops.add_layernorm(stream.x, delta, self.weight, self.bias, self.eps,
                                 self.out_dtype, round_parts=stream.round_parts,
                                 delta_scale=scale)

    def forward_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        return ops.add_layernorm(stream.x, stream.delta(), self.weight, self.bias, self.eps,
                                 self.out_dtype, rows=rows, round_parts=stream.round_parts,
                                 delta_scale=stream.pending_scale)
