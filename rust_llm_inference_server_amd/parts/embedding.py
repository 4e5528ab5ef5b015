"""Token embedding and output head.

Embedding: ``x[t] = E[ids[t]]`` with no scaling and no position term
(crates/model/src/llama.rs:256-262), written straight into the 32-bit residual stream.
Head: ``logits = h * W^T`` on the selected rows, ``W`` being the embedding table when the
embeddings are tied (llama.rs:152-156); logits are float32 (llama.rs:285)."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .. import ops
from .base import BuildContext, Embedding, Head, TensorSpec, join, project, register


@register("embedding", "token")
class TokenEmbedding(Embedding):
    """Parameters: ``vocab_size``, ``hidden_size``; optional ``scale`` (the rows are multiplied
    by it as they enter the float32 stream), ``weight_name`` (the table's name under the
    prefix, "weight" by default; "" when it is stored under the prefix itself) and
    ``learned_positions``: ``{"name": full tensor name, "rows": positions}``, a table of
    learned position vectors of which row p is added, unscaled, to the token at position p."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out = [TensorSpec(join(prefix, params.get("weight_name", "weight")),
                          (params["vocab_size"], params["hidden_size"]))]
        learned = params.get("learned_positions")
        if learned:
            out.append(TensorSpec(learned["name"], (learned["rows"], params["hidden_size"])))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.weight = ctx.take(join(prefix, params.get("weight_name", "weight")))
        self.vocab_size = int(params["vocab_size"])
        self.scale = float(params.get("scale", 1.0))
        self.learned = None
        self.position_rows = None          # positions the part can place (None: any)
        learned = params.get("learned_positions")
        if learned:
            self.learned = ctx.take(learned["name"])
            if self.learned.dtype != self.weight.dtype:
                self.learned = self.learned.to(torch.float32).contiguous()
                self.weight = self.weight.to(torch.float32).contiguous()
            self.position_rows = int(self.learned.shape[0])

    def forward(self, ids: torch.Tensor, positions: Any = None) -> torch.Tensor:
        if self.learned is None:
            return ops.embed(ids, self.weight, self.scale)
        if positions is None:
            raise ValueError("embedding: learned position vectors need the tokens' positions")
        return ops.embed(ids, self.weight, self.scale, self.learned, positions)


@register("head", "linear")
class LinearHead(Head):
    """Parameters: ``vocab_size``, ``hidden_size``, ``tied_to`` (name of the tensor to share,
    or None for a weight of its own at ``prefix.weight``; ``weight_name`` names it otherwise,
    "" for the prefix itself); optional ``scale`` (the float32 logits are multiplied by it) and
    ``soft_cap`` c: logits become ``c * tanh(logits / c)``."""

    graph_safe = True

    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        if params.get("tied_to"):
            return []
        return [TensorSpec(join(prefix, params.get("weight_name", "weight")),
                           (params["vocab_size"], params["hidden_size"]))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.weight = ctx.take(params.get("tied_to")
                               or join(prefix, params.get("weight_name", "weight")))
        cap = params.get("soft_cap")
        self.soft_cap = float(cap) if cap else None
        self.scale = float(params.get("scale", 1.0))

    def forward(self, x: Any) -> torch.Tensor:
        logits = project(x, self.weight, torch.float32)
        if self.scale != 1.0:
            ops.scale_(logits, self.scale)
        if self.soft_cap is not None:
            ops.soft_cap_(logits, self.soft_cap)
        return logits
