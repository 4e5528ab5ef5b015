"""Feed-forwards.  SwiGLU: ``down(silu(gate(x)) * up(x))`` with three bias-free projections
(crates/model/src/layers.rs:156-187).  Gate and up run as one product over the row-concatenated
weights; ``silu`` and the product are 32-bit with one rounding."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .. import ops
from .base import BuildContext, FeedForward, TensorSpec, join, project, register


@register("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size``."""

    graph_safe = True

    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        return [TensorSpec(join(prefix, "gate_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "up_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "down_proj.weight"), (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        gate = ctx.weights.pop(join(prefix, "gate_proj.weight"))
        up = ctx.weights.pop(join(prefix, "up_proj.weight"))
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        del gate, up
        self.w_down = ctx.take(join(prefix, "down_proj.weight"))
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        hidden = project(x, self.w_gate_up, self.act_dtype, gated=True)
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)


@register("feed_forward", "mlp")
class DenseMLP(FeedForward):
    """Two bias-free projections around an activation: ``down(act(up(x)))``.

    Parameters: ``hidden_size``, ``intermediate_size``, ``activation`` ("gelu_tanh": 0.5 z (1 +
    tanh(sqrt(2 / pi) (z + 0.044715 z^3))), float32 arithmetic on the stored product),
    ``names`` (the tensors of up and down under the prefix; default ``up_proj.weight`` and
    ``down_proj.weight``)."""

    graph_safe = True
    takes_normed_input = True        # the norm in front goes into the up product where it can

    # activation -> the kernel's name in ops ("gelu_erf": 0.5 z (1 + erf(z / sqrt 2)))
    ACTIVATIONS = {"gelu_tanh": "gelu_tanh", "gelu_erf": "gelu_erf"}

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str) -> Dict[str, str]:
        names = {"up": "up_proj.weight", "down": "down_proj.weight", **(params.get("names") or {})}
        return {k: join(prefix, v) for k, v in names.items()}

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        n = cls._names(params, prefix)
        return [TensorSpec(n["up"], (I, H)), TensorSpec(n["down"], (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        n = self._names(params, prefix)
        self.w_up, self.w_down = ctx.take(n["up"]), ctx.take(n["down"])
        kind = params.get("activation", "gelu_tanh")
        if kind not in self.ACTIVATIONS:
            raise ValueError(f"feed-forward 'mlp': activation '{kind}' is not known "
                             f"(known: {sorted(self.ACTIVATIONS)})")
        self.activation = self.ACTIVATIONS[kind]
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        hidden = getattr(ops, self.activation)(project(x, self.w_up, self.act_dtype))
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)


@register("feed_forward", "clamped_glu")
class ClampedGLU(FeedForward):
    """A gated unit whose branches are bounded before they meet:
    ``down(g * sigmoid(alpha * g) * (u + 1))`` with ``g = min(gate(x), limit)`` and
    ``u = clamp(up(x), -limit, limit)``; three bias-free projections, gate and up as one
    product over the row-concatenated weights.

    Parameters: ``hidden_size``, ``intermediate_size``, ``limit``, ``alpha`` (1.702 by
    default), ``names`` (the tensors of gate, up and down under the prefix; default
    ``gate_proj.weight`` and so on)."""

    graph_safe = True
    takes_normed_input = True        # the norm in front goes into the gate/up product where it can

    _DEFAULT_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight",
                      "down": "down_proj.weight"}

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str) -> Dict[str, str]:
        names = {**cls._DEFAULT_NAMES, **(params.get("names") or {})}
        return {k: join(prefix, v) for k, v in names.items()}

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        n = cls._names(params, prefix)
        return [TensorSpec(n["gate"], (I, H)), TensorSpec(n["up"], (I, H)),
                TensorSpec(n["down"], (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        n = self._names(params, prefix)
        gate, up = ctx.weights.pop(n["gate"]), ctx.weights.pop(n["up"])
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        del gate, up
        self.w_down = ctx.take(n["down"])
        self.limit = float(params["limit"])
        self.alpha = float(params.get("alpha", 1.702))
        if not self.limit > 0:
            raise ValueError(f"feed-forward 'clamped_glu': limit {self.limit} must be positive")
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        gu = project(x, self.w_gate_up, self.act_dtype)
        hidden = ops.clamped_glu(gu, self.limit, self.alpha)
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)


@register("feed_forward", "routed_swiglu")
class RoutedSwiGLU(FeedForward):
    """A mixture of small SwiGLU units of which every token takes ``top``, and optionally a
    shared unit that every token takes.

    Parameters: ``hidden_size``, ``expert_size`` (an expert's inner width), ``experts``,
    ``top``, ``groups`` and ``keep`` (experts stand in ``groups`` equal groups of neighbours;
    only those of the ``keep`` groups with the largest sum of their two best choice scores
    can be chosen), ``scale`` (multiplies the chosen experts' scores, which are not
    renormalised), ``shared_size`` (None: no shared unit).  Optional: ``scores`` ("sigmoid",
    or "softmax" over all experts), ``group_score`` ("top2", or "max": a group's largest
    score), ``renormalise`` (the chosen experts' weights are divided by their sum + 1e-20),
    ``correction`` (False: the router has no correction tensor), ``limit`` and ``alpha`` (with a
    limit the units are of the bounded kind, ``g sigmoid(alpha g) (u + 1)`` with
    ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``).

    Tensors under the prefix: ``router`` (experts, W), ``correction`` (experts: added to the
    sigmoid scores for the choice only), ``e<i>.gate|up`` (F, W), ``e<i>.down`` (W, F),
    ``shared.gate|up|down``.  Router logits, scores and the choice are float32.  A block that
    hands over the float32 residual rows and the layer norm in front (``wants_residual``) lets
    the router decide on the unrounded normalised input: the logits then come from one kernel
    that normalises in float32 itself, and a choice between two close experts does not hang on
    the rounding of the activations that the experts read."""

    graph_safe = True
    wants_residual = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, F, E = params["hidden_size"], params["expert_size"], params["experts"]
        out: List[TensorSpec] = []
        for e in range(E):
            out += [TensorSpec(join(prefix, f"e{e}.gate"), (F, W)),
                    TensorSpec(join(prefix, f"e{e}.up"), (F, W)),
                    TensorSpec(join(prefix, f"e{e}.down"), (W, F))]
        out += [TensorSpec(join(prefix, "router"), (E, W), std=0.5)]
        if params.get("correction", True):
            out += [TensorSpec(join(prefix, "correction"), (E,), std=0.1)]
        S = params.get("shared_size")
        if S:
            out += [TensorSpec(join(prefix, "shared.gate"), (S, W)),
                    TensorSpec(join(prefix, "shared.up"), (S, W)),
                    TensorSpec(join(prefix, "shared.down"), (W, S))]
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        E = self.experts = int(params["experts"])
        self.top, self.groups, self.keep = int(params["top"]), int(params["groups"]), int(params["keep"])
        self.scale = float(params.get("scale", 1.0))
        self.scores = params.get("scores", "sigmoid")
        self.group_score = params.get("group_score", "top2")
        self.renormalise = bool(params.get("renormalise", False))
        self.limit = float(params.get("limit") or 0.0)
        self.alpha = float(params.get("alpha", 1.0))
        if self.scores not in ("sigmoid", "softmax") or self.group_score not in ("top2", "max"):
            raise ValueError(f"routed_swiglu: unknown scores '{self.scores}' or group score "
                             f"'{self.group_score}'")
        if self.limit < 0:
            raise ValueError(f"routed_swiglu: limit {self.limit} must be positive")
        if E % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * (E // self.groups):
            raise ValueError(f"routed_swiglu: {E} experts in {self.groups} groups, {self.keep} "
                             f"kept, {self.top} chosen do not fit")
        pop = lambda n: ctx.weights.pop(join(prefix, n))
        self.act_dtype = ctx.act_dtype
        to = lambda t: t.to(ctx.act_dtype)
        # per expert the gate rows in front of the up rows; all experts in one tensor
        self.w_gate_up = torch.stack([torch.cat([to(pop(f"e{e}.gate")), to(pop(f"e{e}.up"))], dim=0)
                                      for e in range(E)]).contiguous()
        self.w_down = torch.stack([to(pop(f"e{e}.down")) for e in range(E)]).contiguous()
        self.w_router = ctx.take(join(prefix, "router"))
        self.correction = None
        if params.get("correction", True):
            self.correction = ctx.take(join(prefix, "correction")).to(torch.float32).contiguous()
        self.w_shared_gate_up = self.w_shared_down = None
        if params.get("shared_size"):
            gate, up = pop("shared.gate"), pop("shared.up")
            if gate.dtype != up.dtype:
                gate, up = gate.to(torch.float32), up.to(torch.float32)
            self.w_shared_gate_up = torch.cat([gate, up], dim=0).contiguous()
            self.w_shared_down = ctx.take(join(prefix, "shared.down"))

    def forward(self, x: torch.Tensor, step: Any, resid: Any = None, norm: Any = None
                ) -> torch.Tensor:
        weight, bias = getattr(norm, "weight", None), getattr(norm, "bias", None)
        if resid is not None and weight is not None and bias is not None \
                and weight.dtype == bias.dtype == self.w_router.dtype:
            logits = ops.router_logits(resid, weight, bias, norm.eps, self.w_router)
        else:
            logits = ops.linear(x, self.w_router, torch.float32)
        chosen, weights = ops.route(logits, self.correction, self.groups, self.keep, self.top,
                                    self.scale, scores=self.scores, group_score=self.group_score,
                                    renormalise=self.renormalise)
        shared = None
        if self.w_shared_gate_up is not None:
            shared = ops.linear(ops.linear_swiglu(x, self.w_shared_gate_up), self.w_shared_down,
                                self.act_dtype)
        return ops.routed_units(x, self.w_gate_up, self.w_down, chosen, weights, shared,
                                limit=self.limit, alpha=self.alpha)


@register("feed_forward", "routed_mlp")
class RoutedMLP(FeedForward):
    """A mixture of small two-projection units ``down(act(up(x)))`` without gates, of which
    every token takes the ``top`` with the largest router logits; their weights are the softmax
    over the chosen logits alone.

    Parameters: ``hidden_size``, ``expert_size`` (an expert's inner width), ``experts``, ``top``,
    ``activation`` ("relu2": the square of ReLU), ``router_bias`` (the suffix of the bias tensor
    behind the router's name, None: no bias).  Tensors under the prefix: ``router`` (experts, W),
    ``router<suffix>`` (experts), ``e<i>.up`` (F, W), ``e<i>.down`` (W, F).  Router logits, the
    choice and the weights are float32; the logits are the product of the activations as the
    experts read them."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, F, E = params["hidden_size"], params["expert_size"], params["experts"]
        out: List[TensorSpec] = []
        for e in range(E):
            out += [TensorSpec(join(prefix, f"e{e}.up"), (F, W)),
                    TensorSpec(join(prefix, f"e{e}.down"), (W, F))]
        out += [TensorSpec(join(prefix, "router"), (E, W), std=0.5)]
        if params.get("router_bias"):
            out += [TensorSpec(join(prefix, "router") + params["router_bias"], (E,), std=0.1)]
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        E = self.experts = int(params["experts"])
        self.top = int(params["top"])
        if params.get("activation", "relu2") != "relu2":
            raise ValueError(f"routed_mlp: activation '{params['activation']}' is not known "
                             "(known: 'relu2')")
        if not 1 <= self.top <= E:
            raise ValueError(f"routed_mlp: {self.top} chosen of {E} experts")
        self.act_dtype = ctx.act_dtype
        pop = lambda n: ctx.weights.pop(join(prefix, n)).to(ctx.act_dtype)
        up = torch.stack([pop(f"e{e}.up") for e in range(E)])
        down = torch.stack([pop(f"e{e}.down") for e in range(E)])
        if up.shape[1] % 2:
            # the kernels take the inner width in two halves: one more unit that is always zero
            up = torch.cat([up, up.new_zeros((E, 1, up.shape[2]))], dim=1)
            down = torch.cat([down, down.new_zeros((E, down.shape[1], 1))], dim=2)
        self.w_up, self.w_down = up.contiguous(), down.contiguous()
        self.w_router = ctx.take(join(prefix, "router"))
        self.router_bias = None
        if params.get("router_bias"):
            self.router_bias = ctx.take(join(prefix, "router") + params["router_bias"]).to(
                torch.float32).contiguous()

    def forward(self, x: torch.Tensor, step: Any) -> torch.Tensor:
        logits = ops.linear(x, self.w_router, torch.float32)
        # softmax over all experts, renormalised over the chosen: the softmax over the chosen
        chosen, weights = ops.route(logits, None, 1, 1, self.top, 1.0, scores="softmax",
                                    group_score="max", renormalise=True, bias=self.router_bias)
        return ops.routed_units(x, self.w_up, self.w_down, chosen, weights, plain=True)
