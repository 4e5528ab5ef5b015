"""Decoder blocks.  The pre-norm block: ``x += mixer(norm(x)); x += feed_forward(norm(x))``
(crates/model/src/llama.rs:264-271).  Which mixer, feed-forward and norms it holds, and under
which weight names, is given by its parameters, layer by layer.  The parallel block:
``x += mixer(h) + feed_forward(h)`` with ``h = norm(x)``, one norm that both sublayers read, or
``x += mixer(norm(x)) + feed_forward(ffn_norm(x))`` with a norm each of the same x.  Behind
either, optionally, the depth mix: the next layer reads a learned weighted sum of the embedding
output and of every layer's result so far."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .base import (Block, BuildContext, CacheBinding, ResidualStream, TensorSpec,
                   create, join, normed, register, tensor_specs)
from .. import ops


@register("block", "prenorm")
class PreNormBlock(Block):
    """Parameters: ``mixer``, ``feed_forward``, ``mixer_norm``, ``ffn_norm`` (PartSpecs) and
    ``names``: the weight-name suffix of each of the four under the block's prefix.  A block
    whose ``feed_forward`` is None has the mixer's sublayer only.  Optional
    ``residual_scale`` m: each sublayer's output joins the stream as ``x += m * f(norm(x))``,
    the product formed in float32 where the sum is."""

    _SLOTS = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"),
              ("feed_forward", "feed_forward"))

    @classmethod
    def _slots(cls, params: Dict[str, Any]):
        if params.get("feed_forward") is None:
            return cls._SLOTS[:2]
        return cls._SLOTS

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for slot, category in cls._slots(params):
            out += tensor_specs(category, params[slot], join(prefix, params["names"][slot]))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        built = {slot: create(category, params[slot], join(prefix, params["names"][slot]), ctx)
                 for slot, category in self._slots(params)}
        self.mixer_norm, self.mixer = built["mixer_norm"], built["mixer"]
        self.ffn_norm, self.feed_forward = built.get("ffn_norm"), built.get("feed_forward")
        self.residual_scale = float(params.get("residual_scale", 1.0))

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer_norm, self.mixer, self.ffn_norm,
                                          self.feed_forward) if p is not None)

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        m = self.residual_scale
        stream.add(self.mixer.forward(normed(self.mixer_norm, stream, self.mixer), step, binding),
                   m)
        if self.feed_forward is not None:
            stream.add(self.feed_forward.forward(
                normed(self.ffn_norm, stream, self.feed_forward), step), m)


@register("block", "hyper")
class HyperBlock(PreNormBlock):
    """The pre-norm block over several residual streams (hyper-connections).  In place of one
    x there are ``streams`` copies x_1 .. x_S, all equal to the block's input stream when the
    first such block meets it.  Sublayer q (1: the mixer, 2: the feed-forward) reads
    ``u = sum_s in_q[s] x_s`` through its norm, and its result y comes back into all streams at
    once, from the old ones: ``x_t <- sum_s mix_q[s, t] x_s + out_q[t] y``.

    Parameters: those of ``prenorm`` (without ``residual_scale``), ``streams`` and ``connections``:
    the tensors' prefixes under the block's prefix, one per sublayer (``("hc1", "hc2")``), each
    with ``.in`` (S), ``.out`` (S) and ``.mix`` (S, S, indexed [from, to]).  ``last``: the block
    leaves one stream behind, the sum of the S, for blocks of another kind behind it (a norm
    behind the last block reads that sum from the streams by itself).  The streams,
    the coefficients and every sum are float32; update and next read run as one kernel."""

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out = super().tensor_specs(params, prefix)
        S = int(params["streams"])
        subs = 1 if params.get("feed_forward") is None else 2
        for name in tuple(params["connections"])[:subs]:
            base = join(prefix, name)
            out += [TensorSpec(base + ".in", (S,), init="ones_normal", std=0.2),
                    TensorSpec(base + ".out", (S,), init="ones_normal", std=0.2),
                    TensorSpec(base + ".mix", (S, S), std=0.4)]
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        if self.residual_scale != 1.0:
            raise ValueError("block 'hyper': the streams' own coefficients scale the results")
        self.streams = int(params["streams"])
        self.last = bool(params.get("last"))
        subs = 1 if self.feed_forward is None else 2
        take = lambda n: ctx.take(n).to(torch.float32).contiguous()
        self.connections = [tuple(take(join(prefix, name) + part) for part in (".in", ".mix", ".out"))
                            for name in tuple(params["connections"])[:subs]]
        for read, mix, back in self.connections:
            if read.numel() != self.streams or back.numel() != self.streams \
                    or tuple(mix.shape) != (self.streams, self.streams):
                raise ValueError(f"block 'hyper': coefficients do not fit {self.streams} streams")

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        lanes = stream.split_lanes(self.streams)
        read, mix, back = self.connections[0]
        lanes.reading(read)
        lanes.update(self.mixer.forward(normed(self.mixer_norm, stream, self.mixer), step, binding),
                     mix, back)
        if self.feed_forward is not None:
            read, mix, back = self.connections[1]
            lanes.reading(read)
            lanes.update(self.feed_forward.forward(
                normed(self.ffn_norm, stream, self.feed_forward), step), mix, back)
        lanes.reading(None)          # whoever reads next without weights reads the plain sum
        if self.last:
            stream.merge_lanes()


@register("block", "parallel")
class ParallelBlock(Block):
    """Parameters: ``mixer``, ``feed_forward`` (None: the mixer alone), ``norm`` (PartSpecs) and
    ``names``: the weight-name suffix of each under the block's prefix.  The two sublayers'
    outputs are added in float32 and join the stream as one delta.  A feed-forward that sets
    ``wants_residual`` also gets the float32 residual rows that the norm normalised and the
    norm itself (``forward(h, step, resid=..., norm=...)``), for decisions that it wants to make
    on the unrounded input."""

    _SLOTS = (("norm", "norm"), ("mixer", "mixer"), ("feed_forward", "feed_forward"),
              ("ffn_norm", "norm"))

    @classmethod
    def _slots(cls, params: Dict[str, Any]):
        if params.get("feed_forward") is None:
            return cls._SLOTS[:2]
        return cls._SLOTS if params.get("ffn_norm") is not None else cls._SLOTS[:3]

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for slot, category in cls._slots(params):
            out += tensor_specs(category, params[slot], join(prefix, params["names"][slot]))
        return out + DepthMix.tensor_specs(params.get("depth_mix"), prefix)

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        built = {slot: create(category, params[slot], join(prefix, params["names"][slot]), ctx)
                 for slot, category in self._slots(params)}
        self.norm, self.mixer = built["norm"], built["mixer"]
        self.feed_forward = built.get("feed_forward")
        self.ffn_norm = built.get("ffn_norm")
        self.depth_mix = DepthMix(params["depth_mix"], prefix, ctx) \
            if params.get("depth_mix") else None

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.norm, self.mixer, self.feed_forward,
                                          self.ffn_norm) if p is not None)

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        h = self.norm.forward(stream)
        mixed = self.mixer.forward(h, step, binding)
        if self.feed_forward is None:
            delta = mixed
        else:
            # (the first norm has folded the pending delta in: stream.x is what both normalise)
            h2 = h if self.ffn_norm is None else self.ffn_norm.forward(stream)
            if getattr(self.feed_forward, "wants_residual", False):
                fed = self.feed_forward.forward(h2, step, resid=stream.x,
                                                norm=self.ffn_norm or self.norm)
            else:
                fed = self.feed_forward.forward(h2, step)
            mixed, fed = (d if isinstance(d, torch.Tensor) else d.run() for d in (mixed, fed))
            delta = ops.weighted_sum(mixed, 1.0, fed, 1.0, round_parts=stream.round_parts)
        if self.depth_mix is None:
            stream.add(delta)
        else:
            self.depth_mix.apply(stream, delta)


class DepthMix:
    """What a block that names ``depth_mix`` does behind its sublayers: the block's result
    ``y = x + delta`` is kept beside the embedding output and the results of the layers before
    it, and the stream becomes ``sum_j w[j] * source_j`` over all of them (source 0 the embedding
    output, source j the result of the j-th such layer), in float32.

    Parameters: ``weight_name`` (the weights' tensor under the block's prefix, one per source:
    ``sources`` of them, the number of layers so far plus one) and ``slots`` (sources the model
    has in all: its layers plus one).  The first such layer (``sources`` 2) makes the history
    for the step and stores its input as source 0."""

    @staticmethod
    def tensor_specs(params: Any, prefix: str) -> List[TensorSpec]:
        if not params:
            return []
        return [TensorSpec(join(prefix, params["weight_name"]), (int(params["sources"]),),
                           init="ones_normal", std=0.3)]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        self.sources, self.slots = int(params["sources"]), int(params["slots"])
        if not 2 <= self.sources <= self.slots:
            raise ValueError(f"depth mix: {self.sources} sources of {self.slots}")
        self.weights = ctx.take(join(prefix, params["weight_name"])).to(torch.float32).contiguous()

    def apply(self, stream: ResidualStream, delta: Any) -> None:
        x = stream.flush()
        if not isinstance(delta, torch.Tensor):
            delta = delta.run()
        if delta.dim() == 3 or delta.dtype != torch.float32:
            delta = ops.weighted_sum(delta, 1.0, None, round_parts=stream.round_parts)
        first = self.sources == 2
        if first:
            stream.history = torch.empty((self.slots, *x.shape), dtype=torch.float32,
                                         device=x.device)
        elif stream.history is None:
            raise ValueError("depth mix: a layer mixes earlier results, but no layer before it "
                             "kept any")
        ops.depth_mix_(x, delta, stream.history, self.sources, self.weights, save_input=first)
