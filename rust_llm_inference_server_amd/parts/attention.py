"""Grouped-query attention over the paged cache.

As the reference's ``Attention::forward`` (crates/model/src/attention.rs:61-103): three
bias-free projections (here fused into one product over the row-concatenated weights), heads
split column-wise (column ``h * d + j`` is head ``h``, dim ``j``), rotation of q and k by
absolute position, K and V of the new tokens written to the cache before attention reads them
(crates/model/src/paged.rs:324-337), query head ``h`` using KV head ``h / group``
(attention.rs:166-171), scores scaled by ``scale``, float32 softmax, heads merged head-major,
output projection."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import (BuildContext, CacheBinding, CacheRequest, Mixer, NormedInput, PartSpec,
                   TensorSpec, join, project, register)
from .rope import shared_position


@register("mixer", "attention")
class PagedAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``scale``,
    ``window`` (None: all earlier positions), ``position`` (a PartSpec); optional ``value_dim``
    (size of a value head when it differs from ``head_dim``, the size of a query and key head)
    and ``names`` (the tensors of q, k, v and o under the prefix; default ``q_proj.weight`` and
    so on).  Further options, none of which the reference's Llama has:

    * ``conv`` (taps K): a short causal convolution over time on every channel of q, k and v,
      directly behind the projection and in front of the rotation, no bias, no activation:
      ``y_t = sum_j w[:, j] u_(t - K + 1 + j)`` with zeros in front of the sequence; tensors
      ``<q|k|v name>.conv`` (channels, K).  The last K - 1 projected rows of a request live in
      its state slot (float32); the products' results are float32 and the convolution is
      float32 arithmetic.
    * ``head_scales``: the name (under the prefix) of a tensor with one number per query head
      that multiplies the head's scores on top of ``scale``.
    * ``softcap`` c: the scaled score becomes ``c tanh(score / c)`` in front of the softmax.
    * ``value_mix``: ``{"name": tensor under the prefix, "key": a name, "source": bool}``.
      The source layer hands its values (behind the convolution) on to the later layers of the
      step under ``key``; every other layer with that key replaces its values by
      ``(1 - w) v + w v_source`` (``w`` the tensor's one number) before they are cached.
    * ``bias``: a suffix; the q, k and v projections add the tensors ``<q|k|v name><suffix>``
      (one number per output column, float32 arithmetic on the stored product).
    * ``qk_norm``: ``{"q": name, "k": name, "eps": e}``.  Every query head and every key head is
      divided by the root mean square of its own numbers (eps inside the root) and multiplied by
      the named weight of ``head_dim`` numbers, which all heads share, behind the bias and in
      front of the rotation; the cache holds the normalised keys.
    * ``query_temperature``: ``{"coef": c, "every": n}``.  The queries of a token at position p
      are multiplied by ``1 + c ln(floor((p + 1) / n) + 1)`` (behind the norm).
    * ``sinks``: the name of a tensor with one number per query head: the softmax's denominator
      also holds ``e^sink``, once, unscaled, with no key and no value behind it.
    * ``keep_first`` n (with a ``window``): the first n keys of a sequence stay visible to every
      later query beside the window's keys, at their own positions; the cache keeps their pages
      while it gives back those that the window has passed.
    * ``gate``: the name of a projection ``(num_heads, hidden_size)`` of the mixer's input: head
      h of the result is multiplied by the sigmoid of output h, in front of the output
      projection.
    * ``cache_like``: ``{"window": w or None, "keep_first": n}``: what the cache keeps for this
      layer's pages when that is more than the layer's own mask sees (a layer whose pages another
      layer with a wider mask reads, and that reader itself: both name the wider of the two).
    * ``shared_kv``: the layer has no key and value projections (nor what belongs to them:
      biases, the keys' norm); its run reads the cache that another run wrote.

    With ``value_dim != head_dim`` (or an odd head size) the kernels run at one head size ``D``,
    the larger of the two rounded up to a multiple of 16: the rows of the narrower projection's weight are padded
    with zero rows per head at build time (and the output projection's columns with zero
    columns), so the extra query and key dims add exact zeros to every score and the extra
    value dims come out as exact zeros that meet zero columns.  The kernels stay specialised on
    one head size; the price is that the narrower of keys and values is cached at ``D``.

    What the position part may carry: ``rot_dim``, ``cos``, ``sin`` (float32 tables, a rotation
    of the first ``rot_dim`` dims of every q and k head; rot_dim 0: none), ``interleaved``
    (the rotation pairs dim 2j with 2j + 1 instead of j with j + rot/2), ``bias_slopes``
    (float32, one per query head: slope * (key position - query position) is added to the
    scores).  The reference's Llama uses the first three (crates/model/src/rope.rs:61-117)."""

    graph_safe = True
    takes_normed_input = True

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str) -> Dict[str, str]:
        names = {**{n: f"{n}_proj.weight" for n in "qkvo"}, **(params.get("names") or {})}
        return {k: join(prefix, v) for k, v in names.items()}

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, nh, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads",
                                             "head_dim"))
        dv = params.get("value_dim") or d
        n = cls._names(params, prefix)
        own_kv = not params.get("shared_kv")
        out = [TensorSpec(n["q"], (nh * d, H))]
        if own_kv:
            out += [TensorSpec(n["k"], (nkv * d, H)), TensorSpec(n["v"], (nkv * dv, H))]
        out.append(TensorSpec(n["o"], (H, nh * dv)))
        if params.get("bias"):
            out += [TensorSpec(n[c] + params["bias"], (rows,), std=0.1) for c, rows in
                    (("q", nh * d), ("k", nkv * d), ("v", nkv * dv)) if c == "q" or own_kv]
        norm = params.get("qk_norm")
        if norm:
            out += [TensorSpec(join(prefix, norm[c]), (d,), init="ones_normal", std=0.1)
                    for c in "qk" if c == "q" or own_kv]
        if params.get("sinks"):
            out.append(TensorSpec(join(prefix, params["sinks"]), (nh,), std=1.0))
        if params.get("gate"):
            out.append(TensorSpec(join(prefix, params["gate"]), (nh, H), std=0.1))
        taps = params.get("conv")
        if taps:
            out += [TensorSpec(n[c] + ".conv", (rows, int(taps)), std=0.3)
                    for c, rows in (("q", nh * d), ("k", nkv * d), ("v", nkv * dv))]
        if params.get("head_scales"):
            out.append(TensorSpec(join(prefix, params["head_scales"]), (nh,), init="ones_normal",
                                  std=0.2))
        if params.get("value_mix"):
            out.append(TensorSpec(join(prefix, params["value_mix"]["name"]), (), std=0.3))
        return out

    @staticmethod
    def _pad_heads(w: torch.Tensor, heads: int, size: int, to: int, rows: bool) -> torch.Tensor:
        """A projection whose heads of ``size`` lie along its rows (or columns) with every head
        padded to ``to`` by zeros."""
        if size == to:
            return w
        if rows:
            out = w.new_zeros((heads, to, w.shape[1]))
            out[:, :size] = w.reshape(heads, size, w.shape[1])
            return out.reshape(heads * to, w.shape[1])
        out = w.new_zeros((w.shape[0], heads, to))
        out[:, :, :size] = w.reshape(w.shape[0], heads, size)
        return out.reshape(w.shape[0], heads * to)

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        qk_dim = int(params["head_dim"])
        v_dim = int(params.get("value_dim") or qk_dim)
        # the one head size the kernels run at
        # (equal sizes stay as they are when the kernels take them: even head sizes)
        self.head_dim = qk_dim if v_dim == qk_dim and qk_dim % 2 == 0 \
            else -(-max(qk_dim, v_dim) // 16) * 16
        self.v_dim = v_dim
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"attention: {self.num_heads} heads are not a multiple of "
                             f"{self.num_kv_heads} KV heads")
        names = self._names(params, prefix)
        self.shared_kv = bool(params.get("shared_kv"))
        self.qk_dim = qk_dim
        # (heads, real size) of the projections this layer has, in the order of the row
        kinds = [("q", self.num_heads, qk_dim)]
        if not self.shared_kv:
            kinds += [("k", self.num_kv_heads, qk_dim), ("v", self.num_kv_heads, v_dim)]
        mats = [ctx.weights.pop(names[c]) for c, _, _ in kinds]
        gate = ctx.weights.pop(join(prefix, params["gate"])) if params.get("gate") else None
        if len({t.dtype for t in mats + ([gate] if gate is not None else [])}) > 1:
            mats = [t.to(torch.float32) for t in mats]
            gate = None if gate is None else gate.to(torch.float32)
        mats = [self._pad_heads(t, heads, size, self.head_dim, rows=True)
                for t, (_, heads, size) in zip(mats, kinds)]
        # the columns of q, k and v in the product's rows
        self.qkv_cols = sum(t.shape[0] for t in mats)
        self.gated = gate is not None
        if gate is not None:
            # the gates' rows ride behind v, padded so that rows stay 16-byte aligned
            pad = -gate.shape[0] % 8
            mats.append(torch.cat([gate, gate.new_zeros((pad, gate.shape[1]))], dim=0))
        # One product for q, k and v (and the gates): the rows of the weights, concatenated.
        self.w_qkv = torch.cat(mats, dim=0).contiguous()
        del mats, gate
        self.bias = None
        if params.get("bias"):
            self.bias = torch.cat([
                self._pad_heads(ctx.take(names[c] + params["bias"]).to(torch.float32).reshape(-1, 1),
                                heads, size, self.head_dim, rows=True).reshape(-1)
                for c, heads, size in kinds]).contiguous()
        self.q_norm = self.k_norm = None
        self.norm_eps = 0.0
        norm = params.get("qk_norm")
        if norm:
            self.norm_eps = float(norm["eps"])
            self.q_norm = ctx.take(join(prefix, norm["q"])).to(torch.float32).contiguous()
            if not self.shared_kv:
                self.k_norm = ctx.take(join(prefix, norm["k"])).to(torch.float32).contiguous()
        temp = params.get("query_temperature") or {}
        self.temp_coef, self.temp_every = float(temp.get("coef", 0.0)), int(temp.get("every", 0))
        self.sinks = None
        if params.get("sinks"):
            self.sinks = ctx.take(join(prefix, params["sinks"])).to(torch.float32).contiguous()
        self.keep_first = int(params.get("keep_first") or 0)
        like = params.get("cache_like")
        self.cache_like = None if like is None else (like.get("window"),
                                                     int(like.get("keep_first") or 0))
        self.w_o = self._pad_heads(ctx.take(names["o"]), self.num_heads, v_dim, self.head_dim,
                                   rows=False).contiguous()
        self.act_dtype = ctx.act_dtype
        self.position = shared_position(params.get("position") or PartSpec("none"), ctx)
        if self.position.rot_dim > qk_dim:
            raise ValueError("attention: the rotated width exceeds the head size")

        D, nh, nkv = self.head_dim, self.num_heads, self.num_kv_heads
        self.taps = int(params.get("conv") or 0)
        self.conv_w = None
        if self.taps:
            if not 1 <= self.taps <= 16:
                raise ValueError(f"attention: {self.taps} taps (1 to 16)")
            # the taps of every channel of the one product, padded channels with zero taps
            if self.shared_kv or self.gated:
                raise ValueError("attention: the convolutions are built for layers with q, k and "
                                 "v projections of their own and no gate")
            pads = ((names["q"], nh, qk_dim), (names["k"], nkv, qk_dim), (names["v"], nkv, v_dim))
            self.conv_w = torch.cat([
                self._pad_heads(ctx.take(n + ".conv").to(torch.float32), heads, size, D, rows=True)
                for n, heads, size in pads], dim=0).contiguous()
        self.head_scales = None
        if params.get("head_scales"):
            self.head_scales = ctx.take(join(prefix, params["head_scales"])).to(
                torch.float32).contiguous()
        self.softcap = float(params.get("softcap") or 0.0)
        if self.softcap < 0:
            raise ValueError(f"attention: softcap {self.softcap} must be positive")
        mix = params.get("value_mix")
        self.mix_key = self.mix_source = None
        self.mix_weight = 0.0
        if mix:
            self.mix_key, self.mix_source = str(mix["key"]), bool(mix["source"])
            # (one number, read once while the model is built)
            self.mix_weight = float(ctx.take(join(prefix, mix["name"])).to(torch.float32).item())

        self.planner = ops.attention_planner(
            self.num_heads, self.num_kv_heads, self.head_dim, self.act_dtype,
            biased=getattr(self.position, "bias_slopes", None) is not None,
            shaped=self.head_scales is not None or self.softcap > 0,
            plain=self.sinks is not None or bool(self.keep_first and self.window))

    def cache_request(self) -> CacheRequest:
        if self.cache_like is not None:
            return CacheRequest.kv(self.num_kv_heads, self.head_dim, *self.cache_like)
        return CacheRequest.kv(self.num_kv_heads, self.head_dim, self.window, self.keep_first)

    def step_planner(self):
        return self.planner

    def state_bytes(self) -> int:
        """The last ``taps - 1`` rows of the q, k, v product, float32."""
        if self.taps <= 1:
            return 0
        return 4 * (self.taps - 1) * self.w_qkv.shape[0]

    def _project(self, x: Any, step: Any, binding: CacheBinding) -> torch.Tensor:
        """q, k and v of the step's tokens ``(T, (nh + 2 nkv) D)`` in the activation dtype:
        the product, and behind it the convolution and the mix of the values where the layer
        has them."""
        if not self.taps:
            qkv = project(x, self.w_qkv, self.act_dtype)
            if self.bias is not None or self.q_norm is not None or self.temp_every:
                ops.head_prepare_(qkv, self.num_heads, 0 if self.shared_kv else self.num_kv_heads,
                                  self.head_dim, self.qk_dim, self.bias, self.q_norm, self.k_norm,
                                  self.norm_eps, step.positions, self.temp_coef, self.temp_every)
        else:
            C = self.w_qkv.shape[0]
            if isinstance(x, NormedInput) and not ops.can_fuse_norm_linear(
                    x.stream.x, self.w_qkv, x.stream.x.shape[0]):
                x = x.tensor()
            p = (project(x, self.w_qkv, torch.float32) if isinstance(x, NormedInput)
                 else ops.linear_f32(x, self.w_qkv))
            if self.taps > 1 and binding.state is None:
                raise ValueError("attention with a convolution needs a state slot per request; "
                                 "the runner has none")
            tail = binding.state.view(torch.float32) if self.taps > 1 else p.new_zeros((1, 1))
            cu, slots, n = step.cu_seqlens, step.state_slots, step.num_seqs
            blend = None
            if self.mix_key is not None and not self.mix_source:
                handed = step.carried.get(self.mix_key)
                if handed is None:
                    raise ValueError(f"attention: no earlier layer of the step handed on values "
                                     f"under '{self.mix_key}'")
                blend, heads, size, padded = handed
                if (heads, size) != (self.num_kv_heads, self.v_dim):
                    raise ValueError(f"attention: values of {heads} heads of {size} cannot be "
                                     f"mixed into {self.num_kv_heads} heads of {self.v_dim}")
                if padded != self.head_dim:      # the two layers pad their heads differently
                    wide = blend.new_zeros((blend.shape[0], heads, self.head_dim))
                    wide[:, :, :size] = blend.reshape(-1, heads, padded)[:, :, :size]
                    blend = wide.reshape(blend.shape[0], heads * self.head_dim)
            v_from = (self.num_heads + self.num_kv_heads) * self.head_dim
            qkv = ops.causal_conv(p, self.conv_w, tail, step.seq_of_token, cu, slots, n,
                                  out_dtype=self.act_dtype, activation=False, blend=blend,
                                  blend_from=v_from, blend_weight=self.mix_weight)
            if self.taps > 1:
                ops.tail_update(tail, p, C, self.taps - 1, cu, slots, n)
            if self.mix_source:
                step.carried[self.mix_key] = (qkv[:, v_from:], self.num_kv_heads, self.v_dim,
                                              self.head_dim)
            return qkv
        if self.mix_key is not None:
            raise ValueError("attention: mixing values across layers is built behind the "
                             "convolution only")
        return qkv

    def forward(self, x: Any, step: Any, binding: CacheBinding) -> torch.Tensor:
        group = step.groups[binding.group]
        if self.shared_kv and binding.writes:
            raise ValueError("attention: a layer without keys and values of its own must read "
                             "another run's cache")
        rows = self._project(x, step, binding)
        qkv = rows[:, :self.qkv_cols] if self.gated else rows
        if step.max_context > self.position.max_positions:
            raise ValueError(f"sequence of {step.max_context} positions exceeds max_seq_len "
                             f"{self.position.max_positions}")
        out = ops.rope_attention(qkv, self.num_heads, self.num_kv_heads, self.head_dim,
                                 self.position.cos, self.position.sin, step.positions,
                                 group.slots, binding.k_pages, binding.v_pages, group.page_size,
                                 group.block_tables, step, self.scale, self.window,
                                 write_kv=binding.writes and not self.shared_kv,
                                 plan=step.plans.get(self.planner.key()),
                                 interleaved=bool(getattr(self.position, "interleaved", False)),
                                 bias_slopes=getattr(self.position, "bias_slopes", None),
                                 counters=binding.counters, head_scales=self.head_scales,
                                 softcap=self.softcap, sinks=self.sinks,
                                 keep_first=self.keep_first)
        if self.gated:
            ops.head_gate_(out, rows[:, self.qkv_cols:], self.num_heads, self.head_dim)
        return ops.pending_linear(out, self.w_o, self.act_dtype)
