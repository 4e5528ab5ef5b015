"""Mixers that keep a state of fixed size per request, and one that runs two mixers side by
side.

``time_mix`` (RWKV-style): every projection reads its own blend of the token's input and the
previous token's; per head a matrix state S (key channel x value channel) that each token
decays per key channel and writes ``k v^T`` into, read with a bonus for the current token.

``gated_delta``: q, k and v pass a short causal convolution and SiLU, q and k become unit
vectors; per head S decays by one factor, then the token overwrites what its key reads
(``u = beta (v - S^T k)``, ``S += k u^T``) and reads with its query.

Both keep S in float32 in the request's state slot together with the inputs of the last
tokens that the next step's first token needs (one row for the token shift, taps - 1 rows for
the convolution), walk a sequence's tokens in order with whatever else the batch holds, and
leave the state as after the step's last token.  What enters a recurrence (decays, step
sizes, unit norms, the state itself) is float32 in either activation dtype; the projections
that feed it store float32 results.

``selective_scan`` (Mamba): the input passes a short causal convolution and SiLU; a state of N
numbers per channel decays by ``exp(dt A)`` with a step ``dt`` that the token chooses, takes
``dt x B`` and is read with ``C``; the result is gated by ``silu(z)``.

``decay_attention`` (linear attention with a fixed decay per head): q, k and v pass SiLU; per
head ``S <- decay_h S + k v^T`` and the read-out ``S^T q`` includes the token's own key and
value; the heads' read-outs are normalised together, gated by a sigmoid and projected.

``parallel``: two mixers read the same input, and their outputs meet as a weighted sum in
float32.  Each keeps what it keeps: the pages of the one that asks for a cache, the state
bytes of both, one after the other.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import (BuildContext, CacheBinding, CacheRequest, Mixer, NormedInput, PartSpec,
                   TensorSpec, create, join, project, register, tensor_specs)


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


def _state_views(binding: CacheBinding, first: int):
    """The mixer's state area as float32, cut into its first ``first`` floats and the rest."""
    if binding.state is None:
        raise ValueError("this mixer needs a state slot per request; the runner has none")
    st = binding.state.view(torch.float32)
    return st[:, :first], st[:, first:]


def _ran(delta: Any) -> torch.Tensor:
    """A mixer's result as a tensor, whole or as a stack of float32 partial sums; a projection
    that has not run yet runs now."""
    return delta if isinstance(delta, torch.Tensor) else delta.run()


# ------------------------------------------------------------------------------ time mix
@register("mixer", "time_mix")
class TimeMix(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim`` (keys, values and receptances
    share it), ``decay_rank`` (rows of ``w1``), ``eps`` (of the per-head norm of the read-out).

    Tensors under the prefix: ``mu.r|k|v|g|w`` (W) blend weights; ``r``, ``k``, ``v``, ``g``
    (heads * d, W); ``w1`` (rank, W), ``w2`` (heads * d, rank), ``w0`` (heads * d): the decay
    ``exp(-exp(w2 tanh(w1 x_w) + w0))``; ``u`` (heads, d) the bonus; ``norm`` (heads * d);
    ``o`` (W, heads * d)."""

    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, H, d = params["hidden_size"], params["num_heads"], params["head_dim"]
        rank = params["decay_rank"]
        out = [TensorSpec(join(prefix, f"mu.{m}"), (W,), std=0.3) for m in cls.MIXES]
        out += [TensorSpec(join(prefix, n), (H * d, W)) for n in ("r", "k", "v", "g")]
        out += [TensorSpec(join(prefix, "w1"), (rank, W)),
                TensorSpec(join(prefix, "w2"), (H * d, rank)),
                TensorSpec(join(prefix, "w0"), (H * d,)), TensorSpec(join(prefix, "u"), (H, d)),
                TensorSpec(join(prefix, "norm"), (H * d,), init="ones_normal"),
                TensorSpec(join(prefix, "o"), (W, H * d))]
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.width = int(params["hidden_size"])
        self.heads, self.dim = int(params["num_heads"]), int(params["head_dim"])
        self.eps = float(params["eps"])
        take = lambda n: ctx.take(join(prefix, n))
        self.mu = torch.stack([_f32(take(f"mu.{m}")) for m in self.MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = take("r"), take("k"), take("v"), take("g")
        self.w_1, self.w_2 = take("w1"), take("w2")
        self.w0, self.bonus, self.norm = _f32(take("w0")), _f32(take("u")), _f32(take("norm"))
        self.w_o = take("o")
        self.act_dtype = ctx.act_dtype

    def state_bytes(self) -> int:
        return 4 * (self.width + self.heads * self.dim * self.dim)

    def forward(self, x: torch.Tensor, step: Any, binding: CacheBinding) -> Any:
        tail, S = _state_views(binding, self.width)
        cu, slots, n = step.cu_seqlens, step.state_slots, step.num_seqs
        mixes = ops.shift_mix(x, self.mu, tail, step.seq_of_token, cu, slots, n)
        ops.tail_update(tail, x, self.width, 1, cu, slots, n)
        f32 = torch.float32
        r = ops.linear_f32(mixes[0], self.w_r)
        k = ops.linear_f32(mixes[1], self.w_k)
        v = ops.linear_f32(mixes[2], self.w_v)
        gate = ops.linear_f32(mixes[3], self.w_g)
        low = ops.soft_cap_(ops.linear(mixes[4], self.w_1, self.act_dtype), 1.0)     # tanh
        z = ops.linear(low, self.w_2, f32)
        o = ops.decay_scan(r, k, v, z, self.w0, self.bonus, S, cu, slots, n, self.heads, self.dim)
        y = ops.head_norm_gate(o, self.norm, gate, self.heads, self.dim, self.eps, self.act_dtype)
        return ops.pending_linear(y, self.w_o, self.act_dtype)


# --------------------------------------------------------------------------- gated delta
@register("mixer", "gated_delta")
class GatedDelta(Mixer):
    """Parameters: ``hidden_size``, ``num_heads`` (value heads), ``num_kv_heads`` (query/key
    heads; value head h uses head ``h // (heads / kv_heads)``), ``head_dim``, ``value_dim``,
    ``conv`` (taps), ``eps`` (of the per-head norm of the read-out).

    Tensors under the prefix: ``q``, ``k`` (kv_heads * d, W), ``v`` (heads * dv, W), each with
    ``.conv`` (channels, taps); ``b``, ``a`` (heads, W); ``A_log``, ``dt_bias`` (heads);
    ``g`` (heads * dv, W); ``norm`` (dv); ``o`` (W, heads * dv).

    One product makes q, k, v, the gate and the raw step size and decay (rows concatenated, each
    part starting on a multiple of 8 columns), stored in float32."""

    graph_safe = True
    takes_normed_input = True        # the norm in front goes into the one input product where it can
    UNIT_EPS = 1e-6

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, H, G = params["hidden_size"], params["num_heads"], params["num_kv_heads"]
        d, dv, taps = params["head_dim"], params["value_dim"], params["conv"]
        out = []
        for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
            out += [TensorSpec(join(prefix, n), (rows, W)),
                    TensorSpec(join(prefix, f"{n}.conv"), (rows, taps), std=0.3)]
        out += [TensorSpec(join(prefix, "b"), (H, W)), TensorSpec(join(prefix, "A_log"), (H,)),
                TensorSpec(join(prefix, "norm"), (dv,), init="ones_normal"),
                TensorSpec(join(prefix, "a"), (H, W)), TensorSpec(join(prefix, "dt_bias"), (H,)),
                TensorSpec(join(prefix, "g"), (H * dv, W)), TensorSpec(join(prefix, "o"), (W, H * dv))]
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.width = int(params["hidden_size"])
        self.heads, self.kv_heads = int(params["num_heads"]), int(params["num_kv_heads"])
        self.dim, self.vdim = int(params["head_dim"]), int(params["value_dim"])
        self.taps = int(params["conv"])
        self.eps = float(params["eps"])
        if self.heads % self.kv_heads:
            raise ValueError(f"gated_delta: {self.heads} heads are not a multiple of "
                             f"{self.kv_heads} query/key heads")
        if not 1 <= self.taps <= 16:
            raise ValueError(f"gated_delta: {self.taps} taps (1 to 16)")
        take = lambda n: ctx.take(join(prefix, n))
        G, H, d, dv = self.kv_heads, self.heads, self.dim, self.vdim
        self.conv_channels = C = 2 * G * d + H * dv
        parts = [take("q"), take("k"), take("v"), take("g"), take("b"), take("a")]
        if len({p.dtype for p in parts}) > 1:
            parts = [p.to(torch.float32) for p in parts]
        # column ranges of the one product: q | k | v | gate | b | a, each from a multiple of 8
        self.cols: Dict[str, int] = {}
        rows, at = [], 0
        for name, p in zip(("q", "k", "v", "g", "b", "a"), parts):
            if name in ("g", "b", "a"):
                pad = -at % 8
                if pad:
                    rows.append(p.new_zeros((pad, self.width)))
                    at += pad
            self.cols[name] = at
            rows.append(p)
            at += p.shape[0]
        if at % 8:
            rows.append(parts[0].new_zeros((-at % 8, self.width)))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.conv_w = torch.cat([_f32(take(f"{n}.conv")) for n in "qkv"], dim=0).contiguous()
        self.a_log, self.dt_bias = _f32(take("A_log")), _f32(take("dt_bias"))
        self.norm = _f32(take("norm"))
        self.w_o = take("o")
        self.act_dtype = ctx.act_dtype

    def state_bytes(self) -> int:
        return 4 * ((self.taps - 1) * self.conv_channels + self.heads * self.vdim * self.dim)

    def forward(self, x: Any, step: Any, binding: CacheBinding) -> Any:
        G, H, d, dv, C = self.kv_heads, self.heads, self.dim, self.vdim, self.conv_channels
        tail, S = _state_views(binding, (self.taps - 1) * C)
        cu, slots, n = step.cu_seqlens, step.state_slots, step.num_seqs
        if isinstance(x, NormedInput) and not ops.can_fuse_norm_linear(
                x.stream.x, self.w_in, x.stream.x.shape[0]):
            x = x.tensor()
        p = (project(x, self.w_in, torch.float32) if isinstance(x, NormedInput)
             else ops.linear_f32(x, self.w_in))                           # (T, q|k|v|g|b|a)
        qkv = ops.causal_conv(p, self.conv_w, tail, step.seq_of_token, cu, slots, n,
                              unit_channels=2 * G * d, unit_group=d, scaled_channels=G * d,
                              scale=d ** -0.5, unit_eps=self.UNIT_EPS, rest_group=dv)
        ops.tail_update(tail, p, C, self.taps - 1, cu, slots, n)
        c = self.cols
        o = ops.delta_scan(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:],
                           p[:, c["b"]:c["b"] + H], p[:, c["a"]:c["a"] + H], self.a_log,
                           self.dt_bias, S, cu, slots, n, H, G, d, dv)
        y = ops.head_norm_gate(o, self.norm, p[:, c["g"]:c["g"] + H * dv], H, dv, self.eps,
                               self.act_dtype)
        return ops.pending_linear(y, self.w_o, self.act_dtype)


# ------------------------------------------------------------------------ selective scan
@register("mixer", "selective_scan")
class SelectiveScan(Mixer):
    """Parameters: ``hidden_size``, ``inner`` (channels), ``state`` (numbers per channel),
    ``dt_rank``, ``conv`` (taps).

    Tensors under the prefix: ``in`` (2 * inner, W): x in front of z; ``conv`` (inner, taps)
    and ``conv.b`` (inner); ``x`` (dt_rank + 2 * state, inner): the step's low-rank input, B
    and C; ``dt`` (inner, dt_rank) and ``dt.b`` (inner); ``A_log`` (inner, state); ``D``
    (inner); ``o`` (W, inner).

    Per token and channel: ``dt = softplus(W_dt low + dt.b)``, ``S <- exp(dt A) S + dt x B``
    with ``A = -exp(A_log)``, ``y = S . C + D x``, result ``y * silu(z)``.  The state slot holds
    the last ``conv - 1`` inputs of the convolution and S, float32; steps, decays and the state
    are float32 in either activation dtype."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, C, N = params["hidden_size"], params["inner"], params["state"]
        rank, taps = params["dt_rank"], params["conv"]
        return [TensorSpec(join(prefix, "in"), (2 * C, W)),
                TensorSpec(join(prefix, "conv"), (C, taps), std=0.3),
                TensorSpec(join(prefix, "conv.b"), (C,)),
                TensorSpec(join(prefix, "x"), (rank + 2 * N, C)),
                TensorSpec(join(prefix, "dt"), (C, rank), std=0.3),
                TensorSpec(join(prefix, "dt.b"), (C,), std=0.5),
                TensorSpec(join(prefix, "A_log"), (C, N), std=0.5),
                TensorSpec(join(prefix, "D"), (C,), init="ones_normal"),
                TensorSpec(join(prefix, "o"), (W, C))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.channels, self.states = int(params["inner"]), int(params["state"])
        self.rank, self.taps = int(params["dt_rank"]), int(params["conv"])
        if not 1 <= self.taps <= 16:
            raise ValueError(f"selective_scan: {self.taps} taps (1 to 16)")
        take = lambda n: ctx.take(join(prefix, n))
        self.w_in, self.w_x, self.w_dt, self.w_o = take("in"), take("x"), take("dt"), take("o")
        self.conv_w, self.conv_b = _f32(take("conv")), _f32(take("conv.b"))
        self.dt_bias, self.a_log, self.skip = _f32(take("dt.b")), _f32(take("A_log")), _f32(take("D"))
        self.act_dtype = ctx.act_dtype

    def state_bytes(self) -> int:
        return 4 * ((self.taps - 1) * self.channels + self.channels * self.states)

    def forward(self, x: torch.Tensor, step: Any, binding: CacheBinding) -> Any:
        C, N, rank = self.channels, self.states, self.rank
        tail, S = _state_views(binding, (self.taps - 1) * C)
        cu, slots, n = step.cu_seqlens, step.state_slots, step.num_seqs
        xz = ops.linear_f32(x, self.w_in)                                  # (T, x | z)
        xc = ops.causal_conv(xz, self.conv_w, tail, step.seq_of_token, cu, slots, n,
                             bias=self.conv_b, out_dtype=self.act_dtype)
        ops.tail_update(tail, xz, C, self.taps - 1, cu, slots, n)
        low = ops.linear_f32(xc, self.w_x)                                 # (T, dt | B | C)
        dt_raw = ops.linear(low[:, :rank], self.w_dt, torch.float32)
        y = ops.selective_scan(xc, dt_raw, self.dt_bias, low[:, rank:rank + N],
                               low[:, rank + N:rank + 2 * N], xz[:, C:], self.a_log, self.skip,
                               S, cu, slots, n)
        return ops.pending_linear(y, self.w_o, self.act_dtype)


# ----------------------------------------------------------------------- decay attention
@register("mixer", "decay_attention")
class DecayAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim`` (queries and keys),
    ``value_dim``, ``decay`` (one number in (0, 1] per head), ``eps`` (of the norm over the
    concatenated heads).

    Tensors under the prefix: ``q``, ``k`` (heads * d, W), ``v``, ``g`` (heads * dv, W),
    ``norm`` (heads * dv), ``o`` (W, heads * dv).

    Per token: ``q, k, v = silu(W h)``; per head ``S <- decay_h S + k v^T``, ``o = S^T q`` (no
    other scale); the concatenated heads are divided by their root mean square, multiplied by
    ``norm`` and by ``sigmoid(W_g h)``, and projected by ``o``.  One product makes q, k, v and
    the gate (rows concatenated), stored in float32; SiLU, the state (float32, in the request's
    slot, [head][value channel][key channel]), the norm and the gate are float32 in either
    activation dtype."""

    graph_safe = True
    takes_normed_input = True        # the norm in front goes into the one input product where it can

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, H = params["hidden_size"], params["num_heads"]
        d, dv = params["head_dim"], params["value_dim"]
        return [TensorSpec(join(prefix, "q"), (H * d, W)), TensorSpec(join(prefix, "k"), (H * d, W)),
                TensorSpec(join(prefix, "v"), (H * dv, W)), TensorSpec(join(prefix, "g"), (H * dv, W)),
                TensorSpec(join(prefix, "o"), (W, H * dv)),
                TensorSpec(join(prefix, "norm"), (H * dv,), init="ones_normal")]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.width = int(params["hidden_size"])
        self.heads = int(params["num_heads"])
        self.dim, self.vdim = int(params["head_dim"]), int(params["value_dim"])
        self.eps = float(params["eps"])
        decay = [float(x) for x in params["decay"]]
        if len(decay) != self.heads or not all(0.0 < x <= 1.0 for x in decay):
            raise ValueError(f"decay_attention: {self.heads} heads need a decay in (0, 1] each, "
                             f"got {decay}")
        if self.dim > 256:
            raise ValueError(f"decay_attention: heads of {self.dim} key channels (at most 256)")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=ctx.device)
        take = lambda n: ctx.weights.pop(join(prefix, n))
        parts = [take("q"), take("k"), take("v"), take("g")]
        if len({p.dtype for p in parts}) > 1:
            parts = [p.to(torch.float32) for p in parts]
        # column ranges of the one product: q | k | v | gate, each from a multiple of 8
        self.cols: Dict[str, int] = {}
        rows, at = [], 0
        for name, p in zip("qkvg", parts):
            pad = -at % 8
            if pad:
                rows.append(p.new_zeros((pad, self.width)))
                at += pad
            self.cols[name] = at
            rows.append(p)
            at += p.shape[0]
        if at % 8:
            rows.append(parts[0].new_zeros((-at % 8, self.width)))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        del parts, rows
        self.norm = _f32(ctx.take(join(prefix, "norm")))
        self.w_o = ctx.take(join(prefix, "o"))
        self.act_dtype = ctx.act_dtype

    def state_bytes(self) -> int:
        return 4 * self.heads * self.vdim * self.dim

    def forward(self, x: Any, step: Any, binding: CacheBinding) -> Any:
        H, d, dv = self.heads, self.dim, self.vdim
        if binding.state is None:
            raise ValueError("decay_attention needs a state slot per request; the runner has none")
        S = binding.state.view(torch.float32)
        cu, slots, n = step.cu_seqlens, step.state_slots, step.num_seqs
        if isinstance(x, NormedInput) and not ops.can_fuse_norm_linear(
                x.stream.x, self.w_in, x.stream.x.shape[0]):
            x = x.tensor()
        p = (project(x, self.w_in, torch.float32) if isinstance(x, NormedInput)
             else ops.linear_f32(x, self.w_in))                           # (T, q | k | v | gate)
        c = self.cols
        o = ops.decay_attention(p[:, c["q"]:c["q"] + H * d], p[:, c["k"]:c["k"] + H * d],
                                p[:, c["v"]:c["v"] + H * dv], self.decay, S, cu, slots, n,
                                H, d, dv, longest=getattr(step, "max_new", None))
        y = ops.head_norm_gate(o, self.norm, p[:, c["g"]:c["g"] + H * dv], 1, H * dv, self.eps,
                               self.act_dtype, sigmoid_gate=True)
        return ops.pending_linear(y, self.w_o, self.act_dtype)


# ------------------------------------------------------------------------------ parallel
@register("mixer", "parallel")
class ParallelMixers(Mixer):
    """Two mixers on one input: ``scale_a * a(x) + scale_b * b(x)``, the sum in float32.

    Parameters: ``branches``: two dicts ``{"mixer": PartSpec, "name": suffix under the prefix,
    "scale": number}``.  At most one branch may keep pages (the cache request and the step
    planner are that branch's); state bytes are the branches' one after the other."""

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for b in params["branches"]:
            out += tensor_specs("mixer", b["mixer"], join(prefix, b["name"]))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        branches = params["branches"]
        if len(branches) != 2:
            raise ValueError(f"parallel mixer: two branches, got {len(branches)}")
        self.branches: List[Mixer] = [create("mixer", b["mixer"], join(prefix, b["name"]), ctx)
                                      for b in branches]
        self.scales = [float(b["scale"]) for b in branches]
        with_cache = [m for m in self.branches if m.cache_request() is not None]
        if len(with_cache) > 1:
            raise ValueError("parallel mixer: only one branch may keep pages")
        self._cached: Optional[Mixer] = with_cache[0] if with_cache else None
        planners = [m.step_planner() for m in self.branches if m.step_planner() is not None]
        if len(planners) > 1:
            raise ValueError("parallel mixer: only one branch may bring a step planner")
        self._planner = planners[0] if planners else None
        self._offsets, at = [], 0
        for m in self.branches:
            n = int(m.state_bytes())
            self._offsets.append((at, n))
            at += -(-n // 16) * 16
        self._state_bytes = at

    @property
    def graph_safe(self) -> bool:
        return all(m.graph_safe for m in self.branches)

    def cache_request(self) -> Optional[CacheRequest]:
        return self._cached.cache_request() if self._cached is not None else None

    def step_planner(self):
        return self._planner

    def state_bytes(self) -> int:
        return self._state_bytes

    def forward(self, x: torch.Tensor, step: Any, binding: CacheBinding) -> torch.Tensor:
        outs = []
        for m, (at, n) in zip(self.branches, self._offsets):
            own = CacheBinding(counters=binding.counters)
            if m is self._cached:
                own.group, own.pages, own.writes = binding.group, binding.pages, binding.writes
            if n:
                if binding.state is None:
                    raise ValueError("parallel mixer: a branch needs state, the runner has none")
                own.state = binding.state[:, at:at + n]
            outs.append(_ran(m.forward(x, step, own)))
        return ops.weighted_sum(outs[0], self.scales[0], outs[1], self.scales[1],
                                round_parts=x.dtype == torch.bfloat16)
